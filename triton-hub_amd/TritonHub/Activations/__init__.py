from .gelu import GeLU
from .silu import SiLU
from .relu import ReLU
from .leaky_relu import LeakyReLU
from .softmax import Softmax
from .softplus import Softplus
from .tanh import Tanh
from .softmin import Softmin
from .sigmoid import Sigmoid
from .mish import Mish
from .relu6 import ReLU6
from .threshold import Threshold
from .logsoftmax import LogSoftmax

__all__ = ['GeLU', 'SiLU', 'ReLU', 'LeakyReLU', 'Softmax', 'Softplus', 'Tanh', 'Softmin', 'Sigmoid', 'Mish', 'ReLU6',
           'Threshold', 'LogSoftmax']
