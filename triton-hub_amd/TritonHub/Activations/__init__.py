"""Activations of the reference's ``TritonHub.Activations`` package, on HIP kernels for gfx950.

Row reductions over the last dimension (``Softmax``, ``Softmin``, ``LogSoftmax``) run on the row engine of the norm
kernels; the ten element-wise activations are one streaming kernel each way.  The public names and their order are
the reference's (TritonHub/Activations/__init__.py:15).
"""
# row reductions
from .logsoftmax import LogSoftmax
from .softmax import Softmax
from .softmin import Softmin
# element-wise, parameter free
from .gelu import GeLU
from .mish import Mish
from .relu import ReLU
from .relu6 import ReLU6
from .sigmoid import Sigmoid
from .silu import SiLU
from .tanh import Tanh
# element-wise, with parameters
from .leaky_relu import LeakyReLU
from .softplus import Softplus
from .threshold import Threshold

__all__ = ['GeLU', 'SiLU', 'ReLU', 'LeakyReLU', 'Softmax', 'Softplus', 'Tanh', 'Softmin', 'Sigmoid', 'Mish', 'ReLU6',
           'Threshold', 'LogSoftmax']
