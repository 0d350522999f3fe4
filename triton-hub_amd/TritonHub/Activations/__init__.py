from .softmax import Softmax
from .softmin import Softmin
from .logsoftmax import LogSoftmax

__all__ = ['Softmax', 'Softmin', 'LogSoftmax']
