from .normalize import normalize
from .norm import norm

__all__ = ['normalize', 'norm']
