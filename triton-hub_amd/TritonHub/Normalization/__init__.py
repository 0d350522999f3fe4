from .layernorm import LayerNorm
from .rmsnorm import RMSNorm

__all__ = ['LayerNorm', 'RMSNorm']
