"""``LayerNorm`` and ``RMSNorm`` of the reference's ``TritonHub.Normalization`` package, on HIP kernels for gfx950.
``TritonHub.Normalization.fused`` adds the same two modules with an activation applied in the same pass."""
from .layernorm import LayerNorm
from .rmsnorm import RMSNorm

__all__ = ['LayerNorm', 'RMSNorm']
