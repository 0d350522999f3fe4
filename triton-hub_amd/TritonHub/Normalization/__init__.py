"""``LayerNorm`` and ``RMSNorm`` of the reference's ``TritonHub.Normalization`` package, on HIP kernels for gfx950.
``TritonHub.Normalization.fused`` adds the same two modules with an activation applied in the same pass."""
from ._launch import get_cache_policy, set_cache_policy  # noqa: F401  (not in __all__: the reference has no such knob)
from .layernorm import LayerNorm
from .rmsnorm import RMSNorm

__all__ = ['LayerNorm', 'RMSNorm']
