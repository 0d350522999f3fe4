"""Row p-norm (``norm``) and p-normalisation (``normalize``) of the reference's ``TritonHub.Ops`` package, on HIP
kernels for gfx950.  (``bmm`` of the reference is a GEMM and is not part of this library.)"""
from .norm import norm
from .normalize import normalize

__all__ = ['normalize', 'norm']
