"""MI355X-native drop-in for the ``TritonHub.Normalization`` package of AliYoussef97/Triton-Hub.

Only the LayerNorm / RMSNorm path exists here; the device code is hand-written HIP for gfx950 behind the
C ABI declared in ``include/thnorm.h`` (``libthnorm.so``).  Import surface mirrors the reference's
``TritonHub/__init__.py:1-10`` for that one sub-package.
"""
__version__ = '1.1.1'

from . import Normalization

__all__ = ['Normalization']
