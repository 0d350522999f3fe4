"""MI355X-native drop-in for the ``TritonHub.Normalization`` package of AliYoussef97/Triton-Hub.

The LayerNorm / RMSNorm path and, next to it, the row-reduction activations Softmax / Softmin / LogSoftmax and
the row p-norm / normalize operators and ``Layers.Dropout`` exist here; the device code is hand-written HIP for gfx950 behind the C ABI declared in
``include/thnorm.h`` (``libthnorm.so``).  Import surface mirrors the reference's ``TritonHub/__init__.py:1-10``
for those sub-packages.
"""
__version__ = '1.1.1'

from . import Activations, Layers, Normalization, Ops

__all__ = ['Activations', 'Layers', 'Normalization', 'Ops']
