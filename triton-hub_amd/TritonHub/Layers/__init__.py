"""``Dropout`` of the reference's ``TritonHub.Layers`` package, on a HIP kernel for gfx950.  The package's ``Linear``
and ``MLP`` (matrix products, Layers/linear.py and mlp.py of the reference) are not part of this library."""
from .dropout import Dropout

__all__ = ['Dropout']
