"""Softmin over the last dimension: drop-in for ``TritonHub/Activations/softmin.py`` of the reference.

In the reference the ``softmin`` autograd Function is a softmax of ITS input (softmin.py:11-24, :86-97) and the
``Softmin`` callable negates first: ``self.softmin_fn(-x)`` (softmin.py:103).  Both are kept: ``softmin.apply(z)``
is softmax(z), ``Softmin()(x)`` is softmax(-x).  The callable does not spend a pass of its own on the
negation: it calls a second Function whose kernels negate on load (forward) and on store (backward), which
gives the same values and gradients as negating with a tensor op.
"""
import torch

from .. import _native
from ._launch import softmax_bwd, softmax_fwd


class softmin(torch.autograd.Function):
    """forward(ctx, input) -> softmax(input, dim=-1), exactly as in the reference; saves the output."""

    @staticmethod
    def forward(ctx, input):
        output = softmax_fwd(input, _native.SOFTMAX)
        ctx.save_for_backward(output)
        return output

    @staticmethod
    def backward(ctx, d_out):
        output, = ctx.saved_tensors
        return softmax_bwd(output, d_out, _native.SOFTMAX)


class _softmin_of(torch.autograd.Function):
    """forward(ctx, x) -> softmax(-x, dim=-1) in one pass; backward returns d/dx, sign included."""

    @staticmethod
    def forward(ctx, input):
        output = softmax_fwd(input, _native.SOFTMIN)
        ctx.save_for_backward(output)
        return output

    @staticmethod
    def backward(ctx, d_out):
        output, = ctx.saved_tensors
        return softmax_bwd(output, d_out, _native.SOFTMIN)


class Softmin:
    def __init__(self):
        self.softmin_fn = softmin.apply

    def __call__(self, x):
        return _softmin_of.apply(x)          # == self.softmin_fn(-x), without the extra pass
