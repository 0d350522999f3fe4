"""Softmax over the last dimension: drop-in for ``TritonHub/Activations/softmax.py`` of the reference
(the ``softmax`` autograd Function, softmax.py:86-97, and the ``Softmax`` callable, :99-103)."""
import torch

from .. import _native
from ._launch import softmax_bwd, softmax_fwd


class softmax(torch.autograd.Function):
    """forward(ctx, input) -> softmax(input, dim=-1); saves the OUTPUT; backward: y*dy - y*sum(y*dy)."""

    @staticmethod
    def forward(ctx, input):
        output = softmax_fwd(input, _native.SOFTMAX)
        ctx.save_for_backward(output)
        return output

    @staticmethod
    def backward(ctx, d_out):
        output, = ctx.saved_tensors
        return softmax_bwd(output, d_out, _native.SOFTMAX)


class Softmax:
    def __init__(self):
        self.softmax_fn = softmax.apply

    def __call__(self, x):
        return self.softmax_fn(x)
