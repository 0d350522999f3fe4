"""Mish: drop-in for ``TritonHub/Activations/mish.py`` of the reference (the ``mish`` autograd Function,
mish.py:91-102, and the ``Mish`` callable, :104-108).  The Function saves its input."""
import torch

from .. import _native
from ._launch import act_bwd, act_fwd


class mish(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input):
        output = act_fwd(input, _native.ACT_MISH)
        ctx.save_for_backward(input)
        return output

    @staticmethod
    def backward(ctx, d_out):
        input, = ctx.saved_tensors
        return act_bwd(input, d_out, _native.ACT_MISH)


class Mish:
    def __init__(self):
        self.mish_fn = mish.apply

    def __call__(self, x):
        return self.mish_fn(x)
