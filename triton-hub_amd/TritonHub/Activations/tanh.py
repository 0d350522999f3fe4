"""Tanh: drop-in for ``TritonHub/Activations/tanh.py`` of the reference (the ``tanh`` autograd Function,
tanh.py:83-94, and the ``Tanh`` callable, :96-100).  The Function saves its OUTPUT."""
import torch

from .. import _native
from ._launch import act_bwd, act_fwd


class tanh(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input):
        output = act_fwd(input, _native.ACT_TANH)
        ctx.save_for_backward(output)
        return output

    @staticmethod
    def backward(ctx, d_out):
        output, = ctx.saved_tensors
        return act_bwd(output, d_out, _native.ACT_TANH)


class Tanh:
    def __init__(self):
        self.tanh_fn = tanh.apply

    def __call__(self, x):
        return self.tanh_fn(x)
