"""Softplus: drop-in for ``TritonHub/Activations/softplus.py`` of the reference (the ``softplus`` autograd
Function, softplus.py:89-102, and the ``Softplus`` callable, :104-110)."""
import torch

from .. import _native
from ._launch import act_bwd, act_fwd


class softplus(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, beta, threshold):
        output = act_fwd(input, _native.ACT_SOFTPLUS, beta, threshold)
        ctx.save_for_backward(input)
        ctx.beta = beta
        ctx.threshold = threshold
        return output

    @staticmethod
    def backward(ctx, d_out):
        input, = ctx.saved_tensors
        grad = act_bwd(input, d_out, _native.ACT_SOFTPLUS, ctx.beta, ctx.threshold)
        return grad, None, None


class Softplus:
    def __init__(self, beta=1.0, threshold=20):
        self.beta = beta
        self.threshold = threshold
        self.softplus_fn = softplus.apply

    def __call__(self, x):
        return self.softplus_fn(x, self.beta, self.threshold)
