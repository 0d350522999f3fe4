"""Threshold: drop-in for ``TritonHub/Activations/threshold.py`` of the reference (the ``threshold_fn`` autograd
Function, threshold.py:85-100, and the ``Threshold`` callable, :102-108)."""
import torch

from .. import _native
from ._launch import act_bwd, act_fwd


class threshold_fn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, threshold, value):
        output = act_fwd(input, _native.ACT_THRESHOLD, threshold, value)
        ctx.save_for_backward(input)
        ctx.threshold = threshold
        ctx.value = value
        return output

    @staticmethod
    def backward(ctx, d_out):
        input, = ctx.saved_tensors
        grad = act_bwd(input, d_out, _native.ACT_THRESHOLD, ctx.threshold, ctx.value)
        return grad, None, None


class Threshold:
    def __init__(self, threshold, value):
        self.threshold_fn = threshold_fn.apply
        self.threshold = threshold
        self.value = value

    def __call__(self, x):
        return self.threshold_fn(x, self.threshold, self.value)
