"""Sigmoid: drop-in for ``TritonHub/Activations/sigmoid.py`` of the reference (the ``sigmoid`` autograd Function,
sigmoid.py:81-92, and the ``Sigmoid`` callable, :94-98).  The Function saves its OUTPUT."""
import torch

from .. import _native
from ._launch import act_bwd, act_fwd


class sigmoid(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input):
        output = act_fwd(input, _native.ACT_SIGMOID)
        ctx.save_for_backward(output)
        return output

    @staticmethod
    def backward(ctx, d_out):
        output, = ctx.saved_tensors
        return act_bwd(output, d_out, _native.ACT_SIGMOID)


class Sigmoid:
    def __init__(self):
        self.sigmoid_fn = sigmoid.apply

    def __call__(self, x):
        return self.sigmoid_fn(x)
