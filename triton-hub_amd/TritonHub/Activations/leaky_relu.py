"""LeakyReLU: drop-in for ``TritonHub/Activations/leaky_relu.py`` of the reference (the ``leakyrelu`` autograd
Function, leaky_relu.py:85-97, and the ``LeakyReLU`` callable, :99-104)."""
import torch

from .. import _native
from ._launch import act_bwd, act_fwd


class leakyrelu(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, negative_slope):
        output = act_fwd(input, _native.ACT_LEAKY_RELU, negative_slope)
        ctx.save_for_backward(input)
        ctx.negative_slope = negative_slope
        return output

    @staticmethod
    def backward(ctx, d_out):
        input, = ctx.saved_tensors
        grad = act_bwd(input, d_out, _native.ACT_LEAKY_RELU, ctx.negative_slope)
        return grad, None


class LeakyReLU:
    def __init__(self, negative_slope=0.01):
        self.negative_slope = negative_slope
        self.leakyrelu_fn = leakyrelu.apply

    def __call__(self, x):
        return self.leakyrelu_fn(x, self.negative_slope)
