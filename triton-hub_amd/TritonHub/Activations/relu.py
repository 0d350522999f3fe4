"""ReLU: drop-in for ``TritonHub/Activations/relu.py`` of the reference (the ``relu`` autograd Function,
relu.py:81-92, and the ``ReLU`` callable, :94-98).  The Function saves its input."""
import torch

from .. import _native
from ._launch import act_bwd, act_fwd


class relu(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input):
        output = act_fwd(input, _native.ACT_RELU)
        ctx.save_for_backward(input)
        return output

    @staticmethod
    def backward(ctx, d_out):
        input, = ctx.saved_tensors
        return act_bwd(input, d_out, _native.ACT_RELU)


class ReLU:
    def __init__(self):
        self.relu_fn = relu.apply

    def __call__(self, x):
        return self.relu_fn(x)
