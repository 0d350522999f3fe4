"""ReLU6: drop-in for ``TritonHub/Activations/relu6.py`` of the reference (the ``relu6`` autograd Function,
relu6.py:83-94, and the ``ReLU6`` callable, :96-100).  The Function saves its input."""
import torch

from .. import _native
from ._launch import act_bwd, act_fwd


class relu6(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input):
        output = act_fwd(input, _native.ACT_RELU6)
        ctx.save_for_backward(input)
        return output

    @staticmethod
    def backward(ctx, d_out):
        input, = ctx.saved_tensors
        return act_bwd(input, d_out, _native.ACT_RELU6)


class ReLU6:
    def __init__(self):
        self.relu6_fn = relu6.apply

    def __call__(self, x):
        return self.relu6_fn(x)
