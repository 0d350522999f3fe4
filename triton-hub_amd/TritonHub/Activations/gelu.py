"""GeLU: drop-in for ``TritonHub/Activations/gelu.py`` of the reference (the ``gelu`` autograd Function,
gelu.py:107-119, and the ``GeLU`` callable, :121-129)."""
import torch

from .. import _native
from ._launch import act_bwd, act_fwd


def _code(approximate):
    return _native.ACT_GELU_TANH if approximate == 'tanh' else _native.ACT_GELU


class gelu(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, approximate):
        output = act_fwd(input, _code(approximate))
        ctx.save_for_backward(input)
        ctx.approximate = approximate
        return output

    @staticmethod
    def backward(ctx, d_out):
        input, = ctx.saved_tensors
        grad = act_bwd(input, d_out, _code(ctx.approximate))
        return grad, None


class GeLU:
    def __init__(self, approximate='none'):
        assert approximate in ['none', 'tanh'], 'GeLU approximate must be either none or tanh'
        self.approximate = approximate
        self.gelu_fn = gelu.apply

    def __call__(self, x):
        return self.gelu_fn(x, self.approximate)
