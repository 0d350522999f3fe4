"""SiLU: drop-in for ``TritonHub/Activations/silu.py`` of the reference (the ``silu`` autograd Function,
silu.py:82-93, and the ``SiLU`` callable, :95-99).  The Function saves its input."""
import torch

from .. import _native
from ._launch import act_bwd, act_fwd


class silu(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input):
        output = act_fwd(input, _native.ACT_SILU)
        ctx.save_for_backward(input)
        return output

    @staticmethod
    def backward(ctx, d_out):
        input, = ctx.saved_tensors
        return act_bwd(input, d_out, _native.ACT_SILU)


class SiLU:
    def __init__(self):
        self.silu_fn = silu.apply

    def __call__(self, x):
        return self.silu_fn(x)
