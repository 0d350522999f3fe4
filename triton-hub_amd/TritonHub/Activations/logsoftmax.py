"""LogSoftmax over the last dimension: drop-in for ``TritonHub/Activations/logsoftmax.py`` of the reference
(the ``logsoftmax`` autograd Function, logsoftmax.py:93-110, and the ``LogSoftmax`` callable, :126-130)."""
import torch

from .. import _native
from ._launch import softmax_bwd, softmax_fwd


class logsoftmax(torch.autograd.Function):
    """forward(ctx, input) -> log_softmax(input, dim=-1); saves the OUTPUT; backward: dy - exp(y)*sum(dy)."""

    @staticmethod
    def forward(ctx, input):
        output = softmax_fwd(input, _native.LOGSOFTMAX)
        ctx.save_for_backward(output)
        return output

    @staticmethod
    def backward(ctx, d_out):
        output, = ctx.saved_tensors
        return softmax_bwd(output, d_out, _native.LOGSOFTMAX)


class LogSoftmax:
    def __init__(self):
        self.logsoftmax_fn = logsoftmax.apply

    def __call__(self, x):
        return self.logsoftmax_fn(x)
