"""Dropout: drop-in for ``TritonHub/Layers/dropout.py`` of the reference -- the ``dropout`` autograd Function
(dropout.py:95-111) and the ``Dropout`` module (:113-119).

The mask is the reference's: element i of the flattened tensor is dropped when Triton's ``tl.rand(seed, i) < p``
(dropout.py:20-21), and the HIP kernel evaluates the same Philox-4x32-10 stream.  The seed is drawn as the reference
draws it, ``random.randint(0, 2**16)`` from Python's ``random`` module once per forward call (dropout.py:98), so a
program that seeds ``random`` sees the same masks with either library.
"""
import random

import torch

from .. import _native
from ..Activations._launch import _call


def _dropout_apply(t: torch.Tensor, p, seed, training, what: str) -> torch.Tensor:
    """Forward and backward are the same function of their tensor (dropout.py:25-50, :69-94)."""
    if not t.is_cuda:
        _native.require_gpu(t)
    if t.stride(-1) != 1:
        t = t.contiguous()
    assert t.stride(-1) == 1 or t.numel() == 0, 'expect input to be row-major'     # (empty: any strides)
    if (p == 0.0) or (not training):
        return t
    if p == 1.0:
        return torch.zeros_like(t, memory_format=torch.contiguous_format)
    flat = t.reshape(-1)                      # a copy when the tensor is not contiguous, as in the reference
    out = torch.empty_like(flat, memory_format=torch.contiguous_format)
    assert out.shape == flat.shape, 'expect output shape to be the same as input shape'
    assert out.stride(-1) == 1, 'expect output to be row-major'
    if flat.numel() > 0:
        _call(t.device, 'thn_dropout', flat.data_ptr(), out.data_ptr(), flat.numel(), 0, float(p), int(seed),
              _native.dtype_code(t.dtype))
    return out.reshape(t.shape)


class dropout(torch.autograd.Function):
    """forward(ctx, input, p, training) -> output; keeps (p, seed, training) on ctx and no tensor: the backward
    regenerates the mask from the seed."""

    @staticmethod
    def forward(ctx, input, p, training):
        seed = random.randint(0, 2**16)
        output = _dropout_apply(input, p, seed, training, 'input')
        ctx.p = p
        ctx.seed = seed
        ctx.training = training
        return output

    @staticmethod
    def backward(ctx, d_out):
        grad = _dropout_apply(d_out, ctx.p, ctx.seed, ctx.training, 'gradient')
        return grad, None, None


class Dropout(torch.nn.Module):
    """Dropout(p=0.5): zeroes each element with probability p while training and scales the rest by 1 / (1 - p)."""

    def __init__(self, p=0.5):
        super().__init__()
        self.p = p
        self.dropout_fn = dropout.apply

    def forward(self, x):
        return self.dropout_fn(x, self.p, self.training)
