"""RMSNorm over the last dimension: drop-in for ``TritonHub/Normalization/rmsnorm.py`` of the reference.

Same public surface -- the ``rmsnorm`` autograd Function (rmsnorm.py:169-181) and the ``RMSNorm`` module
(rmsnorm.py:183-204) -- with the Triton kernels replaced by HIP kernels for gfx950.
"""
import torch

from ._launch import norm_bwd, norm_fwd


class rmsnorm(torch.autograd.Function):
    """forward(ctx, input, weight, eps) -> output; saves (input, weight, rstd) with rstd the (M,) float32
    row statistic 1/sqrt(mean(x^2) + eps)."""

    @staticmethod
    def forward(ctx, input, weight, eps):
        output, _, rstd = norm_fwd(input, weight, None, eps, layernorm=False, backward_follows=any(ctx.needs_input_grad))
        ctx.save_for_backward(input, weight, rstd)
        ctx.eps = eps
        return output

    @staticmethod
    def backward(ctx, d_out):
        input, weight, rstd = ctx.saved_tensors
        grad, dw, _ = norm_bwd(input, d_out, weight, None, None, rstd, layernorm=False,
                               need_dw=ctx.needs_input_grad[1])           # a frozen weight: no column sums
        return grad, dw, None


class RMSNorm(torch.nn.Module):
    """RMSNorm(dimension, eps=1e-5, elementwise_affine=True, device=None, dtype=None).

    ``weight`` has shape (dimension,) and starts at ones (None when ``elementwise_affine`` is false);
    ``bias`` is always registered as None, as in the reference (rmsnorm.py:194).
    """

    def __init__(self, dimension, eps=1e-5, elementwise_affine=True, device=None, dtype=None):
        super().__init__()
        self.dim = dimension
        self.eps = eps
        self.elementwise_affine = elementwise_affine
        weight = torch.nn.Parameter(torch.empty(self.dim, device=device, dtype=dtype)) if elementwise_affine else None
        self.register_parameter('weight', weight)
        self.register_parameter('bias', None)
        self.reset_parameters()
        self.rmsnorm_fn = rmsnorm.apply

    def reset_parameters(self):
        if self.weight is not None:
            torch.nn.init.ones_(self.weight)

    def forward(self, x):
        return self.rmsnorm_fn(x, self.weight, self.eps)
