"""LayerNorm over the last dimension: drop-in for ``TritonHub/Normalization/layernorm.py`` of the reference.

Same public surface -- the ``layernorm`` autograd Function (layernorm.py:211-223) and the ``LayerNorm``
module (layernorm.py:225-252) -- with the Triton kernels replaced by HIP kernels for gfx950.
"""
import torch

from ._launch import norm_bwd, norm_fwd


class layernorm(torch.autograd.Function):
    """forward(ctx, input, weight, bias, eps) -> output; saves (input, weight, bias, mean, rstd), the last two
    being (M,) float32 row statistics: mean = sum(x)/N, rstd = 1/sqrt(biased variance + eps)."""

    @staticmethod
    def forward(ctx, input, weight, bias, eps):
        output, mean, rstd = norm_fwd(input, weight, bias, eps, layernorm=True, backward_follows=any(ctx.needs_input_grad))
        ctx.save_for_backward(input, weight, bias, mean, rstd)
        ctx.eps = eps
        return output

    @staticmethod
    def backward(ctx, d_out):
        input, weight, bias, mean, rstd = ctx.saved_tensors
        _, need_dw, need_db = ctx.needs_input_grad[:3]        # frozen parameters: their sums are skipped
        grad, dw, db = norm_bwd(input, d_out, weight, bias, mean, rstd, layernorm=True, need_dw=need_dw,
                                need_db=need_db)
        return grad, dw, db, None


class LayerNorm(torch.nn.Module):
    """LayerNorm(dimension, eps=1e-5, elementwise_affine=True, bias=True, device=None, dtype=None).

    Parameters are named ``weight`` and ``bias`` with shape (dimension,), initialised to ones and zeros, and
    registered as None when disabled, so ``state_dict`` interchanges with the reference and with
    ``torch.nn.LayerNorm``.
    """

    def __init__(self, dimension, eps=1e-5, elementwise_affine=True, bias=True, device=None, dtype=None):
        super().__init__()
        self.dim = dimension
        self.eps = eps
        self.elementwise_affine = elementwise_affine
        has_weight = bool(elementwise_affine)
        has_bias = has_weight and bool(bias)
        for name, present in (('weight', has_weight), ('bias', has_bias)):
            value = torch.nn.Parameter(torch.empty(self.dim, device=device, dtype=dtype)) if present else None
            self.register_parameter(name, value)
        self.reset_parameters()
        self.layernorm_fn = layernorm.apply

    def reset_parameters(self):
        if self.weight is not None:
            torch.nn.init.ones_(self.weight)
        if self.bias is not None:
            torch.nn.init.zeros_(self.bias)

    def forward(self, x):
        return self.layernorm_fn(x, self.weight, self.bias, self.eps)
