"""x / max(||x||_p, eps) over the last dimension of a (B, L, D) tensor: drop-in for
``TritonHub/Ops/normalize.py`` of the reference (the ``Normalize`` autograd Function, normalize.py:144-160, and the
``normalize`` callable, :162-170)."""
import torch

from ._launch import normalize_bwd, normalize_fwd


class Normalize(torch.autograd.Function):
    """forward(ctx, x, p=2, eps=1e-6) -> x_norm; saves (x, x_norm, norms) with the norms in x.dtype."""

    @staticmethod
    @torch.amp.custom_fwd(device_type='cuda')
    def forward(ctx, x, p=2, eps=1e-6):
        assert len(x.shape) == 3, "Expected Tensor to be 3D (B, L, D), add batch dim input is 2D"
        ctx.p = p
        x_norm, norms_x = normalize_fwd(x, p, eps)
        ctx.save_for_backward(x, x_norm, norms_x)
        return x_norm

    @staticmethod
    @torch.amp.custom_bwd(device_type='cuda')
    def backward(ctx, grad_output):
        p = ctx.p
        x, x_norm, norms_x = ctx.saved_tensors
        grad_x = normalize_bwd(x, x_norm, norms_x, grad_output, p)
        return grad_x, None, None


class normalize:
    def __init__(self, p=2, eps=1e-6):
        assert p >= 1 and p <= 6, "p must be in [1, 6] for numerical stability"
        assert eps >= 0, "eps must be non-negative"
        self.p = p
        self.eps = eps
        self.normalize = Normalize.apply

    def __call__(self, x):
        return self.normalize(x, self.p, self.eps)
