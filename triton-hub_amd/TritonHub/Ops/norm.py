"""Row p-norm over the last dimension of a (B, L, D) tensor: drop-in for ``TritonHub/Ops/norm.py`` of the
reference (the ``Norm`` autograd Function, norm.py:128-144, and the ``norm`` callable, :146-154)."""
import torch

from ._launch import norm_bwd, norm_fwd


class Norm(torch.autograd.Function):
    """forward(ctx, x, p=2, eps=1e-6) -> max(||x||_p, eps) of shape (B, L) in x.dtype; saves (x, norms)."""

    @staticmethod
    @torch.amp.custom_fwd(device_type='cuda')
    def forward(ctx, x, p=2, eps=1e-6):
        assert len(x.shape) == 3, "Expected Tensor to be 3D (B, L, D), add batch dim input is 2D"
        ctx.p = p
        norms_x = norm_fwd(x, p, eps)
        ctx.save_for_backward(x, norms_x)
        return norms_x

    @staticmethod
    @torch.amp.custom_bwd(device_type='cuda')
    def backward(ctx, grad_output):
        p = ctx.p
        x, norms_x = ctx.saved_tensors
        grad_x = norm_bwd(x, norms_x, grad_output, p)
        return grad_x, None, None


class norm:
    def __init__(self, p=2, eps=1e-6):
        assert p >= 1 and p <= 6, "p must be in [1, 6] for numerical stability"
        assert eps >= 0, "eps must be non-negative"
        self.p = p
        self.eps = eps
        self.norm = Norm.apply

    def __call__(self, x):
        return self.norm(x, self.p, self.eps)
