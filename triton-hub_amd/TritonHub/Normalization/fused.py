"""LayerNorm / RMSNorm with an activation applied in the same pass.

The reference has no such operator: its quick start chains ``LayerNorm`` and ``GeLU`` (README.md:47-48), which costs
a second read and write of the tensor in the forward and three more passes in the backward.  The modules below
compute ``act(norm(x))`` in one forward kernel and one backward kernel (plus the dW / dB reduction): the
pre-activation is never written, the backward recomputes it from the saved (input, weight, bias, mean, rstd).
Constructor arguments are those of ``LayerNorm`` / ``RMSNorm`` plus ``activation``: 'gelu', 'gelu_tanh', 'silu' or
'relu' (the parameter-free activations whose backward needs only their input).  Because the intermediate is not
rounded to the storage type, results are closer to exact arithmetic than the chained modules', not bit-identical.
"""
import torch

from .. import _native
from ._launch import norm_bwd, norm_fwd
from .layernorm import LayerNorm
from .rmsnorm import RMSNorm

ACTIVATIONS = {'gelu': _native.ACT_GELU, 'gelu_tanh': _native.ACT_GELU_TANH, 'silu': _native.ACT_SILU,
               'relu': _native.ACT_RELU}


def _code(activation: str) -> int:
    assert activation in ACTIVATIONS, f'activation must be one of {sorted(ACTIVATIONS)}'
    return ACTIVATIONS[activation]


class layernorm_act(torch.autograd.Function):
    """forward(ctx, input, weight, bias, eps, act) -> act(layernorm(input)); saves what ``layernorm`` saves."""

    @staticmethod
    def forward(ctx, input, weight, bias, eps, act):
        output, mean, rstd = norm_fwd(input, weight, bias, eps, layernorm=True, act=act, backward_follows=any(ctx.needs_input_grad))
        ctx.save_for_backward(input, weight, bias, mean, rstd)
        ctx.eps = eps
        ctx.act = act
        return output

    @staticmethod
    def backward(ctx, d_out):
        input, weight, bias, mean, rstd = ctx.saved_tensors
        _, need_dw, need_db = ctx.needs_input_grad[:3]
        grad, dw, db = norm_bwd(input, d_out, weight, bias, mean, rstd, layernorm=True, act=ctx.act, need_dw=need_dw,
                                need_db=need_db)
        return grad, dw, db, None, None


class rmsnorm_act(torch.autograd.Function):
    """forward(ctx, input, weight, eps, act) -> act(rmsnorm(input)); saves what ``rmsnorm`` saves."""

    @staticmethod
    def forward(ctx, input, weight, eps, act):
        output, _, rstd = norm_fwd(input, weight, None, eps, layernorm=False, act=act, backward_follows=any(ctx.needs_input_grad))
        ctx.save_for_backward(input, weight, rstd)
        ctx.eps = eps
        ctx.act = act
        return output

    @staticmethod
    def backward(ctx, d_out):
        input, weight, rstd = ctx.saved_tensors
        grad, dw, _ = norm_bwd(input, d_out, weight, None, None, rstd, layernorm=False, act=ctx.act,
                               need_dw=ctx.needs_input_grad[1])
        return grad, dw, None, None


class LayerNormActivation(LayerNorm):
    """LayerNormActivation(dimension, activation='gelu', eps=1e-5, elementwise_affine=True, bias=True, device=None,
    dtype=None): ``Activation()(LayerNorm(...)(x))`` in one pass.  Parameters and state dict as ``LayerNorm``."""

    def __init__(self, dimension, activation='gelu', eps=1e-5, elementwise_affine=True, bias=True, device=None, dtype=None):
        super().__init__(dimension, eps=eps, elementwise_affine=elementwise_affine, bias=bias, device=device, dtype=dtype)
        self.activation = activation
        self.act = _code(activation)
        self.layernorm_act_fn = layernorm_act.apply

    def forward(self, x):
        return self.layernorm_act_fn(x, self.weight, self.bias, self.eps, self.act)


class RMSNormActivation(RMSNorm):
    """RMSNormActivation(dimension, activation='silu', eps=1e-5, elementwise_affine=True, device=None, dtype=None):
    ``Activation()(RMSNorm(...)(x))`` in one pass.  Parameters and state dict as ``RMSNorm``."""

    def __init__(self, dimension, activation='silu', eps=1e-5, elementwise_affine=True, device=None, dtype=None):
        super().__init__(dimension, eps=eps, elementwise_affine=elementwise_affine, device=device, dtype=dtype)
        self.activation = activation
        self.act = _code(activation)
        self.rmsnorm_act_fn = rmsnorm_act.apply

    def forward(self, x):
        return self.rmsnorm_act_fn(x, self.weight, self.eps, self.act)
