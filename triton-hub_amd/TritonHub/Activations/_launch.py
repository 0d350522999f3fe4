"""Host launch wrappers of the activations (softmax family and element-wise).

They do what the reference's ``_softmax_fwd`` / ``_softmax_bwd`` (softmax.py:25-41, :64-84) and their softmin /
logsoftmax twins do on the host -- make the last dimension contiguous, flatten to (M, N), allocate the output
with the same assertion messages -- and then call the C ABI of libthnorm.so on the current stream.
"""
import torch

from .. import _native
from ..Normalization._launch import _current_device, _stream_handle


def _rows(t: torch.Tensor) -> torch.Tensor:
    if t.stride(-1) != 1:
        t = t.contiguous()
    t = t.reshape(-1, t.shape[-1])
    if t.shape[0] > 1 and t.stride(0) < t.shape[1]:
        t = t.contiguous()
    return t


def _flatten(t: torch.Tensor):
    """(tensor to pass, M, N, row stride in elements, needs un-flattening): a contiguous tensor is passed as it is."""
    n = t.shape[-1]
    if t.is_contiguous() and n > 0:
        return t, t.numel() // n, n, n, False
    t2 = _rows(t)
    m = t2.shape[0]
    return t2, m, n, (t2.stride(0) if m > 1 else n), True


def _call(device, fn_name, *args):
    """One C-ABI call on torch's current stream of `device`, with that device current."""
    index = device.index
    other_device = _current_device() != index
    if other_device:
        guard = torch.cuda.device(index)
        guard.__enter__()
    try:
        status = getattr(_native.lib(), fn_name)(*args, _stream_handle(index))
    finally:
        if other_device:
            guard.__exit__(None, None, None)
    if status != 0:
        _native.check(status)


def softmax_fwd(x: torch.Tensor, kind: int) -> torch.Tensor:
    if not x.is_cuda:
        _native.require_gpu(x)
    x2, m, n, x_stride, reshaped = _flatten(x)
    out = torch.empty((m, n), dtype=x.dtype, device=x.device) if reshaped else torch.empty_like(x)
    assert out.numel() == x2.numel(), 'expect output shape to be the same as input shape'
    assert out.stride(-1) == 1, 'expect output to be row-major'
    if m > 0:
        _call(x.device, 'thn_softmax_fwd', x2.data_ptr(), x_stride, out.data_ptr(), n, m, n, kind,
              _native.dtype_code(x.dtype))
    return out.reshape(*x.shape[:-1], n) if reshaped else out


def softmax_bwd(y: torch.Tensor, dout: torch.Tensor, kind: int) -> torch.Tensor:
    """`y` is the saved OUTPUT of the forward (softmax.py:86-97)."""
    if not y.is_cuda:
        _native.require_gpu(y)
    y2, m, n, y_stride, reshaped = _flatten(y)
    d2, dm, dn, d_stride, _ = _flatten(dout)
    assert dm == m and dn == n, 'expect input and output shape to be the same'
    if d2.dtype != y2.dtype:
        d2 = d2.to(y2.dtype)
    dx = torch.empty((m, n), dtype=y.dtype, device=y.device) if reshaped else torch.empty_like(y)
    assert dx.stride(-1) == 1, 'expect derivative to be row-major'
    if m > 0:
        _call(y.device, 'thn_softmax_bwd', y2.data_ptr(), y_stride, d2.data_ptr(), d_stride, dx.data_ptr(), n, m, n, kind,
              _native.dtype_code(y.dtype))
    return dx.reshape(*y.shape[:-1], n) if reshaped else dx


def act_fwd(x: torch.Tensor, act: int, param0: float = 0.0, param1: float = 0.0) -> torch.Tensor:
    """Element-wise forward: what the reference's ``_<name>_fwd`` wrappers do on the host (e.g. gelu.py:31-49) --
    last dimension contiguous, flatten to (M, N), allocate the output with the same assertions -- then the C ABI."""
    if not x.is_cuda:
        _native.require_gpu(x)
    x2, m, n, x_stride, reshaped = _flatten(x)
    out = torch.empty((m, n), dtype=x.dtype, device=x.device) if reshaped else torch.empty_like(x)
    assert out.numel() == x2.numel(), 'expect output shape to be the same as input shape'
    assert out.stride(-1) == 1, 'expect output to be row-major'
    if m > 0:
        _call(x.device, 'thn_act_fwd', x2.data_ptr(), x_stride, out.data_ptr(), n, m, n, act, float(param0),
              float(param1), _native.dtype_code(x.dtype))
    return out.reshape(*x.shape[:-1], n) if reshaped else out


def act_bwd(saved: torch.Tensor, dout: torch.Tensor, act: int, param0: float = 0.0, param1: float = 0.0) -> torch.Tensor:
    """Element-wise backward (e.g. gelu.py:83-105); ``saved`` is what the reference's Function saved."""
    if not saved.is_cuda:
        _native.require_gpu(saved)
    s2, m, n, s_stride, reshaped = _flatten(saved)
    d2, dm, dn, d_stride, _ = _flatten(dout)
    assert dm == m and dn == n, 'expect input and output shape to be the same'
    if d2.dtype != s2.dtype:
        d2 = d2.to(s2.dtype)
    dx = torch.empty((m, n), dtype=saved.dtype, device=saved.device) if reshaped else torch.empty_like(saved)
    assert dx.stride(-1) == 1, 'expect derivative to be row-major'
    if m > 0:
        _call(saved.device, 'thn_act_bwd', s2.data_ptr(), s_stride, d2.data_ptr(), d_stride, dx.data_ptr(), n, m, n, act,
              float(param0), float(param1), _native.dtype_code(saved.dtype))
    return dx.reshape(*saved.shape[:-1], n) if reshaped else dx
