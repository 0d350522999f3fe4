"""Host launch wrappers of the activations (softmax family and element-wise).

They do what the reference's ``_softmax_fwd`` / ``_softmax_bwd`` (softmax.py:25-41, :64-84) and their softmin /
logsoftmax twins do on the host -- make the last dimension contiguous, flatten to (M, N), allocate the output
with the same assertion messages -- and then call the C ABI of libthnorm.so on the current stream.
"""
import torch

from .. import _native
from ..Normalization._launch import FEATURE_DIM_MESSAGE, _on_device, _stream_handle


def _rows(t: torch.Tensor) -> torch.Tensor:
    if t.stride(-1) != 1:
        t = t.contiguous()
    t = t.reshape(-1, t.shape[-1])
    if t.shape[0] > 1 and t.stride(0) < t.shape[1]:
        t = t.contiguous()
    return t


def _check_row(n: int, element_size: int) -> None:
    # The reference launches a second program per row beyond 64 KiB, each normalising its own chunk
    # (softmax.py:34-36): rows that wide are refused here instead of being computed chunk-wise.
    if n * element_size > 65536:
        raise RuntimeError(FEATURE_DIM_MESSAGE)


def softmax_fwd(x: torch.Tensor, kind: int) -> torch.Tensor:
    _native.require_gpu(x)
    batch_shape = x.shape[:-1]
    x2 = _rows(x)
    m, n = x2.shape
    out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    assert out.shape == x2.shape, 'expect output shape to be the same as input shape'
    assert out.stride(-1) == 1, 'expect output to be row-major'
    _check_row(n, x.element_size())
    code = _native.dtype_code(x.dtype)
    if m > 0:
        index = x.device.index
        with _on_device(index):
            status = _native.lib().thn_softmax_fwd(x2.data_ptr(), x2.stride(0) if m > 1 else n, out.data_ptr(), n,
                                                   m, n, kind, code, _stream_handle(index))
        if status != 0:
            _native.check(status)
    return out.reshape(*batch_shape, n)


def softmax_bwd(y: torch.Tensor, dout: torch.Tensor, kind: int) -> torch.Tensor:
    """`y` is the saved OUTPUT of the forward (softmax.py:86-97)."""
    _native.require_gpu(y)
    batch_shape = y.shape[:-1]
    y2 = _rows(y)
    d2 = _rows(dout)
    assert y2.shape == d2.shape, 'expect input and output shape to be the same'
    if d2.dtype != y2.dtype:
        d2 = d2.to(y2.dtype)
    m, n = y2.shape
    dx = torch.empty((m, n), dtype=y.dtype, device=y.device)
    assert dx.stride(-1) == 1, 'expect derivative to be row-major'
    _check_row(n, y.element_size())
    code = _native.dtype_code(y.dtype)
    if m > 0:
        index = y.device.index
        with _on_device(index):
            status = _native.lib().thn_softmax_bwd(y2.data_ptr(), y2.stride(0) if m > 1 else n, d2.data_ptr(),
                                                   d2.stride(0) if m > 1 else n, dx.data_ptr(), n, m, n, kind, code,
                                                   _stream_handle(index))
        if status != 0:
            _native.check(status)
    return dx.reshape(*batch_shape, n)


def act_fwd(x: torch.Tensor, act: int, param0: float = 0.0, param1: float = 0.0) -> torch.Tensor:
    """Element-wise forward: what the reference's ``_<name>_fwd`` wrappers do on the host (e.g. gelu.py:31-49) --
    last dimension contiguous, flatten to (M, N), allocate the output with the same assertions -- then the C ABI."""
    _native.require_gpu(x)
    batch_shape = x.shape[:-1]
    x2 = _rows(x)
    m, n = x2.shape
    out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    assert out.shape == x2.shape, 'expect output shape to be the same as input shape'
    assert out.stride(-1) == 1, 'expect output to be row-major'
    if m > 0 and n > 0:
        index = x.device.index
        with _on_device(index):
            status = _native.lib().thn_act_fwd(x2.data_ptr(), x2.stride(0) if m > 1 else n, out.data_ptr(), n, m, n, act,
                                               float(param0), float(param1), _native.dtype_code(x.dtype),
                                               _stream_handle(index))
        if status != 0:
            _native.check(status)
    return out.reshape(*batch_shape, n)


def act_bwd(saved: torch.Tensor, dout: torch.Tensor, act: int, param0: float = 0.0, param1: float = 0.0) -> torch.Tensor:
    """Element-wise backward (e.g. gelu.py:83-105); ``saved`` is what the reference's Function saved."""
    _native.require_gpu(saved)
    batch_shape = saved.shape[:-1]
    s2 = _rows(saved)
    d2 = _rows(dout)
    assert s2.shape == d2.shape, 'expect input and output shape to be the same'
    if d2.dtype != s2.dtype:
        d2 = d2.to(s2.dtype)
    m, n = s2.shape
    dx = torch.empty((m, n), dtype=saved.dtype, device=saved.device)
    assert dx.stride(-1) == 1, 'expect derivative to be row-major'
    if m > 0 and n > 0:
        index = saved.device.index
        with _on_device(index):
            status = _native.lib().thn_act_bwd(s2.data_ptr(), s2.stride(0) if m > 1 else n, d2.data_ptr(),
                                               d2.stride(0) if m > 1 else n, dx.data_ptr(), n, m, n, act, float(param0),
                                               float(param1), _native.dtype_code(saved.dtype), _stream_handle(index))
        if status != 0:
            _native.check(status)
    return dx.reshape(*batch_shape, n)
