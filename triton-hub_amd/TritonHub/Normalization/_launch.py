"""Host launch wrappers shared by LayerNorm and RMSNorm.

They do what the reference's ``_layernorm_fwd`` / ``_layernorm_bwd`` / ``_rmsnorm_fwd`` / ``_rmsnorm_bwd`` do
on the host (layernorm.py:48-87, :155-209; rmsnorm.py:40-70, :124-167): make the last dimension contiguous,
flatten to (M, N), check the parameter shapes with the same assertion messages, allocate the outputs and
the float32 row statistics, refuse rows wider than 64 KiB -- and then, instead of launching Triton kernels,
call the C ABI of libthnorm.so on the current stream of the input's device.
"""
from __future__ import annotations

import ctypes

import torch

from .. import _native

FEATURE_DIM_MESSAGE = "This layer norm doesn't support feature dim >= 64KB."


def _rows(t: torch.Tensor, what: str) -> torch.Tensor:
    """(…, N) -> (M, N) with unit column stride (layernorm.py:49-53)."""
    if t.stride(-1) != 1:
        t = t.contiguous()
    t = t.reshape(-1, t.shape[-1])
    if t.shape[0] > 1 and t.stride(0) < t.shape[1]:
        t = t.contiguous()          # broadcast (stride 0) rows: materialise, the kernels need distinct rows
    assert t.stride(-1) == 1, f'expect {what} to be row-major'
    return t


def _param(p, n: int, name: str):
    if p is None:
        return None
    p = p.contiguous()
    assert p.shape == (n,), f'expect {name} to have shape (N,)'
    assert p.stride(-1) == 1, f'expect {name} to be row-major'
    return p


def _check_feature_dim(n: int, element_size: int) -> None:
    if n * element_size > 65536:
        raise RuntimeError(FEATURE_DIM_MESSAGE)


_raw_stream = getattr(torch._C, '_cuda_getCurrentRawStream', None)
_workspace_bytes_cache = {}


def _stream_handle(index: int) -> int:
    """hipStream_t of torch's current stream on device `index`, as an integer."""
    if _raw_stream is not None:
        return _raw_stream(index)
    return torch.cuda.current_stream(index).cuda_stream


class _on_device:
    """Makes `index` the current HIP device for the duration of a launch; free when it already is
    (the reference wraps its launches in `with torch.cuda.device(x.device.index)`, layernorm.py:73)."""

    __slots__ = ('index', 'guard')

    def __init__(self, index: int):
        self.index = index
        self.guard = None

    def __enter__(self):
        if torch.cuda.current_device() != self.index:
            self.guard = torch.cuda.device(self.index)
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)
        return False


def norm_fwd(x: torch.Tensor, weight, bias, eps: float, layernorm: bool):
    """Returns (y like x, mean (M,) float32 or None, rstd (M,) float32)."""
    _native.require_gpu(x)
    batch_shape = x.shape[:-1]
    x2 = _rows(x, 'input')
    m, n = x2.shape
    weight = _param(weight, n, 'weight')
    bias = _param(bias, n, 'bias')
    out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    assert out.stride(-1) == 1, 'expect output to be row-major'
    mean = torch.empty((m,), dtype=torch.float32, device=x.device) if layernorm else None
    rstd = torch.empty((m,), dtype=torch.float32, device=x.device)
    _check_feature_dim(n, x.element_size())
    x_code = _native.dtype_code(x.dtype)
    if m == 0:                       # nothing to launch (and empty tensors have no address to pass)
        return out.reshape(*batch_shape, n), mean, rstd
    params = weight if weight is not None else bias
    if weight is not None and bias is not None and weight.dtype != bias.dtype:
        bias = bias.to(weight.dtype)
    w_code = _native.dtype_code(params.dtype) if params is not None else x_code
    index = x.device.index
    with _on_device(index):
        status = _native.lib().thn_norm_fwd(
            x2.data_ptr(), x2.stride(0) if m > 1 else n, out.data_ptr(), n,
            _native.ptr(weight), _native.ptr(bias), _native.ptr(mean), rstd.data_ptr(),
            m, n, float(eps), x_code, w_code, _stream_handle(index))
    if status != 0:
        _native.check(status)
    return out.reshape(*batch_shape, n), mean, rstd


def norm_bwd(x: torch.Tensor, dout: torch.Tensor, weight, bias, mean, rstd, layernorm: bool):
    """Returns (dx like x, dw or None, db or None); dw/db take the dtype of weight/bias (layernorm.py:207-208)."""
    _native.require_gpu(x)
    batch_shape = x.shape[:-1]
    x2 = _rows(x, 'input')
    m, n = x2.shape
    d2 = _rows(dout, 'output')
    assert d2.shape == (m, n), 'expect input and output shape to be the same'
    if d2.dtype != x2.dtype:
        d2 = d2.to(x2.dtype)
    weight = _param(weight, n, 'weight')
    bias = _param(bias, n, 'bias')
    dx = torch.empty((m, n), dtype=x.dtype, device=x.device)
    assert dx.stride(-1) == 1, 'expect derivative to be row-major'
    _check_feature_dim(n, x.element_size())
    x_code = _native.dtype_code(x.dtype)
    want_db = layernorm and bias is not None
    mixed = weight is not None and want_db and weight.dtype != bias.dtype
    grad_dtype = weight.dtype if weight is not None else (bias.dtype if want_db else x.dtype)
    w_code = _native.dtype_code(grad_dtype)
    dw = torch.empty((n,), dtype=grad_dtype, device=x.device) if weight is not None else None
    db = torch.empty((n,), dtype=grad_dtype, device=x.device) if want_db else None
    if m == 0:                       # the sum over no rows
        dw = None if dw is None else dw.zero_()
        db = None if db is None else db.zero_().to(bias.dtype)
        return dx.reshape(*batch_shape, n), dw, db
    lib = _native.lib()
    index = x.device.index
    with _on_device(index):
        key = (index, m, n, dw is not None, db is not None, x_code)
        nbytes = _workspace_bytes_cache.get(key)
        if nbytes is None:
            nbytes = int(lib.thn_norm_bwd_workspace_bytes(m, n, int(dw is not None), int(db is not None), x_code))
            if nbytes < 0:
                _native.check(nbytes)
            _workspace_bytes_cache[key] = nbytes
        # the counterpart of the reference's per-call _dw / _db buffers (layernorm.py:183-184)
        workspace = torch.empty((max(nbytes, 16) // 4,), dtype=torch.float32, device=x.device)
        status = lib.thn_norm_bwd(
            x2.data_ptr(), x2.stride(0) if m > 1 else n, d2.data_ptr(), d2.stride(0) if m > 1 else n,
            dx.data_ptr(), n, _native.ptr(weight), _native.ptr(mean), rstd.data_ptr(),
            _native.ptr(dw), _native.ptr(db), workspace.data_ptr(), nbytes, m, n, x_code, w_code,
            _stream_handle(index))
    if status != 0:
        _native.check(status)
    if mixed:
        db = db.to(bias.dtype)
    return dx.reshape(*batch_shape, n), dw, db


def query_launch(which: int, layernorm: bool, m: int, n: int, dtype: torch.dtype):
    """(vecs_per_thread, threads_per_row, block_threads, grid_blocks, vector_path) the library would use."""
    shape = (ctypes.c_int32 * 5)()
    _native.check(_native.lib().thn_norm_query_launch(which, int(layernorm), m, n, _native.dtype_code(dtype), shape))
    return tuple(shape)
