"""Host launch wrappers shared by LayerNorm and RMSNorm.

They do what the reference's ``_layernorm_fwd`` / ``_layernorm_bwd`` / ``_rmsnorm_fwd`` / ``_rmsnorm_bwd`` do
on the host (layernorm.py:48-87, :155-209; rmsnorm.py:40-70, :124-167): make the last dimension contiguous,
flatten to (M, N), check the parameter shapes with the same assertion messages, allocate the outputs and
the float32 row statistics, refuse rows wider than 64 KiB -- and then, instead of launching Triton kernels,
call the C ABI of libthnorm.so on the current stream of the input's device.
"""
from __future__ import annotations

import ctypes
import threading

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
    if not p.is_contiguous():
        p = p.contiguous()
    assert p.shape == (n,), f'expect {name} to have shape (N,)'
    assert p.stride(-1) == 1, f'expect {name} to be row-major'
    return p


def _check_feature_dim(n: int, element_size: int) -> None:
    if n * element_size > 65536:
        raise RuntimeError(FEATURE_DIM_MESSAGE)


# How the forward reads x (include/thnorm.h, thn_cache_policy): 'keep' leaves x in the caches for the backward,
# 'stream' does not; 'auto' keeps it exactly when autograd will run a backward for the call.
_CACHE_POLICIES = ('auto', 'keep', 'stream')
_cache_policy = 'auto'


def set_cache_policy(policy: str) -> None:
    """'auto' (default): the forward keeps x in the caches when a backward will follow (some input of the autograd
    Function requires a gradient) and streams it otherwise (inference); 'keep' / 'stream': always.  Choose 'stream'
    for training loops in which so much other work runs between a layer's forward and its backward that nothing of
    x would still be cached: the forward alone is 2-3 % faster that way.  Results are bit-identical under all three."""
    global _cache_policy
    if policy not in _CACHE_POLICIES:
        raise ValueError(f'cache policy must be one of {_CACHE_POLICIES}, got {policy!r}')
    _cache_policy = policy


def get_cache_policy() -> str:
    return _cache_policy


def _x_policy_flag(backward_follows: bool) -> int:
    policy = _cache_policy
    if policy == 'auto':
        return _native.X_KEEP if backward_follows else _native.X_STREAM
    return _native.X_KEEP if policy == 'keep' else _native.X_STREAM


_raw_stream = getattr(torch._C, '_cuda_getCurrentRawStream', None)
_get_device = getattr(torch._C, '_cuda_getDevice', None)
_workspace_cache = {}           # (device index, stream handle) -> uint8 tensor, grown on demand
_backward_lock = threading.Lock()   # held from picking the shared workspace until both stages are enqueued
_F32 = torch.float32


def _stream_handle(index: int) -> int:
    """hipStream_t of torch's current stream on device `index`, as an integer."""
    if _raw_stream is not None:
        return _raw_stream(index)
    return torch.cuda.current_stream(index).cuda_stream


def _current_device() -> int:
    """Index of the current HIP device.  The launches below run with the tensor's device current (the reference
    wraps its launches in `with torch.cuda.device(x.device.index)`, layernorm.py:73); switching is skipped when it
    already is."""
    return _get_device() if _get_device is not None else torch.cuda.current_device()


def _flatten(t: torch.Tensor, what: str):
    """(tensor to pass, M, N, row stride in elements, needs un-flattening).  A contiguous tensor is passed as it
    is -- its rows are already N apart -- which skips two reshapes per call on the common path."""
    n = t.shape[-1]
    if t.is_contiguous() and t.dim() >= 1 and n > 0:
        return t, t.numel() // n, n, n, False
    t2 = _rows(t, what)
    m = t2.shape[0]
    return t2, m, n, (t2.stride(0) if m > 1 else n), True


def _workspace(index: int, stream: int, nbytes: int, device) -> torch.Tensor:
    """The counterpart of the reference's per-call `_dw` / `_db` partial buffers (layernorm.py:183-184).  One buffer
    per (device, stream) is kept and grown on demand: both stages of a backward are enqueued on that stream, so a
    later call on the same stream can only reuse the buffer after they have run.  The caller holds
    `_backward_lock` until both stages are enqueued, so two host threads that feed one stream cannot interleave
    their stages on the buffer.  While the stream is being captured into a graph the call gets a buffer of its
    own instead (the graph keeps it alive and would replay on the shared one while eager work uses it)."""
    if torch.cuda.is_current_stream_capturing():
        return torch.empty((max(nbytes, 16),), dtype=torch.uint8, device=device)
    key = (index, stream)
    ws = _workspace_cache.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty((max(nbytes, 16),), dtype=torch.uint8, device=device)
        _workspace_cache[key] = ws
    return ws


def norm_fwd(x: torch.Tensor, weight, bias, eps: float, layernorm: bool, act: int = -1, backward_follows: bool = True):
    """Returns (y like x, mean (M,) float32 or None, rstd (M,) float32).  `act` >= 0: the activation with that
    code is applied in the same pass (thn_norm_act_fwd).  `backward_follows`: whether autograd will run a backward
    for this call (it decides the cache policy of the read of x under set_cache_policy('auto'))."""
    if not x.is_cuda:
        _native.require_gpu(x)
    x2, m, n, x_stride, reshaped = _flatten(x, 'input')
    if weight is not None:
        weight = _param(weight, n, 'weight')
    if bias is not None:
        bias = _param(bias, n, 'bias')
    device = x.device
    out = torch.empty((m, n), dtype=x.dtype, device=device) if reshaped else torch.empty_like(x)
    assert out.stride(-1) == 1, 'expect output to be row-major'
    mean = torch.empty((m,), dtype=_F32, device=device) if layernorm else None
    rstd = torch.empty((m,), dtype=_F32, device=device)
    if n * x.element_size() > 65536:
        raise RuntimeError(FEATURE_DIM_MESSAGE)
    x_code = _native.dtype_code(x.dtype)
    if m == 0:                       # nothing to launch (and empty tensors have no address to pass)
        return (out.reshape(*x.shape[:-1], n) if reshaped else out), mean, rstd
    w_code = x_code
    x_code |= _x_policy_flag(backward_follows)
    if weight is not None:
        w_code = _native.dtype_code(weight.dtype)
        if bias is not None and weight.dtype != bias.dtype:
            bias = bias.to(weight.dtype)
    elif bias is not None:
        w_code = _native.dtype_code(bias.dtype)
    index = device.index
    other_device = _current_device() != index
    if other_device:
        guard = torch.cuda.device(index)
        guard.__enter__()
    try:
        if act < 0:
            status = _native.lib().thn_norm_fwd(
                x2.data_ptr(), x_stride, out.data_ptr(), n,
                0 if weight is None else weight.data_ptr(), 0 if bias is None else bias.data_ptr(),
                0 if mean is None else mean.data_ptr(), rstd.data_ptr(),
                m, n, float(eps), x_code, w_code, _stream_handle(index))
        else:
            status = _native.lib().thn_norm_act_fwd(
                x2.data_ptr(), x_stride, out.data_ptr(), n,
                0 if weight is None else weight.data_ptr(), 0 if bias is None else bias.data_ptr(),
                0 if mean is None else mean.data_ptr(), rstd.data_ptr(),
                m, n, float(eps), act, x_code, w_code, _stream_handle(index))
    finally:
        if other_device:
            guard.__exit__(None, None, None)
    if status != 0:
        _native.check(status)
    return (out.reshape(*x.shape[:-1], n) if reshaped else out), mean, rstd


def norm_bwd(x: torch.Tensor, dout: torch.Tensor, weight, bias, mean, rstd, layernorm: bool, act: int = -1,
             need_dw: bool = True, need_db: bool = True):
    """Returns (dx like x, dw or None, db or None); dw/db take the dtype of weight/bias (layernorm.py:207-208).
    `act` >= 0: the backward of norm_fwd(..., act) (thn_norm_act_bwd).  `need_dw` / `need_db` False: that parameter
    is frozen (autograd's needs_input_grad): its sums are not stored, and with both False the backward is the row
    kernel alone, without partial sums and without the second stage."""
    if not x.is_cuda:
        _native.require_gpu(x)
    x2, m, n, x_stride, reshaped = _flatten(x, 'input')
    d2, dm, dn, d_stride, _ = _flatten(dout, 'output')
    assert dm == m and dn == n, 'expect input and output shape to be the same'
    if d2.dtype != x2.dtype:
        d2 = d2.to(x2.dtype)
    if weight is not None:
        weight = _param(weight, n, 'weight')
    if bias is not None:
        bias = _param(bias, n, 'bias')
    device = x.device
    dx = torch.empty((m, n), dtype=x.dtype, device=device) if reshaped else torch.empty_like(x)
    assert dx.stride(-1) == 1, 'expect derivative to be row-major'
    if n * x.element_size() > 65536:
        raise RuntimeError(FEATURE_DIM_MESSAGE)
    x_code = _native.dtype_code(x.dtype)
    want_db = layernorm and bias is not None and need_db
    mixed = weight is not None and want_db and weight.dtype != bias.dtype
    # the storage type the kernels read w / b in and write dW / dB in: the weight's, else the bias's -- also when
    # the bias is frozen, because the fused backward still reads it to rebuild the pre-activation
    grad_dtype = weight.dtype if weight is not None else (bias.dtype if (layernorm and bias is not None) else x.dtype)
    w_code = _native.dtype_code(grad_dtype)
    dw = torch.empty((n,), dtype=grad_dtype, device=device) if (weight is not None and need_dw) else None
    db = torch.empty((n,), dtype=grad_dtype, device=device) if want_db else None
    if m == 0:                       # the sum over no rows
        dw = None if dw is None else dw.zero_()
        db = None if db is None else db.zero_().to(bias.dtype)
        return (dx.reshape(*x.shape[:-1], n) if reshaped else dx), dw, db
    lib = _native.lib()
    index = device.index
    other_device = _current_device() != index
    locked = False
    if other_device:
        guard = torch.cuda.device(index)
        guard.__enter__()
    try:
        # asked on every call: the answer follows the launch shape, which thn_norm_set_launch_override can change
        if act < 0:
            nbytes = int(lib.thn_norm_bwd_workspace_bytes(m, n, int(dw is not None), int(db is not None), x_code))
        else:
            nbytes = int(lib.thn_norm_act_bwd_workspace_bytes(m, n, int(dw is not None), int(db is not None), act,
                                                              x_code))
        if nbytes < 0:
            _native.check(nbytes)
        stream = _stream_handle(index)
        locked = nbytes > 0
        if locked:
            _backward_lock.acquire()
        workspace = _workspace(index, stream, nbytes, device) if nbytes > 0 else None
        if act < 0:
            status = lib.thn_norm_bwd(
                x2.data_ptr(), x_stride, d2.data_ptr(), d_stride, dx.data_ptr(), n,
                0 if weight is None else weight.data_ptr(), 0 if mean is None else mean.data_ptr(), rstd.data_ptr(),
                0 if dw is None else dw.data_ptr(), 0 if db is None else db.data_ptr(),
                0 if workspace is None else workspace.data_ptr(), nbytes, m, n, x_code, w_code, stream)
        else:
            fwd_bias = bias if layernorm else None
            if fwd_bias is not None and weight is not None and fwd_bias.dtype != weight.dtype:
                fwd_bias = fwd_bias.to(weight.dtype)
            status = lib.thn_norm_act_bwd(
                x2.data_ptr(), x_stride, d2.data_ptr(), d_stride, dx.data_ptr(), n,
                0 if weight is None else weight.data_ptr(), 0 if fwd_bias is None else fwd_bias.data_ptr(),
                0 if mean is None else mean.data_ptr(), rstd.data_ptr(),
                0 if dw is None else dw.data_ptr(), 0 if db is None else db.data_ptr(),
                0 if workspace is None else workspace.data_ptr(), nbytes, m, n, act, x_code, w_code, stream)
    finally:
        if locked:
            _backward_lock.release()
        if other_device:
            guard.__exit__(None, None, None)
    if status != 0:
        _native.check(status)
    if mixed:
        db = db.to(bias.dtype)
    return (dx.reshape(*x.shape[:-1], n) if reshaped else dx), dw, db


def query_launch(which: int, layernorm: bool, m: int, n: int, dtype: torch.dtype):
    """(vecs_per_thread, threads_per_row, block_threads, grid_blocks, vector_path) the library would use.
    `layernorm` is the flavour within the family `which` names: LayerNorm against RMSNorm (0, 1), log-softmax against
    softmax (2, 3), normalize against the p-norm by itself (4); the activation code too for the epilogue families."""
    shape = (ctypes.c_int32 * 5)()
    _native.check(_native.lib().thn_norm_query_launch(which, int(layernorm), m, n, _native.dtype_code(dtype), shape))
    return tuple(shape)
