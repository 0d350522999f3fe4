"""Host launch wrappers of the row p-norm / normalize operators.

They do on the host what the reference's ``_norm_fwd`` / ``_norm_bwd`` (Ops/norm.py:47-60, :104-126) and
``_normalize_fwd`` / ``_normalize_bwd`` (Ops/normalize.py:35-55, :119-142) do -- contiguity of the last dimension,
shape and dtype assertions with the same messages, output allocation -- and then call the C ABI of libthnorm.so
on the current stream.  The (B, M) tensors cross the boundary as contiguous vectors.
"""
import torch

from .. import _native
from ..Activations._launch import _call


def _rows3d(t: torch.Tensor) -> torch.Tensor:
    """(B, M, K) with unit stride along K and rows that do not overlap; batch and row strides are kept."""
    if t.stride(-1) != 1 or (t.shape[1] > 1 and t.stride(1) < t.shape[2]):
        t = t.contiguous()
    return t


def norm_fwd(x, p=2, eps=1e-6):
    _native.require_gpu(x)
    x = _rows3d(x)
    B, M, K = x.shape
    norms_x = torch.empty((B, M), memory_format=torch.contiguous_format, device=x.device, dtype=x.dtype)
    assert x.stride(-1) == 1, "Output tensors must be contiguous"
    if B * M > 0:
        _call(x.device, 'thn_pnorm_fwd', x.data_ptr(), x.stride(0), x.stride(1), norms_x.data_ptr(),
                B, M, K, float(p), float(eps), _native.dtype_code(x.dtype))
    return norms_x


def norm_bwd(x, norms_x, dout, p=2):
    _native.require_gpu(x)
    norms_x = norms_x.contiguous()
    dout = dout.contiguous()
    B, M = norms_x.shape
    K = x.shape[-1]
    assert x.shape == (B, M, K), "Input shape mismatch"
    assert norms_x.shape == (B, M), "Input gradient shape mismatch"
    assert dout.shape == (B, M), "Output gradient shape mismatch"
    assert x.dtype == norms_x.dtype == dout.dtype, "All tensors must have the same dtype"
    x = _rows3d(x)
    dx = torch.empty((B, M, K), memory_format=torch.contiguous_format, device=norms_x.device, dtype=norms_x.dtype)
    assert dx.stride(-1) == 1, "Output tensors must be contiguous"
    if B * M > 0:
        _call(x.device, 'thn_pnorm_bwd', x.data_ptr(), x.stride(0), x.stride(1), norms_x.data_ptr(),
                dout.data_ptr(), dx.data_ptr(), M * K, K, B, M, K, float(p), _native.dtype_code(x.dtype))
    return dx


def normalize_fwd(x, p=2, eps=1e-6):
    _native.require_gpu(x)
    x = _rows3d(x)
    B, M, K = x.shape
    x_norm = torch.empty((B, M, K), memory_format=torch.contiguous_format, device=x.device, dtype=x.dtype)
    norms_x = torch.empty((B, M), memory_format=torch.contiguous_format, device=x.device, dtype=x.dtype)
    assert x.stride(-1) == 1, "Output tensors must be contiguous"
    if B * M > 0:
        _call(x.device, 'thn_normalize_fwd', x.data_ptr(), x.stride(0), x.stride(1), x_norm.data_ptr(),
                M * K, K, norms_x.data_ptr(), B, M, K, float(p), float(eps), _native.dtype_code(x.dtype))
    return x_norm, norms_x


def normalize_bwd(x, x_norm, norms_x, dout, p=2):
    _native.require_gpu(x_norm)
    x_norm = _rows3d(x_norm)
    norms_x = norms_x.contiguous()
    dout = _rows3d(dout)
    B, M, K = x_norm.shape
    assert dout.shape == (B, M, K), "Output gradient shape mismatch"
    assert x_norm.dtype == norms_x.dtype == dout.dtype, "All tensors must have the same dtype"
    x = _rows3d(x)
    dx = torch.empty((B, M, K), memory_format=torch.contiguous_format, device=x_norm.device, dtype=x_norm.dtype)
    assert dx.stride(-1) == 1, "Output tensors must be contiguous"
    if B * M > 0:
        _call(x_norm.device, 'thn_normalize_bwd', x.data_ptr(), x.stride(0), x.stride(1), x_norm.data_ptr(),
                x_norm.stride(0), x_norm.stride(1), norms_x.data_ptr(), dout.data_ptr(), dout.stride(0),
                dout.stride(1), dx.data_ptr(), M * K, K, B, M, K, float(p), _native.dtype_code(x_norm.dtype))
    return dx
