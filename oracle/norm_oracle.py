"""CPU oracle for the LayerNorm / RMSNorm forward + backward path (TEST INFRASTRUCTURE ONLY).

This file is a checker.  It is imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` and by nothing else: the product path (the ``TritonHub`` package and
``libthnorm.so``) never imports it and has no CPU fallback.

It restates, in float64 numpy, the arithmetic of the reference's four device kernels and of its
second-stage parameter-gradient reduction:

* ``layernorm_fwd``  follows ``TritonHub/Normalization/layernorm.py:31-46``
* ``layernorm_bwd``  follows ``TritonHub/Normalization/layernorm.py:128-153`` and ``:207-208``
* ``rmsnorm_fwd``    follows ``TritonHub/Normalization/rmsnorm.py:28-38``
* ``rmsnorm_bwd``    follows ``TritonHub/Normalization/rmsnorm.py:104-122`` and ``:166``
* ``flatten_rows`` / ``check_feature_dim`` follow the host wrappers ``layernorm.py:49-72`` and
  ``rmsnorm.py:41-58`` (flatten to (M, N); reject rows wider than 64 KiB).

The reference accumulates in float32; the oracle accumulates in float64 and returns float64 so that a result
in any storage dtype can be compared against it in units of that dtype's ulp (``ulp_error``).  Nothing is
rounded inside the oracle.

How the oracle itself is pinned (see tests/test_oracle_pins.py): against the float64 CPU kernels of
``torch.native_layer_norm`` / ``native_layer_norm_backward`` / ``torch.nn.functional.rms_norm`` + autograd,
against the frozen vectors in ``tests/golden/`` (written by ``tests/golden/make_golden.py``), against central
finite differences of its own forward (which would expose a dropped term, a wrong sign or a transposed
operand in the backward), and against closed-form special cases and invariants.  The reference's own tests
hold no golden vectors for this path; they compare with ``torch.nn.LayerNorm`` / ``torch.nn.RMSNorm`` live
(``UnitTests/Normalization/layernorm_unittest.py:16-47``), which is the same library routine used here.
"""
from __future__ import annotations

import numpy as np

# Row-width limit of the reference's launch wrappers (layernorm.py:69-72, rmsnorm.py:55-58).
MAX_FUSED_BYTES = 65536
FEATURE_DIM_MESSAGE = "This layer norm doesn't support feature dim >= 64KB."

# Mantissa bits (excluding the implicit one) and minimum normal exponent of the storage dtypes.
_FORMATS = {
    "fp32": (23, -126),
    "fp16": (10, -14),
    "bf16": (7, -126),
    "fp64": (52, -1022),
}


def _f64(a):
    return None if a is None else np.asarray(a, dtype=np.float64)


def flatten_rows(x):
    """(…, N) -> (M, N), as the launch wrappers do before the kernels run (layernorm.py:51-54)."""
    x = np.asarray(x)
    return x.reshape(-1, x.shape[-1])


def check_feature_dim(n: int, element_size: int) -> None:
    """Raise the reference's RuntimeError when a row exceeds 64 KiB (layernorm.py:69-72)."""
    max_fused = MAX_FUSED_BYTES // element_size
    block = min(max_fused, 1 << max(0, (n - 1).bit_length()))
    if n > block:
        raise RuntimeError(FEATURE_DIM_MESSAGE)


def layernorm_fwd(x, weight, bias, eps):
    """y, mean, rstd of LayerNorm over the last dimension (layernorm.py:31-46).

    mean = sum(x)/N; var = sum((x-mean)^2)/N (biased, two pass); rstd = 1/sqrt(var+eps);
    y = (x-mean)*rstd [*w] [+b].  Returns float64 arrays: y like x, mean and rstd of shape (M,).
    """
    x = _f64(x)
    shape = x.shape
    x2 = flatten_rows(x)
    n = x2.shape[1]
    mean = x2.sum(axis=1) / n
    xbar = x2 - mean[:, None]
    var = (xbar * xbar).sum(axis=1) / n
    rstd = 1.0 / np.sqrt(var + np.float64(eps))
    y = xbar * rstd[:, None]
    if weight is not None:
        y = y * _f64(weight)[None, :]
    if bias is not None:
        y = y + _f64(bias)[None, :]
    return y.reshape(shape), mean, rstd


def layernorm_bwd(x, dy, weight, mean, rstd, has_bias=True):
    """dx, dW, dB of LayerNorm from the SAVED mean/rstd (layernorm.py:128-153, :207-208).

    xhat = (x-mean)*rstd; wdy = w*dy (dy when there is no weight); c1 = sum(xhat*wdy)/N; c2 = sum(wdy)/N;
    dx = (wdy - (xhat*c1 + c2))*rstd; dW = sum over rows of dy*xhat; dB = sum over rows of dy.
    dW is None without weight, dB is None when ``has_bias`` is false.
    """
    x = _f64(x)
    shape = x.shape
    x2 = flatten_rows(x)
    g = flatten_rows(_f64(dy))
    n = x2.shape[1]
    mean = _f64(mean).reshape(-1)
    rstd = _f64(rstd).reshape(-1)
    xhat = (x2 - mean[:, None]) * rstd[:, None]
    wdy = g * _f64(weight)[None, :] if weight is not None else g
    c1 = (xhat * wdy).sum(axis=1) / n
    c2 = wdy.sum(axis=1) / n
    dx = (wdy - (xhat * c1[:, None] + c2[:, None])) * rstd[:, None]
    dw = (g * xhat).sum(axis=0) if weight is not None else None
    db = g.sum(axis=0) if has_bias else None
    return dx.reshape(shape), dw, db


def rmsnorm_fwd(x, weight, eps):
    """y, rstd of RMSNorm over the last dimension (rmsnorm.py:28-38).

    rstd = 1/sqrt(sum(x^2)/N + eps); y = x*rstd [*w].
    """
    x = _f64(x)
    shape = x.shape
    x2 = flatten_rows(x)
    n = x2.shape[1]
    ms = (x2 * x2).sum(axis=1) / n
    rstd = 1.0 / np.sqrt(ms + np.float64(eps))
    y = x2 * rstd[:, None]
    if weight is not None:
        y = y * _f64(weight)[None, :]
    return y.reshape(shape), rstd


def rmsnorm_bwd(x, dy, weight, rstd):
    """dx, dW of RMSNorm from the SAVED rstd (rmsnorm.py:104-122, :166).

    xhat = x*rstd; wdy = w*dy; c1 = sum(xhat*wdy)/N; dx = (wdy - xhat*c1)*rstd; dW = sum over rows of dy*xhat.
    """
    x = _f64(x)
    shape = x.shape
    x2 = flatten_rows(x)
    g = flatten_rows(_f64(dy))
    n = x2.shape[1]
    rstd = _f64(rstd).reshape(-1)
    xhat = x2 * rstd[:, None]
    wdy = g * _f64(weight)[None, :] if weight is not None else g
    c1 = (xhat * wdy).sum(axis=1) / n
    dx = (wdy - xhat * c1[:, None]) * rstd[:, None]
    dw = (g * xhat).sum(axis=0) if weight is not None else None
    return dx.reshape(shape), dw


def ulp(ref, fmt: str):
    """Spacing of the storage format ``fmt`` ('fp32', 'fp16', 'bf16', 'fp64') at |ref| (float64 array)."""
    mant, emin = _FORMATS[fmt]
    a = np.abs(_f64(ref))
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(np.where(a > 0, a, 1.0)))
    e = np.maximum(np.where(a > 0, e, emin), emin)
    return np.exp2(e - mant)


def ulp_error(got, ref, fmt: str):
    """|got - ref| in units of ``fmt``'s ulp at ref.  A correctly rounded result scores <= 0.5."""
    got = _f64(got)
    ref = _f64(ref)
    return np.abs(got - ref) / ulp(ref, fmt)
