"""ctypes front end of ``libnorm_oracle.so`` (oracle/norm_oracle.c) -- TEST INFRASTRUCTURE ONLY.

Same functions as oracle/norm_oracle.py, fast enough for the full benchmark shapes.  Inputs are contiguous
CPU ``torch`` tensors in their storage dtype (float32 / float16 / bfloat16 / float64); results come back as
float64 numpy arrays (``out_dtype=None``) or as tensors of a storage dtype (timing mode).  Only tests,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this module.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libnorm_oracle.so")
_CODES = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2, torch.float64: 3}
_lib = None


def build(force: bool = False) -> str:
    """Compile oracle/norm_oracle.c with gcc (``make -C oracle``)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE, "libnorm_oracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        for name in ("thn_oracle_layernorm_fwd", "thn_oracle_rmsnorm_fwd",
                     "thn_oracle_layernorm_bwd", "thn_oracle_rmsnorm_bwd", "thn_oracle_num_threads"):
            getattr(_lib, name).restype = ctypes.c_int
    return _lib


def num_threads() -> int:
    return int(lib().thn_oracle_num_threads())


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _prep(t):
    if t is None:
        return None
    assert t.device.type == "cpu"
    return t.contiguous()


def _out(shape, out_dtype):
    if out_dtype is None:
        return torch.empty(shape, dtype=torch.float64), 3
    return torch.empty(shape, dtype=out_dtype), _CODES[out_dtype]


def _ret(t, out_dtype):
    return t.numpy() if out_dtype is None else t


def _dp(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def _check(rc):
    if rc != 0:
        raise RuntimeError(f"norm_oracle.c returned {rc}")


def layernorm_fwd(x, weight, bias, eps, out_dtype=None, want_y=True):
    x, weight, bias = _prep(x), _prep(weight), _prep(bias)
    x2 = x.reshape(-1, x.shape[-1])
    m, n = x2.shape
    wd = _CODES[(weight if weight is not None else bias if bias is not None else x).dtype]
    if weight is not None and bias is not None:
        assert weight.dtype == bias.dtype
    y, oc = _out(x.shape if want_y else (0,), out_dtype)
    mean = np.empty(m, dtype=np.float64)
    rstd = np.empty(m, dtype=np.float64)
    _check(lib().thn_oracle_layernorm_fwd(_ptr(x2), _CODES[x.dtype], _ptr(weight), _ptr(bias), wd,
                                          ctypes.c_double(eps), ctypes.c_int64(m), ctypes.c_int64(n),
                                          _ptr(y if want_y else None), oc, _dp(mean), _dp(rstd)))
    return (_ret(y, out_dtype) if want_y else None), mean, rstd


def rmsnorm_fwd(x, weight, eps, out_dtype=None, want_y=True):
    x, weight = _prep(x), _prep(weight)
    x2 = x.reshape(-1, x.shape[-1])
    m, n = x2.shape
    wd = _CODES[(weight if weight is not None else x).dtype]
    y, oc = _out(x.shape if want_y else (0,), out_dtype)
    rstd = np.empty(m, dtype=np.float64)
    _check(lib().thn_oracle_rmsnorm_fwd(_ptr(x2), _CODES[x.dtype], _ptr(weight), wd,
                                        ctypes.c_double(eps), ctypes.c_int64(m), ctypes.c_int64(n),
                                        _ptr(y if want_y else None), oc, _dp(rstd)))
    return (_ret(y, out_dtype) if want_y else None), rstd


def layernorm_bwd(x, dy, weight, mean, rstd, has_bias=True, out_dtype=None, param_dtype=None, want_dx=True):
    x, dy, weight = _prep(x), _prep(dy), _prep(weight)
    assert x.dtype == dy.dtype
    x2 = x.reshape(-1, x.shape[-1])
    m, n = x2.shape
    wd = _CODES[(weight if weight is not None else x).dtype]
    mean = np.ascontiguousarray(np.asarray(mean, dtype=np.float64).reshape(-1))
    rstd = np.ascontiguousarray(np.asarray(rstd, dtype=np.float64).reshape(-1))
    dx, oc = _out(x.shape if want_dx else (0,), out_dtype)
    dw, pc = _out((n,), param_dtype)
    db, _ = _out((n,), param_dtype)
    _check(lib().thn_oracle_layernorm_bwd(_ptr(x2), _ptr(dy), _CODES[x.dtype], _ptr(weight), wd,
                                          _dp(mean), _dp(rstd), ctypes.c_int64(m), ctypes.c_int64(n),
                                          _ptr(dx if want_dx else None), oc,
                                          _ptr(dw if weight is not None else None),
                                          _ptr(db if has_bias else None), pc))
    return (_ret(dx, out_dtype) if want_dx else None, _ret(dw, param_dtype) if weight is not None else None,
            _ret(db, param_dtype) if has_bias else None)


def rmsnorm_bwd(x, dy, weight, rstd, out_dtype=None, param_dtype=None, want_dx=True):
    x, dy, weight = _prep(x), _prep(dy), _prep(weight)
    assert x.dtype == dy.dtype
    x2 = x.reshape(-1, x.shape[-1])
    m, n = x2.shape
    wd = _CODES[(weight if weight is not None else x).dtype]
    rstd = np.ascontiguousarray(np.asarray(rstd, dtype=np.float64).reshape(-1))
    dx, oc = _out(x.shape if want_dx else (0,), out_dtype)
    dw, pc = _out((n,), param_dtype)
    _check(lib().thn_oracle_rmsnorm_bwd(_ptr(x2), _ptr(dy), _CODES[x.dtype], _ptr(weight), wd,
                                        _dp(rstd), ctypes.c_int64(m), ctypes.c_int64(n),
                                        _ptr(dx if want_dx else None), oc,
                                        _ptr(dw if weight is not None else None), pc))
    return (_ret(dx, out_dtype) if want_dx else None), (_ret(dw, param_dtype) if weight is not None else None)
