"""ctypes binding of ``libthnorm.so`` -- the only way the Python layer reaches the GPU.

There is no fallback: if the shared library is missing or a call fails, an exception is raised.  The
library is built by ``triton-hub_amd/csrc/Makefile`` (``python __graft_entry__.py`` at the repository
root drives it) and lives next to this file.
"""
from __future__ import annotations

import ctypes
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'libthnorm.so')

F32, F16, BF16, F64 = 0, 1, 2, 3
SOFTMAX, SOFTMIN, LOGSOFTMAX = 0, 1, 2
(ACT_GELU, ACT_GELU_TANH, ACT_SILU, ACT_RELU, ACT_LEAKY_RELU, ACT_RELU6, ACT_SIGMOID, ACT_TANH, ACT_MISH, ACT_SOFTPLUS,
 ACT_THRESHOLD) = range(11)
DTYPE_CODES = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16, torch.float64: F64}

# or-ed into the x_dtype argument of thn_norm_fwd / thn_norm_act_fwd: this call's cache policy for its read of x
X_KEEP, X_STREAM = 0x100, 0x200

OK = 0
E_DTYPE, E_FEATURE_DIM, E_NULL, E_SHAPE, E_WORKSPACE, E_LAUNCH, E_DEVICE = -1, -2, -3, -4, -5, -6, -7

# Every symbol include/thnorm.h declares: (restype, argtypes).
_vp, _i64, _i32, _f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
SYMBOLS = {
    'thn_abi_version': (_i32, []),
    'thn_strerror': (ctypes.c_char_p, [_i32]),
    'thn_norm_fwd': (_i32, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _f32, _i32, _i32, _vp]),
    'thn_norm_bwd_workspace_bytes': (_i64, [_i64, _i64, _i32, _i32, _i32]),
    'thn_norm_bwd': (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64,
                            _i32, _i32, _vp]),
    'thn_norm_bwd_static_workspace': (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _vp]),
    'thn_norm_bwd_dx_partials': (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _i32, _i32, _vp, _i64,
                                        ctypes.POINTER(ctypes.c_int32), _i64, _i64, _i32, _i32, _vp]),
    'thn_norm_bwd_reduce_partials': (_i32, [_vp, ctypes.c_int32, _vp, _vp, _i64, _i32, _vp]),
    'thn_softmax_fwd': (_i32, [_vp, _i64, _vp, _i64, _i64, _i64, _i32, _i32, _vp]),
    'thn_softmax_bwd': (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _i32, _i32, _vp]),
    'thn_pnorm_fwd': (_i32, [_vp, _i64, _i64, _vp, _i64, _i64, _i64, _f32, _f32, _i32, _vp]),
    'thn_normalize_fwd': (_i32, [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _i64, _f32, _f32, _i32, _vp]),
    'thn_pnorm_bwd': (_i32, [_vp, _i64, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _f32, _i32, _vp]),
    'thn_normalize_bwd': (_i32, [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _vp, _i64, _i64, _vp, _i64, _i64,
                                 _i64, _i64, _i64, _f32, _i32, _vp]),
    'thn_act_fwd': (_i32, [_vp, _i64, _vp, _i64, _i64, _i64, _i32, _f32, _f32, _i32, _vp]),
    'thn_act_bwd': (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _i32, _f32, _f32, _i32, _vp]),
    'thn_norm_act_fwd': (_i32, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _f32, _i32, _i32, _i32, _vp]),
    'thn_norm_act_bwd_workspace_bytes': (_i64, [_i64, _i64, _i32, _i32, _i32, _i32]),
    'thn_norm_act_bwd': (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64,
                                _i32, _i32, _i32, _vp]),
    'thn_dropout': (_i32, [_vp, _vp, _i64, _i64, _f32, ctypes.c_uint64, _i32, _vp]),
    'thn_norm_set_launch_override': (_i32, [_i32, _i32, _i32, _i32, _i32]),
    'thn_norm_set_cache_policy': (_i32, [_i32]),
    'thn_norm_get_cache_policy': (_i32, []),
    'thn_norm_query_launch': (_i32, [_i32, _i32, _i64, _i64, _i32, ctypes.POINTER(ctypes.c_int32)]),
}

_lib = None
_lock = threading.Lock()


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise RuntimeError(
                        f'{LIB_PATH} is missing: build the HIP extension first '
                        '(make -C triton-hub_amd/csrc, or __graft_entry__.build()). There is no CPU fallback.')
                handle = ctypes.CDLL(LIB_PATH)
                for name, (restype, argtypes) in SYMBOLS.items():
                    fn = getattr(handle, name)
                    fn.restype = restype
                    fn.argtypes = argtypes
                _lib = handle
    return _lib


def strerror(status: int) -> str:
    return lib().thn_strerror(status).decode()


def check(status: int) -> None:
    """Map a status code to the exception the reference raises for the same condition."""
    if status == OK:
        return
    message = strerror(status)
    if status == E_FEATURE_DIM:
        raise RuntimeError(message)           # layernorm.py:71-72 / rmsnorm.py:57-58 of the reference
    raise RuntimeError(f'libthnorm: {message} (status {status})')


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return DTYPE_CODES[dtype]
    except KeyError:
        raise TypeError(f'unsupported dtype {dtype}: expected float32, float16, bfloat16 or float64') from None


def ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


def require_gpu(t: torch.Tensor) -> None:
    if not t.is_cuda:
        raise RuntimeError('this TritonHub build runs on the GPU only: got a tensor on '
                           f'{t.device}. There is no CPU fallback.')

