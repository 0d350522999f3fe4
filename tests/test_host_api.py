"""CPU tests of the host side: the C-ABI library loads and exports what include/thnorm.h declares, its
argument checks answer without a GPU, and the Python modules mirror the reference's operator interface
(TritonHub/Normalization/layernorm.py:211-252, rmsnorm.py:169-204).  Nothing here launches a kernel."""
import ctypes
import os
import re

import pytest
import torch

from conftest import ROOT
from TritonHub import Activations, Normalization, _native
from TritonHub.Normalization import LayerNorm, RMSNorm, _launch
from TritonHub.Normalization.layernorm import layernorm
from TritonHub.Normalization.rmsnorm import rmsnorm

HEADER = os.path.join(ROOT, "include", "thnorm.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(thn_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) == 24 and "thn_norm_set_cache_policy" in names and "thn_norm_bwd_static_workspace" in names and "thn_dropout" in names and "thn_norm_act_fwd" in names and "thn_norm_act_bwd" in names and "thn_act_fwd" in names and "thn_pnorm_fwd" in names and "thn_normalize_bwd" in names and "thn_norm_fwd" in names and "thn_norm_bwd" in names and "thn_softmax_fwd" in names
    handle = ctypes.CDLL(_native.LIB_PATH)
    for name in names:
        assert hasattr(handle, name), f"{name} is declared in include/thnorm.h but not exported"
    assert sorted(_native.SYMBOLS) == names          # the ctypes table binds exactly the declared set


def test_abi_version_and_messages():
    lib = _native.lib()
    version = int(re.search(r"#define THN_ABI_VERSION (\d+)", open(HEADER).read()).group(1))
    assert lib.thn_abi_version() == version
    assert _native.strerror(0) == "ok"
    # the reference's RuntimeError text (layernorm.py:72, rmsnorm.py:58)
    assert _native.strerror(_native.E_FEATURE_DIM) == "This layer norm doesn't support feature dim >= 64KB."
    for code in range(-7, 0):
        assert _native.strerror(code) not in ("", "unknown status")
    assert _native.strerror(-99) == "unknown status"


def test_argument_checks_answer_without_a_gpu():
    lib = _native.lib()
    fwd = lambda m, n, xd, wd=0: lib.thn_norm_fwd(0, n, 0, n, 0, 0, 0, 0, m, n, 1e-5, xd, wd, 0)
    assert fwd(4, 128, 7) == _native.E_DTYPE
    assert fwd(4, 0, 0) == _native.E_SHAPE and fwd(-1, 8, 0) == _native.E_SHAPE
    # 64 KiB row limit per storage type: N <= 16384 (4 bytes), 32768 (2 bytes), 8192 (8 bytes)
    assert fwd(4, 16385, _native.F32) == _native.E_FEATURE_DIM
    assert fwd(4, 32769, _native.BF16) == _native.E_FEATURE_DIM
    assert fwd(4, 8193, _native.F64) == _native.E_FEATURE_DIM
    assert fwd(0, 128, _native.F16) == _native.OK                     # no rows: nothing to do
    assert fwd(4, 128, _native.F16) == _native.E_NULL                 # required pointers are null
    assert lib.thn_norm_bwd_workspace_bytes(4, 128, 1, 1, 9) == _native.E_DTYPE
    assert lib.thn_norm_bwd_workspace_bytes(4, 40000, 1, 1, _native.F16) == _native.E_FEATURE_DIM
    assert lib.thn_norm_bwd_workspace_bytes(4, 128, 0, 0, _native.F32) == 0
    assert lib.thn_norm_bwd_workspace_bytes(0, 128, 1, 1, _native.F32) == 0
    assert lib.thn_norm_set_launch_override(11, 0, 0, 0, 0) == _native.E_SHAPE
    assert lib.thn_norm_set_launch_override(0, 0, 0, 0, 0) == _native.OK
    if not torch.cuda.is_available():
        assert lib.thn_norm_bwd_workspace_bytes(4, 128, 1, 1, _native.F32) == _native.E_DEVICE
    with pytest.raises(RuntimeError, match="doesn't support feature dim >= 64KB"):
        _native.check(_native.E_FEATURE_DIM)
    with pytest.raises(RuntimeError, match="workspace"):
        _native.check(_native.E_WORKSPACE)


def test_cache_policy_switch_and_per_call_flags():
    lib = _native.lib()
    assert lib.thn_norm_get_cache_policy() == 0                              # THN_CACHE_KEEP_X is the default
    assert lib.thn_norm_set_cache_policy(1) == _native.OK and lib.thn_norm_get_cache_policy() == 1
    assert lib.thn_norm_set_cache_policy(2) == _native.E_SHAPE and lib.thn_norm_get_cache_policy() == 1
    assert lib.thn_norm_set_cache_policy(0) == _native.OK and lib.thn_norm_get_cache_policy() == 0
    fwd = lambda xd: lib.thn_norm_fwd(0, 128, 0, 128, 0, 0, 0, 0, 4, 128, 1e-5, xd, 0, 0)
    afwd = lambda xd: lib.thn_norm_act_fwd(0, 128, 0, 128, 0, 0, 0, 0, 4, 128, 1e-5, _native.ACT_SILU, xd, 0, 0)
    for call in (fwd, afwd):
        # the flag rides on the storage code: the code underneath is still checked, then the pointers
        assert call(_native.BF16 | _native.X_STREAM) == _native.E_NULL
        assert call(_native.F32 | _native.X_KEEP) == _native.E_NULL
        assert call(7 | _native.X_STREAM) == _native.E_DTYPE
        assert call(_native.BF16 | _native.X_KEEP | _native.X_STREAM) == _native.E_DTYPE     # both: contradictory
    # no other entry point takes the flags
    assert lib.thn_norm_bwd_workspace_bytes(4, 128, 1, 1, _native.BF16 | _native.X_STREAM) == _native.E_DTYPE
    assert lib.thn_softmax_fwd(0, 128, 0, 128, 4, 128, 0, _native.BF16 | _native.X_STREAM, 0) == _native.E_DTYPE
    # the Python switch
    assert _launch.get_cache_policy() == "auto"
    assert _launch._x_policy_flag(True) == _native.X_KEEP and _launch._x_policy_flag(False) == _native.X_STREAM
    try:
        _launch.set_cache_policy("stream")
        assert _launch._x_policy_flag(True) == _native.X_STREAM
        _launch.set_cache_policy("keep")
        assert _launch._x_policy_flag(False) == _native.X_KEEP
        with pytest.raises(ValueError):
            _launch.set_cache_policy("sometimes")
        assert Normalization.get_cache_policy() == "keep"
    finally:
        _launch.set_cache_policy("auto")
    assert "set_cache_policy" not in Normalization.__all__                    # the reference's surface is unchanged


def test_outputs_that_overlap_inputs_are_refused_on_the_host():
    """The address ranges alone decide: no kernel is launched, so fake addresses do."""
    lib = _native.lib()
    s = 2                                              # bf16
    base, m, n = 1 << 20, 16, 128
    size = m * n * s
    fwd = lambda x, y, ys=n: lib.thn_norm_fwd(x, n, y, ys, 0, 0, 0, 4096, m, n, 1e-5, _native.BF16, 0, 0)
    assert fwd(base, base) == _native.E_SHAPE                                   # in place
    assert fwd(base, base + size - 2) == _native.E_SHAPE                        # last element of x is first of y
    assert fwd(base + size - 2, base) == _native.E_SHAPE
    assert fwd(base, base + n * s, 2 * n) == _native.E_SHAPE                    # different pitches: the ranges decide
    # two column blocks of one buffer (the same pitch, rows that do not touch) may interleave; shifted by less than a row not
    fwd2 = lambda x, y: lib.thn_norm_fwd(x, 2 * n, y, 2 * n, 0, 0, 0, 4096, m, n, 1e-5, _native.BF16, 0, 0)
    assert fwd2(base, base + n * s - 2) == _native.E_SHAPE and fwd2(base + 2, base + n * s) == _native.E_SHAPE
    assert fwd2(base + n * s - 2, base) == _native.E_SHAPE
    if not torch.cuda.is_available():
        assert fwd2(base, base + n * s) == _native.E_DEVICE and fwd2(base + n * s, base) == _native.E_DEVICE
    not_refused = (_native.OK, _native.E_DEVICE, _native.E_LAUNCH)
    if not torch.cuda.is_available():
        assert fwd(base, base + size) == _native.E_DEVICE                       # adjacent is fine: the next check answers
    bwd = lambda x, dy, dx: lib.thn_norm_bwd_dx_partials(x, n, dy, n, dx, n, 0, 0, 4096, 0, 0, 0, 0, None, m, n,
                                                          _native.BF16, 0, 0)
    assert bwd(base, base + size, base) == _native.E_SHAPE and bwd(base, base + size, base + size + 64) == _native.E_SHAPE
    sm = lambda x, y: lib.thn_softmax_fwd(x, n, y, n, m, n, 0, _native.BF16, 0)
    smb = lambda y, dy, dx: lib.thn_softmax_bwd(y, n, dy, n, dx, n, m, n, 0, _native.BF16, 0)
    assert sm(base, base + 2) == _native.E_SHAPE and smb(base, base + size, base + size) == _native.E_SHAPE
    act = lambda x, y: lib.thn_act_fwd(x, n, y, n, m, n, _native.ACT_RELU, 0.0, 0.0, _native.BF16, 0)
    actb = lambda x, g, dx: lib.thn_act_bwd(x, n, g, n, dx, n, m, n, _native.ACT_RELU, 0.0, 0.0, _native.BF16, 0)
    assert act(base, base) == _native.E_SHAPE and actb(base, base + size, base + size) == _native.E_SHAPE
    k = n
    nz = lambda x, y: lib.thn_normalize_fwd(x, m * k, k, y, m * k, k, 4096, 1, m, k, 2.0, 1e-6, _native.BF16, 0)
    assert nz(base, base) == _native.E_SHAPE
    pb = lambda x, dx: lib.thn_pnorm_bwd(x, m * k, k, 4096, 8192, dx, m * k, k, 1, m, k, 2.0, _native.BF16, 0)
    assert pb(base, base + 16) == _native.E_SHAPE
    nb = lambda y, dy, dx: lib.thn_normalize_bwd(0, m * k, k, y, m * k, k, 4096, dy, m * k, k, dx, m * k, k, 1, m, k,
                                                 2.0, _native.BF16, 0)
    assert nb(base, base + size, base + size + 2) == _native.E_SHAPE and nb(base, base + size, base) == _native.E_SHAPE
    if not torch.cuda.is_available():
        for rc in (sm(base, base + size), act(base, base + size), nz(base, base + size), pb(base, base + size)):
            assert rc in not_refused


def test_softmax_argument_checks_answer_without_a_gpu():
    lib = _native.lib()
    fwd = lambda m, n, kind, dt: lib.thn_softmax_fwd(0, n, 0, n, m, n, kind, dt, 0)
    bwd = lambda m, n, kind, dt: lib.thn_softmax_bwd(0, n, 0, n, 0, n, m, n, kind, dt, 0)
    for call in (fwd, bwd):
        assert call(4, 128, 0, 5) == _native.E_DTYPE
        assert call(4, 128, 3, _native.F32) == _native.E_SHAPE           # unknown kind
        assert call(4, 0, 0, _native.F32) == _native.E_SHAPE and call(-2, 8, 0, _native.F32) == _native.E_SHAPE
        assert call(4, 16385, 0, _native.F32) == _native.E_NULL            # no row-width limit: the next check answers
        assert call(4, 2 ** 31, 0, _native.F32) == _native.E_SHAPE         # the row width must fit in 31 bits
        assert call(0, 128, 0, _native.BF16) == _native.OK
        assert call(4, 128, 0, _native.BF16) == _native.E_NULL
    assert (_native.SOFTMAX, _native.SOFTMIN, _native.LOGSOFTMAX) == (0, 1, 2)   # enum thn_softmax_kind


def test_pnorm_argument_checks_answer_without_a_gpu():
    lib = _native.lib()
    fwd = lambda b, m, k, p, eps, dt: lib.thn_pnorm_fwd(0, m * k, k, 0, b, m, k, p, eps, dt, 0)
    nfwd = lambda b, m, k, p, eps, dt: lib.thn_normalize_fwd(0, m * k, k, 0, m * k, k, 0, b, m, k, p, eps, dt, 0)
    bwd = lambda b, m, k, p, dt: lib.thn_pnorm_bwd(0, m * k, k, 0, 0, 0, m * k, k, b, m, k, p, dt, 0)
    nbwd = lambda b, m, k, p, dt: lib.thn_normalize_bwd(0, m * k, k, 0, m * k, k, 0, 0, m * k, k, 0, m * k, k, b, m, k,
                                                       p, dt, 0)
    for call in (fwd, nfwd):
        assert call(2, 3, 8, 2.0, 1e-6, 9) == _native.E_DTYPE
        assert call(2, 3, 0, 2.0, 1e-6, _native.F32) == _native.E_SHAPE and call(-1, 3, 8, 2.0, 1e-6, 0) == _native.E_SHAPE
        assert call(2, 3, 8, 0.5, 1e-6, _native.F32) == _native.E_SHAPE        # p must be in [1, 6] (Ops/norm.py:148)
        assert call(2, 3, 8, 6.5, 1e-6, _native.F32) == _native.E_SHAPE
        assert call(2, 3, 8, float("nan"), 1e-6, _native.F32) == _native.E_SHAPE
        assert call(2, 3, 8, 2.0, -1.0, _native.F32) == _native.E_SHAPE        # eps must be non-negative (:149)
        assert call(0, 3, 8, 2.0, 1e-6, _native.F16) == _native.OK and call(2, 0, 8, 2.0, 1e-6, _native.F16) == _native.OK
        assert call(2, 3, 8, 2.0, 1e-6, _native.BF16) == _native.E_NULL
        assert call(2, 3, 100000, 2.5, 1e-6, _native.F32) == _native.E_NULL    # no row-width limit, any real p
    for call in (bwd, nbwd):
        assert call(2, 3, 8, 2.0, 7) == _native.E_DTYPE
        assert call(2, 3, 8, 7.0, _native.F32) == _native.E_SHAPE
        assert call(2, 0, 8, 2.0, _native.F32) == _native.OK
        assert call(2, 3, 8, 3.0, _native.F32) == _native.E_NULL


def test_act_argument_checks_answer_without_a_gpu():
    lib = _native.lib()
    fwd = lambda m, n, act, dt: lib.thn_act_fwd(0, n, 0, n, m, n, act, 0.0, 0.0, dt, 0)
    bwd = lambda m, n, act, dt: lib.thn_act_bwd(0, n, 0, n, 0, n, m, n, act, 0.0, 0.0, dt, 0)
    for call in (fwd, bwd):
        assert call(4, 128, 0, 6) == _native.E_DTYPE
        assert call(4, 128, 11, _native.F32) == _native.E_SHAPE and call(4, 128, -1, _native.F32) == _native.E_SHAPE
        assert call(4, 0, 0, _native.F32) == _native.E_SHAPE and call(-1, 8, 0, _native.F32) == _native.E_SHAPE
        assert call(0, 128, 3, _native.F16) == _native.OK
        assert call(4, 1 << 20, 3, _native.F32) == _native.E_NULL        # no row-width limit
    assert [_native.ACT_GELU, _native.ACT_GELU_TANH, _native.ACT_SILU, _native.ACT_RELU, _native.ACT_LEAKY_RELU,
            _native.ACT_RELU6, _native.ACT_SIGMOID, _native.ACT_TANH, _native.ACT_MISH, _native.ACT_SOFTPLUS,
            _native.ACT_THRESHOLD] == list(range(11))                   # enum thn_act
    header = open(HEADER).read()
    for i, name in enumerate(["GELU", "GELU_TANH", "SILU", "RELU", "LEAKY_RELU", "RELU6", "SIGMOID", "TANH", "MISH",
                              "SOFTPLUS", "THRESHOLD"]):
        assert re.search(rf"THN_ACT_{name} = {i}\b", header)


def test_activation_callables_match_the_reference_constructors():
    A = Activations
    assert A.GeLU().approximate == "none" and A.GeLU("tanh").gelu_fn is not None        # gelu.py:122-127
    with pytest.raises(AssertionError, match="GeLU approximate must be either none or tanh"):
        A.GeLU("fast")
    assert A.LeakyReLU().negative_slope == 0.01 and A.LeakyReLU(0.2).leakyrelu_fn is not None     # leaky_relu.py:100-102
    sp = A.Softplus()
    assert (sp.beta, sp.threshold) == (1.0, 20) and sp.softplus_fn is not None         # softplus.py:105-108
    th = A.Threshold(0.5, -1.0)
    assert (th.threshold, th.value) == (0.5, -1.0) and th.threshold_fn is not None     # threshold.py:103-106
    with pytest.raises(TypeError):
        A.Threshold()                                                                  # both arguments are required
    for cls, attr in ((A.SiLU, "silu_fn"), (A.ReLU, "relu_fn"), (A.ReLU6, "relu6_fn"), (A.Sigmoid, "sigmoid_fn"),
                      (A.Tanh, "tanh_fn"), (A.Mish, "mish_fn")):
        assert getattr(cls(), attr) is not None
    x = torch.randn(3, 16)
    for mod in (A.GeLU(), A.GeLU("tanh"), A.SiLU(), A.ReLU(), A.LeakyReLU(), A.ReLU6(), A.Sigmoid(), A.Tanh(), A.Mish(),
                A.Softplus(), A.Threshold(0.1, 0.0)):
        with pytest.raises(RuntimeError, match="no CPU fallback"):
            mod(x)


def test_fused_norm_activation_surface_and_argument_checks():
    from TritonHub.Normalization.fused import ACTIVATIONS, LayerNormActivation, RMSNormActivation
    lib = _native.lib()
    fwd = lambda m, n, act, xd: lib.thn_norm_act_fwd(0, n, 0, n, 0, 0, 0, 0, m, n, 1e-5, act, xd, 0, 0)
    bwd = lambda m, n, act, xd: lib.thn_norm_act_bwd(0, n, 0, n, 0, n, 0, 0, 0, 0, 0, 0, 0, 0, m, n, act, xd, 0, 0)
    for call in (fwd, bwd):
        for act in (-1, _native.ACT_LEAKY_RELU, _native.ACT_SIGMOID, _native.ACT_THRESHOLD, 11):
            assert call(4, 128, act, _native.F32) == _native.E_SHAPE        # only gelu, gelu_tanh, silu, relu ride along
        assert call(4, 128, _native.ACT_GELU, 9) == _native.E_DTYPE
        assert call(4, 32769, _native.ACT_SILU, _native.BF16) == _native.E_FEATURE_DIM
        assert call(0, 128, _native.ACT_RELU, _native.F16) == _native.OK
        assert call(4, 128, _native.ACT_GELU_TANH, _native.F16) == _native.E_NULL
    assert lib.thn_norm_act_bwd_workspace_bytes(4, 128, 1, 1, _native.ACT_MISH, _native.F32) == _native.E_SHAPE
    assert lib.thn_norm_act_bwd_workspace_bytes(4, 128, 0, 0, _native.ACT_GELU, _native.F32) == 0
    assert lib.thn_norm_act_bwd_workspace_bytes(4, 128, 1, 1, _native.ACT_GELU, 8) == _native.E_DTYPE
    assert ACTIVATIONS == {"gelu": 0, "gelu_tanh": 1, "silu": 2, "relu": 3}
    m = LayerNormActivation(48, "gelu_tanh", eps=1e-3, bias=False, dtype=torch.bfloat16)
    assert isinstance(m, LayerNorm) and (m.dim, m.eps, m.activation, m.act) == (48, 1e-3, "gelu_tanh", 1)
    assert m.bias is None and m.weight.dtype == torch.bfloat16
    assert list(m.state_dict()) == list(LayerNorm(48, bias=False).state_dict())
    r = RMSNormActivation(64)
    assert isinstance(r, RMSNorm) and (r.activation, r.act, r.eps) == ("silu", 2, 1e-5) and r.bias is None
    with pytest.raises(AssertionError, match="activation must be one of"):
        LayerNormActivation(8, "mish")
    for mod in (m, r):
        with pytest.raises(RuntimeError, match="no CPU fallback"):
            mod(torch.randn(2, mod.dim, dtype=mod.weight.dtype))
    assert Normalization.__all__ == ["LayerNorm", "RMSNorm"]          # the reference's surface is unchanged


def test_ops_surface_matches_the_reference():
    from TritonHub import Ops
    from TritonHub.Ops.norm import Norm
    from TritonHub.Ops.normalize import Normalize
    assert Ops.__all__ == ["normalize", "norm"]                     # Ops/__init__.py:2-5 without bmm
    assert issubclass(Norm, torch.autograd.Function) and issubclass(Normalize, torch.autograd.Function)
    n = Ops.norm()
    assert (n.p, n.eps) == (2, 1e-6) and n.norm is not None           # Ops/norm.py:147-152
    z = Ops.normalize(p=3, eps=0.0)
    assert (z.p, z.eps) == (3, 0.0) and z.normalize is not None       # Ops/normalize.py:163-168
    for cls in (Ops.norm, Ops.normalize):
        with pytest.raises(AssertionError, match=r"p must be in \[1, 6\] for numerical stability"):
            cls(p=0.5)
        with pytest.raises(AssertionError, match=r"p must be in \[1, 6\]"):
            cls(p=7)
        with pytest.raises(AssertionError, match="eps must be non-negative"):
            cls(eps=-1e-3)
    for op in (n, z):
        with pytest.raises(AssertionError, match="Expected Tensor to be 3D"):
            op(torch.randn(4, 8))
        with pytest.raises(RuntimeError, match="no CPU fallback"):
            op(torch.randn(2, 4, 8))


def test_no_cpu_fallback():
    x = torch.randn(4, 32)
    for mod in (LayerNorm(32), RMSNorm(32), Activations.Softmax(), Activations.Softmin(), Activations.LogSoftmax()):
        with pytest.raises(RuntimeError, match="no CPU fallback"):
            mod(x)


def test_package_surface():
    assert Normalization.__all__ == ["LayerNorm", "RMSNorm"]
    assert issubclass(layernorm, torch.autograd.Function) and issubclass(rmsnorm, torch.autograd.Function)
    import TritonHub
    assert TritonHub.__version__ == "1.1.1"
    # the row-reduction activations of TritonHub/Activations/__init__.py (softmax.py:99-103, softmin.py:99-103,
    # logsoftmax.py:106-110): plain callables holding the Function's apply
    assert Activations.__all__ == ['GeLU', 'SiLU', 'ReLU', 'LeakyReLU', 'Softmax', 'Softplus', 'Tanh', 'Softmin', 'Sigmoid',
                                   'Mish', 'ReLU6', 'Threshold', 'LogSoftmax']      # Activations/__init__.py:15
    from TritonHub.Activations.logsoftmax import logsoftmax
    from TritonHub.Activations.softmax import softmax
    from TritonHub.Activations.softmin import softmin
    for fn in (softmax, softmin, logsoftmax):
        assert issubclass(fn, torch.autograd.Function)
    assert Activations.Softmax().softmax_fn is not None and Activations.Softmin().softmin_fn is not None
    assert Activations.LogSoftmax().logsoftmax_fn is not None


def test_dropout_surface_and_argument_checks_answer_without_a_gpu():
    """Layers/dropout.py:95-119: the Function takes (input, p, training) and keeps (p, seed, training); the module is
    Dropout(p=0.5) and follows train() / eval().  The C entry point checks its arguments before it needs a device."""
    import random
    from TritonHub import Layers
    from TritonHub.Layers.dropout import dropout
    assert Layers.__all__ == ["Dropout"] and issubclass(dropout, torch.autograd.Function)
    mod = Layers.Dropout()
    assert mod.p == 0.5 and mod.training and mod.dropout_fn is not None and not list(mod.parameters())
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        mod(torch.randn(4, 8))
    # the seed comes from Python's `random`, one draw per forward call, also when nothing is dropped
    random.seed(5)
    random.randint(0, 2 ** 16)
    second = random.randint(0, 2 ** 16)
    random.seed(5)
    with pytest.raises(RuntimeError):
        mod(torch.randn(2, 2))
    assert random.randint(0, 2 ** 16) == second
    lib = _native.lib()
    buf = (ctypes.c_float * 16)()
    addr = ctypes.addressof(buf)
    assert lib.thn_dropout(addr, addr, 16, 0, 0.5, 1, 9, None) == _native.E_DTYPE
    assert lib.thn_dropout(addr, addr, -1, 0, 0.5, 1, _native.F32, None) == _native.E_SHAPE
    assert lib.thn_dropout(addr, addr, 16, -1, 0.5, 1, _native.F32, None) == _native.E_SHAPE
    assert lib.thn_dropout(addr, addr, 16, 0, 1.5, 1, _native.F32, None) == _native.E_SHAPE
    assert lib.thn_dropout(addr, addr, 16, 0, float("nan"), 1, _native.F32, None) == _native.E_SHAPE
    assert lib.thn_dropout(0, 0, 0, 0, 0.5, 1, _native.F32, None) == 0                  # nothing to do
    assert lib.thn_dropout(0, addr, 16, 0, 0.5, 1, _native.F32, None) == _native.E_NULL
    assert lib.thn_dropout(addr + 2, addr, 8, 0, 0.5, 1, _native.F32, None) == _native.E_SHAPE     # element alignment


@pytest.mark.parametrize("affine,bias", [(True, True), (True, False), (False, True), (False, False)])
def test_layernorm_module_matches_reference_constructor(affine, bias):
    m = LayerNorm(48, eps=1e-3, elementwise_affine=affine, bias=bias, dtype=torch.bfloat16)
    assert (m.dim, m.eps, m.elementwise_affine) == (48, 1e-3, affine)
    assert m.layernorm_fn is not None
    if affine:
        assert m.weight.shape == (48,) and m.weight.dtype == torch.bfloat16 and bool((m.weight == 1).all())
        if bias:
            assert m.bias.shape == (48,) and bool((m.bias == 0).all())
        else:
            assert m.bias is None
    else:
        assert m.weight is None and m.bias is None          # bias needs elementwise_affine (layernorm.py:232-240)
    ref = torch.nn.LayerNorm(48, eps=1e-3, elementwise_affine=affine, bias=bias, dtype=torch.bfloat16)
    assert list(m.state_dict().keys()) == list(ref.state_dict().keys())
    assert [n for n, _ in m.named_parameters()] == [n for n, _ in ref.named_parameters()]
    ref.load_state_dict(m.state_dict())
    m.load_state_dict(ref.state_dict())


@pytest.mark.parametrize("affine", [True, False])
def test_rmsnorm_module_matches_reference_constructor(affine):
    m = RMSNorm(64, eps=1e-6, elementwise_affine=affine, dtype=torch.float16)
    assert (m.dim, m.eps, m.elementwise_affine) == (64, 1e-6, affine)
    assert m.bias is None and "bias" in m._parameters           # always registered as None (rmsnorm.py:194)
    assert m.rmsnorm_fn is not None
    if affine:
        assert m.weight.shape == (64,) and m.weight.dtype == torch.float16 and bool((m.weight == 1).all())
    else:
        assert m.weight is None
    ref = torch.nn.RMSNorm(64, eps=1e-6, elementwise_affine=affine, dtype=torch.float16)
    assert list(m.state_dict().keys()) == list(ref.state_dict().keys())
    m.load_state_dict(ref.state_dict())


def test_default_arguments():
    m = LayerNorm(8)
    assert m.eps == 1e-5 and m.elementwise_affine and m.bias is not None and m.weight.dtype == torch.float32
    r = RMSNorm(8)
    assert r.eps == 1e-5 and r.elementwise_affine
    m.weight.data.fill_(3.0); m.bias.data.fill_(2.0)
    m.reset_parameters()
    assert bool((m.weight == 1).all()) and bool((m.bias == 0).all())


def test_host_wrapper_helpers():
    # flatten to (M, N) with unit column stride, as layernorm.py:49-53 does
    x = torch.randn(3, 5, 16)
    assert _launch._rows(x, "input").shape == (15, 16)
    xt = torch.randn(16, 15).t()                      # last stride != 1 -> made contiguous
    r = _launch._rows(xt, "input")
    assert r.stride(-1) == 1 and torch.equal(r, xt)
    sl = torch.randn(6, 64)[:, :32]                   # row stride 64 is kept, not copied
    r = _launch._rows(sl, "input")
    assert r.stride(0) == 64 and r.data_ptr() == sl.data_ptr()
    ex = torch.randn(1, 16).expand(4, 16)             # broadcast rows are materialised
    assert _launch._rows(ex, "input").stride(0) == 16
    with pytest.raises(AssertionError, match=r"expect weight to have shape \(N,\)"):
        _launch._param(torch.ones(7), 8, "weight")
    with pytest.raises(AssertionError, match=r"expect bias to have shape \(N,\)"):
        _launch._param(torch.ones(2, 8), 8, "bias")
    assert _launch._param(None, 8, "weight") is None
    with pytest.raises(RuntimeError, match="doesn't support feature dim >= 64KB"):
        _launch._check_feature_dim(16385, 4)
    _launch._check_feature_dim(16384, 4)
    with pytest.raises(TypeError, match="unsupported dtype"):
        _native.dtype_code(torch.int32)
