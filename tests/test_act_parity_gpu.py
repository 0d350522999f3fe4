"""GPU parity tests of the element-wise activations: the HIP path, called through the operator interface and the
C ABI, against the float64 CPU oracle on the same seeded inputs.

Tolerances: float32 storage max(1e-5, 4 float32 ulp); float16 / bfloat16 1 ulp of the output type plus
4 * 2^-24 * scale, scale being the magnitude of the float32 intermediates (1 + exp(..), 1 + erf(..), ...) whose
rounding the 16-bit result inherits; float64 storage: bit-exact for the selections (ReLU, ReLU6, LeakyReLU,
Threshold), 1e-13 for Softplus (all computed in float64, as the reference does), the float32 bound for the
kernels the reference widens to float32.  The backward is compared at the tensor the Function saved.
"""
import numpy as np
import pytest
import torch
import torch.nn as nn

from conftest import check_elementwise, f64
from oracle import act_oracle as ao
from TritonHub import Activations as A
from TritonHub import _native

pytestmark = pytest.mark.gpu

F32 = lambda v: float(np.float32(v))
SPECS = {
    # name: (callable factory, torch module factory, p0, p1)
    "gelu": (lambda: A.GeLU(), lambda: nn.GELU(), 0.0, 0.0),
    "gelu_tanh": (lambda: A.GeLU("tanh"), lambda: nn.GELU(approximate="tanh"), 0.0, 0.0),
    "silu": (lambda: A.SiLU(), lambda: nn.SiLU(), 0.0, 0.0),
    "relu": (lambda: A.ReLU(), lambda: nn.ReLU(), 0.0, 0.0),
    "leaky_relu": (lambda: A.LeakyReLU(0.01), lambda: nn.LeakyReLU(0.01), F32(0.01), 0.0),
    "relu6": (lambda: A.ReLU6(), lambda: nn.ReLU6(), 0.0, 0.0),
    "sigmoid": (lambda: A.Sigmoid(), lambda: nn.Sigmoid(), 0.0, 0.0),
    "tanh": (lambda: A.Tanh(), lambda: nn.Tanh(), 0.0, 0.0),
    "mish": (lambda: A.Mish(), lambda: nn.Mish(), 0.0, 0.0),
    "softplus": (lambda: A.Softplus(1.0, 20), lambda: nn.Softplus(1.0, 20), 1.0, 20.0),
    "threshold": (lambda: A.Threshold(0.1, 20.0), lambda: nn.Threshold(0.1, 20.0), F32(0.1), 20.0),
}
CODE = {n: i for i, n in enumerate(["gelu", "gelu_tanh", "silu", "relu", "leaky_relu", "relu6", "sigmoid", "tanh", "mish",
                                    "softplus", "threshold"])}
LOADED_TYPE = {"relu", "leaky_relu", "relu6", "softplus", "threshold"}
NAMES = list(SPECS)


def announce(msg):
    print(f"\n[case] {msg}", flush=True)


def check(got, ref, scale, dtype, name, what):
    if dtype == torch.float64 and name in LOADED_TYPE:
        got = f64(got)
        if name == "softplus":
            assert (np.abs(got - ref) <= 1e-13 * np.maximum(1.0, np.abs(ref))).all(), f"{what}: float64 softplus"
        else:
            assert np.array_equal(got, ref), f"{what}: float64 {name} must be bit-exact"
        return
    check_elementwise(f64(got), ref, scale, dtype, what)


def run_and_compare(name, x, dy, what, module=None, x_gpu=None, dy_gpu=None):
    factory, _, p0, p1 = SPECS[name]
    mod = module if module is not None else factory()
    dtype = x.dtype
    xg = (x.cuda() if x_gpu is None else x_gpu).requires_grad_(True)
    y = mod(xg)
    y.backward(dy.cuda() if dy_gpu is None else dy_gpu)
    torch.cuda.synchronize()
    assert y.dtype == dtype and y.shape == x.shape and xg.grad.dtype == dtype and xg.grad.shape == x.shape
    x64, g64 = f64(x), f64(dy)
    y_ref = ao.fwd(name, x64, p0, p1)
    check(y, y_ref, 1.0 + np.abs(x64), dtype, name, f"{what} y")
    saved = f64(y) if name in ao.SAVES_OUTPUT else x64
    dx_ref = ao.bwd(name, saved, g64, p0, p1)
    check(xg.grad, dx_ref, np.abs(g64) * (2.0 + np.abs(x64)), dtype, name, f"{what} dx")
    return y.detach(), xg.grad


def make(shape, dtype, seed, scale=3.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype), torch.randn(shape, generator=g).to(dtype)


# ---- the reference's unit-test matrix (UnitTests/Activations/*_unittest.py: B, N, M = 1, 256, 256; D 32..2048) ---
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.float64])
@pytest.mark.parametrize("name", NAMES)
def test_reference_unit_test_matrix(name, dtype):
    factory, torch_factory, _, _ = SPECS[name]
    rtol, atol = (3e-4, 1e-3) if dtype == torch.float32 else (5e-3, 1e-2)       # gelu_unittest.py:30-32
    if dtype == torch.float16:
        rtol, atol = 1e-2, 5e-2
    for dim in (32, 64, 128, 256, 512, 1024, 2048):
        announce(f"reference matrix {name} D={dim} {dtype}")
        torch.manual_seed(42)
        data = torch.randn(1, 256, 256, dim, device="cuda", dtype=dtype)
        a = data.clone().requires_grad_(True)
        r = data.clone().requires_grad_(True)
        ya, yr = factory()(a), torch_factory()(r)
        assert torch.allclose(ya, yr, atol=atol, rtol=rtol), "Error in forward pass"
        g = torch.randn_like(ya)
        ya.backward(g); yr.backward(g)
        assert torch.allclose(a.grad, r.grad, atol=atol, rtol=rtol), "Error in backward pass"
        run_and_compare(name, data[0, :8].cpu(), g[0, :8].cpu(), f"{name} D={dim} {dtype}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize("name", NAMES)
def test_sizes_tails_and_wide_rows(name, dtype):
    """Total element counts that leave every possible tail behind the 16-byte vectors, tensors smaller than one
    vector, one workgroup step, several grid steps, and a row far wider than 64 KiB."""
    for shape in ((1,), (3,), (1, 7), (5, 9), (37, 33), (2, 3, 257), (64, 1000), (3, 40001), (1, 300007), (2048, 1024)):
        announce(f"{name} {dtype} shape={shape}")
        x, dy = make(shape, dtype, seed=sum(shape))
        run_and_compare(name, x, dy, f"{name} {shape} {dtype}")


@pytest.mark.parametrize("name", NAMES)
def test_parameters_and_special_values(name):
    """Non-default parameters, zeros of both signs, the comparison boundaries, large magnitudes (no NaN where the
    function is finite), infinities."""
    announce(f"special values {name}")
    special = torch.tensor([0.0, -0.0, 1e-30, -1e-30, 6.0, 5.9999995, 20.0, 20.000002, 0.1, 0.099999994, 0.5, 88.0, -88.0,
                            104.0, -104.0, 200.0, -200.0, 1e4, -1e4, 3e38, -3e38])
    x = torch.cat([special, torch.linspace(-30, 30, 1003)])
    dy = torch.linspace(-2, 2, x.numel())
    y, dx = run_and_compare(name, x, dy, f"{name} special")
    assert bool(torch.isfinite(y).all()) and bool(torch.isfinite(dx).all())
    if name == "leaky_relu":
        for slope in (0.0, 0.3, 1.0):
            run_and_compare_params("leaky_relu", A.LeakyReLU(slope), x, dy, F32(slope), 0.0)
    if name == "softplus":
        for beta, thr in ((0.5, 5.0), (3.0, 20.0), (1.0, 0.0)):
            run_and_compare_params("softplus", A.Softplus(beta, thr), x, dy, F32(beta), F32(thr))
    if name == "threshold":
        for thr, val in ((-1.0, 3.5), (0.0, 0.0), (6.0, -7.25)):
            run_and_compare_params("threshold", A.Threshold(thr, val), x, dy, F32(thr), F32(val))
    inf = torch.tensor([float("inf"), -float("inf")], device="cuda")
    yi = SPECS[name][0]()(inf)
    expect = {"relu": [float("inf"), 0.0], "relu6": [6.0, 0.0], "sigmoid": [1.0, 0.0], "tanh": [1.0, -1.0],
              "softplus": [float("inf"), 0.0], "threshold": [float("inf"), 20.0]}.get(name)
    if expect is not None:
        assert yi.tolist() == expect


def run_and_compare_params(name, module, x, dy, p0, p1):
    saved = SPECS[name]
    SPECS[name] = (saved[0], saved[1], p0, p1)
    try:
        run_and_compare(name, x, dy, f"{name} p0={p0} p1={p1}", module=module)
    finally:
        SPECS[name] = saved


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64])
@pytest.mark.parametrize("name", ["gelu", "relu", "sigmoid", "softplus"])
def test_strides_views_and_batch_shapes(name, dtype):
    announce(f"act strides {name} {dtype}")
    g = torch.Generator().manual_seed(12)
    base = (torch.randn(40, 640, generator=g) * 2).to(dtype)
    gbase = torch.randn(40, 640, generator=g).to(dtype)
    bg, gg = base.cuda(), gbase.cuda()
    for i, view in enumerate((lambda t: t[:, :512], lambda t: t[:, 3:515], lambda t: t[::2, 64:576], lambda t: t.t()[:600, :32],
                              lambda t: t[:, :512].reshape(5, 8, 512), lambda t: t[0, 1:512], lambda t: t[:, 5:6],
                              lambda t: t[3:4].expand(6, 640), lambda t: t.reshape(-1)[1:-2])):
        xv, gv = view(base), view(gbase)
        y, dx = run_and_compare(name, xv.contiguous(), gv.contiguous(), f"{name} view {i}", x_gpu=view(bg).detach(),
                                dy_gpu=view(gg))
        assert y.is_contiguous() and dx.is_contiguous()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
def test_large_strided_and_misaligned_views(dtype):
    """Views that take the strided kernel with many rows per workgroup and several steps along a row: ragged and
    misaligned wide rows, every third row, rows of a few elements."""
    g = torch.Generator().manual_seed(14)
    for rows, width, view in ((1500, 2077, lambda t: t[:, 3:2070]), (1500, 2077, lambda t: t[::3, :2048]),
                              (1500, 2077, lambda t: t[:, 1:2]), (60000, 24, lambda t: t[:, 1:20]),
                              (7, 70001, lambda t: t[:, 2:69999])):
        base = (torch.randn(rows, width, generator=g) * 2).to(dtype)
        gbase = torch.randn(rows, width, generator=g).to(dtype)
        bg, gg = base.cuda(), gbase.cuda()
        for name in ("silu", "relu"):
            announce(f"act large views {name} {dtype} {rows}x{width}")
            xv, gv = view(base), view(gbase)
            run_and_compare(name, xv.contiguous(), gv.contiguous(), f"{name} large view {rows}x{width}",
                            x_gpu=view(bg).detach(), dy_gpu=view(gg))


def test_empty_inputs():
    announce("act empty")
    for name in NAMES:
        mod = SPECS[name][0]()
        for shape in ((0, 64), (2, 0, 8)):          # a zero-width last dimension fails in the reference's reshape too
            x = torch.empty(shape, device="cuda", requires_grad=True)
            y = mod(x)
            y.sum().backward()
            assert y.shape == shape and x.grad.shape == shape


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_properties_at_large_size(dtype):
    """Size-independent properties on 2^28 elements: determinism; ReLU, ReLU6 and Threshold are exact selections
    and idempotent; LeakyReLU(1) is the identity; sigmoid(-x) = 1 - sigmoid(x) and tanh(-x) = -tanh(x) hold to
    rounding; every output element is written exactly once (a poisoned output buffer comes back fully defined)."""
    announce(f"act properties {dtype}")
    g = torch.Generator(device="cuda").manual_seed(9)
    x = (torch.randn(65536, 4096, device="cuda", generator=g) * 3).to(dtype)
    relu, relu6 = A.ReLU(), A.ReLU6()
    y = relu(x)
    assert torch.equal(y, torch.clamp_min(x, 0)) and torch.equal(relu(y), y) and torch.equal(relu(x), y)
    assert torch.equal(relu6(x), torch.clamp(x, 0, 6)) and torch.equal(relu6(relu6(x)), relu6(x))
    assert torch.equal(A.LeakyReLU(1.0)(x), x)
    assert torch.equal(A.Threshold(-1e30, 0.0)(x), x)
    assert torch.equal(A.Tanh()(-x), -A.Tanh()(x))
    s, sn = A.Sigmoid()(x).float(), A.Sigmoid()(-x).float()
    assert float((s + sn - 1).abs().max()) <= (3e-7 if dtype == torch.float32 else 8e-3)
    assert bool(torch.isfinite(A.GeLU()(x)).all())


def test_c_abi_direct_calls_and_errors():
    announce("act C ABI direct")
    lib = _native.lib()
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(31)
    m, n, pitch = 77, 300, 384
    xb = (torch.randn(m, pitch, generator=g) * 3).cuda()
    gb = torch.randn(m, pitch, generator=g).cuda()
    for name in NAMES:
        _, _, p0, p1 = SPECS[name]
        y = torch.full((m, pitch), 7.0, device="cuda"); dx = torch.full((m, pitch), 7.0, device="cuda")
        assert lib.thn_act_fwd(xb.data_ptr(), pitch, y.data_ptr(), pitch, m, n, CODE[name], p0, p1, _native.F32, st) == 0
        saved = y if name in ao.SAVES_OUTPUT else xb
        assert lib.thn_act_bwd(saved.data_ptr(), pitch, gb.data_ptr(), pitch, dx.data_ptr(), pitch, m, n, CODE[name], p0, p1,
                               _native.F32, st) == 0
        torch.cuda.synchronize()
        assert bool((y[:, n:] == 7.0).all()) and bool((dx[:, n:] == 7.0).all())          # padding untouched
        x64 = f64(xb[:, :n])
        check_elementwise(f64(y[:, :n]), ao.fwd(name, x64, p0, p1), 1.0 + np.abs(x64), torch.float32, f"C ABI {name} y")
        sv = f64(y[:, :n]) if name in ao.SAVES_OUTPUT else x64
        check_elementwise(f64(dx[:, :n]), ao.bwd(name, sv, f64(gb[:, :n]), p0, p1), 1.0, torch.float32, f"C ABI {name} dx")
    y = torch.empty(m, n, device="cuda")
    assert lib.thn_act_fwd(xb.data_ptr(), n - 1, y.data_ptr(), n, m, n, 0, 0.0, 0.0, _native.F32, st) == _native.E_SHAPE
    assert lib.thn_act_fwd(xb.data_ptr(), pitch, 0, n, m, n, 0, 0.0, 0.0, _native.F32, st) == _native.E_NULL
    assert lib.thn_act_bwd(xb.data_ptr(), pitch, 0, pitch, y.data_ptr(), n, m, n, 0, 0.0, 0.0, _native.F32, st) == _native.E_NULL
    # the blocks-per-CU override of families 7 / 8 changes the grid, not the result
    x = xb.contiguous()
    ref = torch.empty_like(x); out = torch.empty_like(x)
    assert lib.thn_act_fwd(x.data_ptr(), pitch, ref.data_ptr(), pitch, m, pitch, 0, 0.0, 0.0, _native.F32, st) == 0
    try:
        for bpc in (1, 4):
            assert lib.thn_norm_set_launch_override(7, 0, 0, 0, bpc) == 0
            assert lib.thn_act_fwd(x.data_ptr(), pitch, out.data_ptr(), pitch, m, pitch, 0, 0.0, 0.0, _native.F32, st) == 0
            torch.cuda.synchronize()
            assert torch.equal(out, ref)
    finally:
        lib.thn_norm_set_launch_override(7, 0, 0, 0, 0)
