"""GPU parity tests: the HIP path, called through the operator interface and the C ABI, against the CPU
oracle on the same seeded inputs -- the five benchmark configurations at full size, the reference's own unit
test matrix, every constructor variant, ragged / strided / misaligned inputs, the size limits, and
size-independent properties.  Tolerances are the north-star ones (see conftest.check_*)."""
import ctypes

import numpy as np
import pytest
import torch

from conftest import CONFIGS, make_case, f64
from parity_util import compare_with_oracle, gpu_forward_backward, run_and_compare
from TritonHub import _native
from TritonHub.Normalization import LayerNorm, RMSNorm, _launch
from TritonHub.Normalization.layernorm import layernorm
from TritonHub.Normalization.rmsnorm import rmsnorm

pytestmark = pytest.mark.gpu


def announce(msg):
    print(f"\n[case] {msg}", flush=True)


# ---- benchmark configurations, full size ---------------------------------------------------------------------
@pytest.mark.parametrize("name", list(CONFIGS))
def test_baseline_config_full_size(name):
    announce(f"baseline {name} shape={CONFIGS[name][1]}")
    c = make_case(name)
    n_elems = c["x"].numel()
    sample = None if n_elems <= 80_000_000 else 12          # the two 268M-element cases: sampled y / dx chunks
    worst, out = run_and_compare(c["kind"], c["x"], c["dy"], c["w"], c["b"], c["eps"], name, sample_chunks=sample)
    print("worst ratios to tolerance:", {k: round(v, 9) for k, v in worst.items()}, flush=True)
    assert out["y"].dtype == c["dtype"] and out["dx"].dtype == c["dtype"] and out["y"].shape == c["x"].shape
    assert out["rstd"].dtype == torch.float32 and out["rstd"].shape == (c["x"].numel() // c["x"].shape[-1],)


# ---- the reference's own unit-test matrix (UnitTests/Normalization/*_unittest.py:57-67) ------------------------
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.float64])
@pytest.mark.parametrize("dim", [32, 64, 128, 256, 512, 1024, 2048])
@pytest.mark.parametrize("kind", ["ln", "rms"])
def test_reference_unit_test_matrix(kind, dim, dtype):
    announce(f"reference matrix {kind} D={dim} {dtype}")
    torch.manual_seed(42)
    data = torch.randn(1, 256, 256, dim, device="cuda", dtype=dtype)
    if kind == "ln":
        ours = LayerNorm(dimension=dim, eps=1e-5, bias=True, elementwise_affine=True, device="cuda", dtype=dtype)
        theirs = torch.nn.LayerNorm(dim, eps=1e-5, bias=True, elementwise_affine=True, device="cuda", dtype=dtype)
    else:
        ours = RMSNorm(dimension=dim, eps=1e-5, elementwise_affine=True, device="cuda", dtype=dtype)
        theirs = torch.nn.RMSNorm(dim, eps=1e-5, elementwise_affine=True, device="cuda", dtype=dtype)
    a = data.clone().requires_grad_(True)
    r = data.clone().requires_grad_(True)
    # tolerances of the reference's test (layernorm_unittest.py:30-32)
    rtol, atol = (3e-4, 1e-3) if dtype == torch.float32 else (5e-3, 1e-2)
    if dtype == torch.float16:
        rtol, atol = 1e-2, 5e-2
    ya, yr = ours(a), theirs(r)
    assert torch.allclose(ya, yr, atol=atol, rtol=rtol), "Error in forward pass"
    g = torch.randn_like(ya)
    ya.backward(g)
    yr.backward(g)
    assert torch.allclose(a.grad, r.grad, atol=atol, rtol=rtol), "Error in backward pass"
    # what the reference's test leaves out: parameter gradients, and the tight tolerance against the oracle
    assert torch.allclose(ours.weight.grad, theirs.weight.grad, atol=max(atol, 0.3), rtol=rtol)
    rows = 4096
    x = data.reshape(-1, dim)[:rows].cpu()
    gy = g.reshape(-1, dim)[:rows].cpu()
    w = ours.weight.detach().cpu()
    b = ours.bias.detach().cpu() if kind == "ln" else None
    run_and_compare(kind, x, gy, w, b, 1e-5, f"{kind} D={dim} {dtype}")


# ---- constructor variants, parameter dtypes, input ranks ---------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("affine,bias", [(True, True), (True, False), (False, False)])
def test_layernorm_variants(dtype, affine, bias):
    announce(f"LayerNorm variant affine={affine} bias={bias} {dtype}")
    g = torch.Generator().manual_seed(7)
    x = torch.randn(3, 17, 384, generator=g).to(dtype)
    dy = torch.randn(3, 17, 384, generator=g).to(dtype)
    mod = LayerNorm(384, eps=1e-5, elementwise_affine=affine, bias=bias, device="cuda", dtype=dtype)
    if affine:
        with torch.no_grad():
            mod.weight.copy_((1 + 0.1 * torch.randn(384, generator=g)).to(dtype))
            if bias:
                mod.bias.copy_((0.1 * torch.randn(384, generator=g)).to(dtype))
    xg = x.cuda().requires_grad_(True)
    y = mod(xg)
    assert y.shape == x.shape and y.dtype == dtype
    saved = y.grad_fn.saved_tensors
    assert len(saved) == 5 and saved[0] is not None             # (input, weight, bias, mean, rstd), layernorm.py:215
    assert saved[3].dtype == torch.float32 and saved[3].shape == (51,) and saved[4].shape == (51,)
    assert (saved[1] is None) == (not affine) and (saved[2] is None) == (not (affine and bias))
    y.backward(dy.cuda())
    out = dict(y=y.detach(), dx=xg.grad, dw=mod.weight.grad if affine else None,
               db=mod.bias.grad if (affine and bias) else None, mean=saved[3], rstd=saved[4])
    w = mod.weight.detach().cpu() if affine else None
    b = mod.bias.detach().cpu() if (affine and bias) else None
    compare_with_oracle("ln", x, dy, w, b, 1e-5, out, "variant")
    if affine:
        assert mod.weight.grad.dtype == dtype and mod.weight.grad.shape == (384,)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("affine", [True, False])
def test_rmsnorm_variants(dtype, affine):
    announce(f"RMSNorm variant affine={affine} {dtype}")
    g = torch.Generator().manual_seed(8)
    x = torch.randn(2, 5, 7, 640, generator=g).to(dtype)
    dy = torch.randn(2, 5, 7, 640, generator=g).to(dtype)
    mod = RMSNorm(640, eps=1e-6, elementwise_affine=affine, device="cuda", dtype=dtype)
    if affine:
        with torch.no_grad():
            mod.weight.copy_((1 + 0.1 * torch.randn(640, generator=g)).to(dtype))
    xg = x.cuda().requires_grad_(True)
    y = mod(xg)
    saved = y.grad_fn.saved_tensors
    assert len(saved) == 3 and saved[2].dtype == torch.float32 and saved[2].shape == (70,)   # (input, weight, rstd)
    y.backward(dy.cuda())
    out = dict(y=y.detach(), dx=xg.grad, dw=mod.weight.grad if affine else None, db=None, mean=None, rstd=saved[2])
    compare_with_oracle("rms", x, dy, mod.weight.detach().cpu() if affine else None, None, 1e-6, out, "variant")


@pytest.mark.parametrize("n", [384, 4096, 12288])
@pytest.mark.parametrize("kind", ["ln", "rms", "ln_gelu"])
def test_frozen_parameters_skip_their_sums(kind, n):
    """requires_grad=False on weight and / or bias: that gradient is None, the others and dx are bit-identical to
    the run with every gradient wanted (the row kernel is the same, only the stores of its sums differ)."""
    from TritonHub.Normalization.fused import LayerNormActivation
    announce(f"frozen parameters {kind} N={n}")
    g = torch.Generator().manual_seed(n)
    x = torch.randn(300, n, generator=g).bfloat16().cuda()
    dy = torch.randn(300, n, generator=g).bfloat16().cuda()
    make = {"ln": lambda: LayerNorm(n, device="cuda", dtype=torch.bfloat16),
            "rms": lambda: RMSNorm(n, device="cuda", dtype=torch.bfloat16),
            "ln_gelu": lambda: LayerNormActivation(n, "gelu", device="cuda", dtype=torch.bfloat16)}[kind]
    full = make()
    with torch.no_grad():
        full.weight.copy_(1 + 0.1 * torch.randn(n, generator=g).cuda())
    xf = x.clone().requires_grad_(True)
    full(xf).backward(dy)
    has_bias = kind != "rms"
    for train_w, train_b in ((False, False), (True, False), (False, True)):
        if train_b and not has_bias:
            continue
        mod = make()
        mod.load_state_dict(full.state_dict())
        mod.weight.requires_grad_(train_w)
        if has_bias:
            mod.bias.requires_grad_(train_b)
        xg = x.clone().requires_grad_(True)
        mod(xg).backward(dy)
        assert torch.equal(xg.grad, xf.grad)
        assert (mod.weight.grad is None) == (not train_w)
        if train_w:
            assert torch.equal(mod.weight.grad, full.weight.grad)
        if has_bias:
            assert (mod.bias.grad is None) == (not train_b)
            if train_b:
                assert torch.equal(mod.bias.grad, full.bias.grad)
    # only the parameters want gradients: the input's is computed and dropped
    mod = make()
    mod.load_state_dict(full.state_dict())
    mod(x).backward(dy)
    assert torch.equal(mod.weight.grad, full.weight.grad)


def test_mixed_parameter_and_activation_dtypes():
    # float32 parameters under bfloat16 activations: dW / dB come back in the parameter dtype (layernorm.py:207-208)
    announce("mixed dtypes")
    g = torch.Generator().manual_seed(9)
    x = torch.randn(64, 1024, generator=g).bfloat16(); dy = torch.randn(64, 1024, generator=g).bfloat16()
    w = 1 + 0.1 * torch.randn(1024, generator=g); b = 0.1 * torch.randn(1024, generator=g)
    worst, out = run_and_compare("ln", x, dy, w, b, 1e-5, "mixed ln")
    assert out["dw"].dtype == torch.float32 and out["db"].dtype == torch.float32 and out["y"].dtype == torch.bfloat16
    worst, out = run_and_compare("rms", x.float(), dy.float(), w.half(), None, 1e-5, "mixed rms")
    assert out["dw"].dtype == torch.float16 and out["dx"].dtype == torch.float32


# ---- ragged, strided and misaligned inputs ---------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64])
@pytest.mark.parametrize("n", [1, 2, 7, 33, 100, 257, 1000, 4099, 6001])
@pytest.mark.parametrize("kind", ["ln", "rms"])
def test_ragged_hidden_sizes(kind, n, dtype):
    announce(f"ragged {kind} N={n} {dtype}")
    g = torch.Generator().manual_seed(n)
    m = 19
    x = (torch.randn(m, n, generator=g) * 2 + 0.5).to(dtype); dy = torch.randn(m, n, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype)
    b = (0.1 * torch.randn(n, generator=g)).to(dtype) if kind == "ln" else None
    run_and_compare(kind, x, dy, w, b, 1e-5, f"ragged N={n}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_odd_widths_of_16_bit_rows_reach_every_two_vector_shape(dtype):
    """Rows off the 128-bit path run in the same slot shapes as rows on it (or, up to 32 vectors, on the flat kernels):
    one odd width for each threads-per-row value, LayerNorm (16-bit and float32 parameters) and RMSNorm."""
    g = torch.Generator().manual_seed(77)
    for n in (9, 121, 201, 499, 1001, 1501, 3001, 4099, 12289, 20001):
        announce(f"odd width {n} {dtype}")
        m = 131
        for which, ln in ((0, True), (0, False), (1, True), (1, False)):
            kk, tt, _, _, vector_path = _launch.query_launch(which, ln, m, n, dtype)
            n_vecs = (n + 7) // 8
            assert vector_path == 0
            if n_vecs <= 32 and tt == n_vecs:
                continue                      # the flat kernels: a lane per vector, kk rows per lane
            assert kk * tt >= n_vecs and (kk - 1) * tt < n_vecs    # no emptier than it has to be
        x = (0.5 + torch.randn(m, n, generator=g)).to(dtype); dy = torch.randn(m, n, generator=g).to(dtype)
        w = (1 + 0.1 * torch.randn(n, generator=g)); b = 0.1 * torch.randn(n, generator=g)
        run_and_compare("ln", x, dy, w.to(dtype), b.to(dtype), 1e-5, f"odd LN N={n}")
        run_and_compare("ln", x, dy, w, b, 1e-5, f"odd LN N={n}, float32 parameters")
        run_and_compare("rms", x, dy, w.to(dtype), None, 1e-5, f"odd RMS N={n}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_row_strides_and_misaligned_views(dtype):
    announce(f"strides {dtype}")
    g = torch.Generator().manual_seed(13)
    big = torch.randn(40, 1024, generator=g).to(dtype).cuda()
    dyb = torch.randn(40, 1024, generator=g).to(dtype).cuda()
    w = (1 + 0.1 * torch.randn(512, generator=g)).to(dtype)
    b = (0.1 * torch.randn(512, generator=g)).to(dtype)
    views = {
        "row stride 1024, aligned": (big[:, :512], dyb[:, 256:768]),
        "row stride 1024, base off by one element": (big[:, 1:513], dyb[:, 3:515]),
        "every other row": (big[::2, 512:], dyb[1::2, :512]),
    }
    for label, (xv, dv) in views.items():
        for kind in ("ln", "rms"):
            xg = xv.detach().requires_grad_(True)
            wg = w.cuda().requires_grad_(True)
            bg = b.cuda().requires_grad_(True) if kind == "ln" else None
            y = layernorm.apply(xg, wg, bg, 1e-5) if kind == "ln" else rmsnorm.apply(xg, wg, 1e-5)
            assert y.is_contiguous()
            saved = y.grad_fn.saved_tensors
            y.backward(dv)
            out = dict(y=y.detach(), dx=xg.grad, dw=wg.grad, db=None if bg is None else bg.grad,
                       mean=saved[3] if kind == "ln" else None, rstd=saved[4] if kind == "ln" else saved[2])
            compare_with_oracle(kind, xv.cpu().contiguous(), dv.cpu().contiguous(), w, b if kind == "ln" else None,
                                1e-5, out, f"{label} {kind}")
    # last stride != 1 is made contiguous by the wrapper (layernorm.py:49-50)
    xt = torch.randn(96, 24, generator=g).to(dtype).cuda().t()          # shape (24, 96), strides (1, 24)
    mod = RMSNorm(96, device="cuda", dtype=dtype)
    y = mod(xt)
    ref = mod(xt.contiguous())
    assert torch.equal(y, ref)


def test_empty_and_single_row():
    announce("empty / single row")
    mod = LayerNorm(64, device="cuda")
    x = torch.empty(0, 64, device="cuda", requires_grad=True)
    y = mod(x)
    assert y.shape == (0, 64)
    y.backward(torch.empty(0, 64, device="cuda"))
    assert x.grad.shape == (0, 64)
    assert torch.equal(mod.weight.grad, torch.zeros(64, device="cuda"))      # the sum over no rows
    assert torch.equal(mod.bias.grad, torch.zeros(64, device="cuda"))
    g = torch.Generator().manual_seed(3)
    x1 = torch.randn(1, 64, generator=g); d1 = torch.randn(1, 64, generator=g)
    run_and_compare("ln", x1, d1, torch.ones(64), torch.zeros(64), 1e-5, "single row")
    # N = 1: variance 0, y = bias
    y = LayerNorm(1, device="cuda")(torch.randn(5, 1, device="cuda"))
    assert torch.equal(y, torch.zeros(5, 1, device="cuda"))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [48, 1000, 4096, 12288])
@pytest.mark.parametrize("kind", ["ln", "rms"])
def test_non_finite_inputs_stay_in_their_row(kind, n, dtype):
    """A NaN or an infinity in the input spoils only its own row of y and dx (the statistics are per row) and,
    through the column sums, every dW entry (xhat of that row is NaN everywhere); dB only sums the upstream
    gradient and stays finite.  The other rows are bit-identical to a run without the spoiled rows."""
    announce(f"non-finite {kind} N={n} {dtype}")
    g = torch.Generator().manual_seed(n)
    rows = 37
    x = torch.randn(rows, n, generator=g).to(dtype)
    dy = torch.randn(rows, n, generator=g).to(dtype)
    bad = {3: float("nan"), 11: float("inf"), 20: float("-inf")}
    for r, v in bad.items():
        x[r, (r * 7) % n] = v
    make = (lambda: LayerNorm(n, device="cuda", dtype=dtype)) if kind == "ln" else \
        (lambda: RMSNorm(n, device="cuda", dtype=dtype))
    mod = make()
    xg = x.cuda().requires_grad_(True)
    y = mod(xg)
    y.backward(dy.cuda())
    good = torch.ones(rows, dtype=torch.bool)
    good[list(bad)] = False
    y, dx = y.detach().cpu(), xg.grad.cpu()
    assert bool(torch.isnan(dx[~good]).all()) and bool(torch.isnan(y[3]).all())
    for r in (11, 20):
        spoiled = torch.zeros(n, dtype=torch.bool)
        spoiled[(r * 7) % n] = True
        if kind == "ln":                # mean = +-inf: every x - mean is NaN or infinite, the variance NaN
            assert bool(torch.isnan(y[r]).all())
        else:                           # mean(x^2) = inf: rstd = 0, so y = 0 except inf * 0 at the spoiled column
            assert bool(torch.isnan(y[r][spoiled]).all()) and bool((y[r][~spoiled] == 0).all())
    assert bool(torch.isfinite(y[good]).all()) and bool(torch.isfinite(dx[good]).all())
    assert bool(torch.isnan(mod.weight.grad).all())
    if kind == "ln":
        assert bool(torch.isfinite(mod.bias.grad).all())
    ref = make()
    xr = x[good].cuda().requires_grad_(True)
    yr = ref(xr)
    yr.backward(dy[good].cuda())
    assert torch.equal(yr.detach().cpu(), y[good]) and torch.equal(xr.grad.cpu(), dx[good])


# ---- the 64 KiB row limit (layernorm.py:69-72) -----------------------------------------------------------------
@pytest.mark.parametrize("dtype,n_max", [(torch.float32, 16384), (torch.bfloat16, 32768), (torch.float16, 32768),
                                         (torch.float64, 8192)])
def test_feature_dim_limit(dtype, n_max):
    announce(f"feature dim limit {dtype} N={n_max}")
    g = torch.Generator().manual_seed(5)
    x = torch.randn(6, n_max, generator=g).to(dtype); dy = torch.randn(6, n_max, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(n_max, generator=g)).to(dtype); b = (0.1 * torch.randn(n_max, generator=g)).to(dtype)
    run_and_compare("ln", x, dy, w, b, 1e-5, f"LN N={n_max}")
    run_and_compare("rms", x, dy, w, None, 1e-5, f"RMS N={n_max}")
    over = torch.randn(2, n_max + 8, device="cuda").to(dtype)
    for mod in (LayerNorm(n_max + 8, device="cuda", dtype=dtype), RMSNorm(n_max + 8, device="cuda", dtype=dtype)):
        with pytest.raises(RuntimeError, match="This layer norm doesn't support feature dim >= 64KB."):
            mod(over)


# ---- rows of 24-64 KiB: the 1024-thread workgroups, several rows per workgroup ----------------------------------
@pytest.mark.parametrize("dtype,widths", [(torch.bfloat16, (12296, 16384, 20480, 24576, 26624, 28680, 32768)),
                                          (torch.float16, (16384, 24568, 28672, 32768)),
                                          (torch.float32, (6148, 8192, 12288, 16384)),
                                          (torch.float64, (4096, 8192))])
def test_wide_rows_many_per_workgroup(dtype, widths):
    """More rows than the persistent grid has workgroups, so every workgroup walks several rows and the last
    grid-stride step is only partly filled; parameters in the row's dtype and (16-bit rows) in float32."""
    g = torch.Generator().manual_seed(31)
    m = 600
    for n in widths:
        announce(f"wide rows {dtype} {m}x{n}")
        x = (0.5 + torch.randn(m, n, generator=g)).to(dtype); dy = torch.randn(m, n, generator=g).to(dtype)
        w = 1 + 0.1 * torch.randn(n, generator=g); b = 0.1 * torch.randn(n, generator=g)
        run_and_compare("ln", x, dy, w.to(dtype), b.to(dtype), 1e-5, f"wide LN N={n}")
        run_and_compare("rms", x, dy, w.to(dtype), None, 1e-5, f"wide RMS N={n}")
        if dtype in (torch.bfloat16, torch.float16) and n >= 24576:
            run_and_compare("ln", x, dy, w, b, 1e-5, f"wide LN N={n}, float32 parameters")


@pytest.mark.parametrize("dtype,n", [(torch.bfloat16, 32768), (torch.float32, 16384), (torch.float16, 24576)])
def test_wide_rows_forward_with_more_workgroups_than_the_chip_holds(dtype, n):
    """From 12 rows of more than 48 KiB (4 x 1024 vectors) per compute unit on, the forward launches up to four times as
    many workgroups as are resident at once (twice for the 16-bit LayerNorm) when that makes whole rounds of them;
    rows of 3 x 1024 vectors and row counts that would leave a round half empty keep one workgroup per compute unit.
    The oracle comparison runs 16 * cus - 3 rows, which leave the last grid-stride step partly filled."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    grid_rms = _launch.query_launch(0, False, 16 * cus, n, dtype)[3]
    grid_ln = _launch.query_launch(0, True, 16 * cus, n, dtype)[3]
    m = 16 * cus - 3
    if _launch.query_launch(0, False, m, n, dtype)[0] == 4:
        assert grid_rms == 4 * cus and grid_ln == (2 if dtype != torch.float32 else 4) * cus, (grid_rms, grid_ln)
        assert _launch.query_launch(0, False, m, n, dtype)[3] == 2 * cus               # two whole rounds, the last rows short
        assert _launch.query_launch(0, False, 12 * cus + 128, n, dtype)[3] <= cus      # 2.5 rounds of workgroups: not taken
    else:
        assert grid_rms <= cus and grid_ln <= cus, (grid_rms, grid_ln)
    assert _launch.query_launch(0, False, 8 * cus, n, dtype)[3] == cus
    assert _launch.query_launch(1, False, m, n, dtype)[3] <= cus          # the backward: one partial row per workgroup
    g = torch.Generator().manual_seed(37)
    announce(f"wide rows, forward grid {grid_rms} / {grid_ln} workgroups: {dtype} {m}x{n}")
    x = (0.5 + torch.randn(m, n, generator=g)).to(dtype); dy = torch.randn(m, n, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype); b = (0.1 * torch.randn(n, generator=g)).to(dtype)
    run_and_compare("ln", x, dy, w, b, 1e-5, f"LN {m}x{n}")
    run_and_compare("rms", x, dy, w, None, 1e-5, f"RMS {m}x{n}")


def test_forward_workgroups_per_compute_unit():
    """The forward's launch rules that depend on the row count: a second workgroup per compute unit for short
    kernels (4 vectors per thread in 256 threads, at most 8 steps each) and for 3-vector 256-thread shapes -- but
    for the one-row workgroup at a pitch off 128-byte lines only up to 32 rows per compute unit.  Each case also
    runs against the oracle at the row count just inside the rule."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    bf16, f16 = torch.bfloat16, torch.float16
    grid = lambda which, ln, m, n, dt: _launch.query_launch(which, ln, m, n, dt)[3]
    # 4096 bf16 columns: two rows per 256-thread workgroup; 8 steps each = 16 rows per compute unit
    assert grid(0, True, 16 * cus, 4096, bf16) == 2 * cus
    assert grid(0, True, 64 * cus, 4096, bf16) == cus
    assert grid(1, True, 16 * cus, 4096, bf16) == cus                   # the backward: one partial row per compute unit
    # 1280 bf16 columns (3 vectors x 64 threads, four rows per workgroup): two at every row count
    assert grid(0, False, 8 * cus, 1280, bf16) == 2 * cus and grid(0, False, 512 * cus, 1280, bf16) == 2 * cus
    # 6000 fp16 columns: 12000-byte rows, one row per workgroup, vectors shifted onto 128-byte lines
    assert grid(0, True, 32 * cus, 6000, f16) == 2 * cus
    assert grid(0, True, 64 * cus, 6000, f16) == cus
    g = torch.Generator().manual_seed(41)
    for m, n, dt in ((16 * cus, 4096, bf16), (32 * cus, 6000, f16), (8 * cus + 3, 1280, bf16)):
        announce(f"forward with two workgroups per compute unit: {dt} {m}x{n}")
        x = (0.5 + torch.randn(m, n, generator=g)).to(dt); dy = torch.randn(m, n, generator=g).to(dt)
        w = (1 + 0.1 * torch.randn(n, generator=g)).to(dt); b = (0.1 * torch.randn(n, generator=g)).to(dt)
        run_and_compare("ln", x, dy, w, b, 1e-5, f"LN {m}x{n}")
        run_and_compare("rms", x, dy, w, None, 1e-5, f"RMS {m}x{n}")


def test_backward_over_few_rows_takes_half_the_workgroups():
    """The backward's launch rule for few rows: when a full grid would visit at most two row blocks per workgroup
    and the partial rows are a quarter or more of the bytes of x, dy and dx, half the workgroups are launched (half
    the partial rows for the second stage).  The grids on both sides of the rule, and the oracle at sizes inside it."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    bf16, f32 = torch.bfloat16, torch.float32
    grid = lambda ln, m, n, dt: _launch.query_launch(1, ln, m, n, dt)[3]
    # 4096 bf16 columns: two rows per workgroup.  2 * cus rows = one row block per workgroup of a full grid
    assert grid(False, 2 * cus, 4096, bf16) == cus // 2 and grid(True, 2 * cus, 4096, bf16) == cus // 2
    assert grid(True, 4 * cus, 4096, bf16) == cus // 2          # two gradients: partial rows still a third of the bytes
    assert grid(False, 4 * cus, 4096, bf16) == cus              # one gradient: a sixth
    assert grid(True, 8 * cus, 4096, bf16) == cus               # four row blocks per workgroup
    assert grid(True, cus, 4096, bf16) == cus // 2              # fewer row blocks than compute units: one each
    assert grid(True, 4 * cus, 4096, f32) == cus                # float32 rows: one row per workgroup, four blocks each
    g = torch.Generator().manual_seed(43)
    for m, n, dt in ((2 * cus, 4096, bf16), (4 * cus - 1, 4096, bf16), (cus, 8192, bf16), (2 * cus + 1, 16384, bf16),
                     (2 * cus, 4096, f32)):
        announce(f"backward with half the workgroups: {dt} {m}x{n}")
        x = (0.5 + torch.randn(m, n, generator=g)).to(dt); dy = torch.randn(m, n, generator=g).to(dt)
        w = (1 + 0.1 * torch.randn(n, generator=g)).to(dt); b = (0.1 * torch.randn(n, generator=g)).to(dt)
        run_and_compare("ln", x, dy, w, b, 1e-5, f"LN {m}x{n}")
        run_and_compare("rms", x, dy, w, None, 1e-5, f"RMS {m}x{n}")


# ---- size-independent properties at full benchmark sizes --------------------------------------------------------
@pytest.mark.parametrize("name", ["c2_rms_bf16_llm", "c5a_ln_f32_hostile", "c4_ln_f32_small_hidden"])
def test_properties_at_full_size(name):
    announce(f"properties {name}")
    rows = 131072 if name.startswith("c4") else None
    c = make_case(name, rows=rows)
    kind = c["kind"]
    a = gpu_forward_backward(kind, c["x"], c["dy"], c["w"], c["b"], c["eps"])
    # 1. run-to-run determinism, bit for bit (no atomics anywhere on the path)
    a2 = gpu_forward_backward(kind, c["x"], c["dy"], c["w"], c["b"], c["eps"])
    for k in ("y", "dx", "dw", "db", "rstd", "mean"):
        if a[k] is not None:
            assert torch.equal(a[k], a2[k]), f"{k} differs between two identical runs"
    # 2. the backward is linear in dy, and scaling by 4 is exact in binary floating point
    s = gpu_forward_backward(kind, c["x"], c["dy"] * 4, c["w"], c["b"], c["eps"])
    assert torch.equal(s["dx"], a["dx"] * 4) and torch.equal(s["dw"], a["dw"] * 4)
    if s["db"] is not None:
        assert torch.equal(s["db"], a["db"] * 4)
    # 3. rows are independent: moving a row moves its y, dx and rstd bit for bit.  Blocks of 8 rows are reversed,
    #    so every row keeps its place modulo 8 and with it the place of its first byte within a 128-byte line
    #    whatever the pitch: rows 24000 bytes apart (8192 x 6000 float32) are summed in the lane order that puts
    #    the wave requests on line boundaries, which depends on that place (and only on it).
    n = c["x"].shape[-1]
    blocks = lambda t: t.reshape(-1, 8, *t.shape[1:]).flip(0).reshape(t.shape)
    x2 = c["x"].reshape(-1, n); d2 = c["dy"].reshape(-1, n)
    r = gpu_forward_backward(kind, blocks(x2), blocks(d2), c["w"], c["b"], c["eps"])
    assert torch.equal(blocks(r["y"]), a["y"].reshape(r["y"].shape))
    assert torch.equal(blocks(r["dx"]), a["dx"].reshape(r["dx"].shape))
    assert torch.equal(blocks(r["rstd"]), a["rstd"])
    # 4. LayerNorm: each dx row sums to ~0 and, without affine parameters, each y row has mean 0 / variance var/(var+eps)
    if kind == "ln":
        dxs = a["dx"].double().sum(-1).abs().max().item()
        bound = 64 * 2.0 ** -24 * a["dx"].double().abs().sum(-1).max().item()
        assert dxs <= bound, (dxs, bound)
        plain = gpu_forward_backward("ln", c["x"], c["dy"], None, None, c["eps"])
        y64 = plain["y"].double()
        assert y64.mean(-1).abs().max().item() < 1e-5
        assert (y64.pow(2).mean(-1) - 1).abs().max().item() < 1e-4


# ---- the C ABI called directly -------------------------------------------------------------------------------
def test_c_abi_direct_calls_and_errors():
    announce("C ABI direct")
    lib = _native.lib()
    g = torch.Generator().manual_seed(17)
    m, n, pitch = 300, 768, 1024
    st = torch.cuda.current_stream().cuda_stream
    xb = torch.randn(m, pitch, generator=g).cuda(); db_ = torch.randn(m, pitch, generator=g).cuda()
    w = (1 + 0.1 * torch.randn(n, generator=g)).cuda(); b = (0.1 * torch.randn(n, generator=g)).cuda()
    x, dy = xb[:, :n], db_[:, :n]
    y = torch.full((m, pitch), 7.0, device="cuda"); dx = torch.full((m, pitch), 7.0, device="cuda")
    mean = torch.empty(m, device="cuda"); rstd = torch.empty(m, device="cuda")
    rc = lib.thn_norm_fwd(x.data_ptr(), pitch, y.data_ptr(), pitch, w.data_ptr(), b.data_ptr(), mean.data_ptr(),
                          rstd.data_ptr(), m, n, 1e-5, _native.F32, _native.F32, st)
    assert rc == 0
    nbytes = lib.thn_norm_bwd_workspace_bytes(m, n, 1, 1, _native.F32)
    assert nbytes > 0
    ws = torch.empty(nbytes // 4, device="cuda")
    dw = torch.empty(n, device="cuda"); dbias = torch.empty(n, device="cuda")
    rc = lib.thn_norm_bwd(x.data_ptr(), pitch, dy.data_ptr(), pitch, dx.data_ptr(), pitch, w.data_ptr(),
                          mean.data_ptr(), rstd.data_ptr(), dw.data_ptr(), dbias.data_ptr(), ws.data_ptr(), nbytes,
                          m, n, _native.F32, _native.F32, st)
    assert rc == 0
    torch.cuda.synchronize()
    assert bool((y[:, n:] == 7.0).all()) and bool((dx[:, n:] == 7.0).all())      # the padding of strided outputs is untouched
    out = dict(y=y[:, :n], dx=dx[:, :n], dw=dw, db=dbias, mean=mean, rstd=rstd)
    compare_with_oracle("ln", x.cpu().contiguous(), dy.cpu().contiguous(), w.cpu(), b.cpu(), 1e-5, out, "C ABI")
    # the two stages called apart give the same bits as the fused entry point
    parts = ctypes.c_int32(0)
    dx2 = torch.empty(m, n, device="cuda"); dw2 = torch.empty(n, device="cuda"); db2 = torch.empty(n, device="cuda")
    rc = lib.thn_norm_bwd_dx_partials(x.data_ptr(), pitch, dy.data_ptr(), pitch, dx2.data_ptr(), n, w.data_ptr(),
                                      mean.data_ptr(), rstd.data_ptr(), 1, 1, ws.data_ptr(), nbytes, ctypes.byref(parts),
                                      m, n, _native.F32, _native.F32, st)
    assert rc == 0 and parts.value > 0
    assert lib.thn_norm_bwd_reduce_partials(ws.data_ptr(), parts.value, dw2.data_ptr(), db2.data_ptr(), n,
                                            _native.F32, st) == 0
    torch.cuda.synchronize()
    assert torch.equal(dx2, dx[:, :n]) and torch.equal(dw2, dw) and torch.equal(db2, dbias)
    # error codes
    assert lib.thn_norm_bwd(x.data_ptr(), pitch, dy.data_ptr(), pitch, dx.data_ptr(), pitch, w.data_ptr(),
                            mean.data_ptr(), rstd.data_ptr(), dw.data_ptr(), dbias.data_ptr(), ws.data_ptr(), 64,
                            m, n, _native.F32, _native.F32, st) == _native.E_WORKSPACE
    # a workspace that is not 16-byte aligned is refused before anything is launched
    assert lib.thn_norm_bwd(x.data_ptr(), pitch, dy.data_ptr(), pitch, dx.data_ptr(), pitch, w.data_ptr(),
                            mean.data_ptr(), rstd.data_ptr(), dw.data_ptr(), dbias.data_ptr(), ws.data_ptr() + 4,
                            nbytes - 4, m, n, _native.F32, _native.F32, st) == _native.E_WORKSPACE
    assert lib.thn_norm_bwd(x.data_ptr(), pitch, 0, pitch, dx.data_ptr(), pitch, w.data_ptr(), mean.data_ptr(),
                            rstd.data_ptr(), dw.data_ptr(), dbias.data_ptr(), ws.data_ptr(), nbytes, m, n,
                            _native.F32, _native.F32, st) == _native.E_NULL
    assert lib.thn_norm_fwd(x.data_ptr(), n - 1, y.data_ptr(), pitch, 0, 0, 0, rstd.data_ptr(), m, n, 1e-5,
                            _native.F32, _native.F32, st) == _native.E_SHAPE         # row stride < N
    assert lib.thn_norm_fwd(x.data_ptr(), pitch, y.data_ptr(), pitch, 0, b.data_ptr(), 0, rstd.data_ptr(), m, n, 1e-5,
                            _native.F32, _native.F32, st) == _native.E_SHAPE         # RMSNorm takes no bias
    # gradients that are not wanted are not computed: dw = db = NULL needs no workspace
    assert lib.thn_norm_bwd(x.data_ptr(), pitch, dy.data_ptr(), pitch, dx2.data_ptr(), n, w.data_ptr(),
                            mean.data_ptr(), rstd.data_ptr(), 0, 0, 0, 0, m, n, _native.F32, _native.F32, st) == 0
    torch.cuda.synchronize()
    assert torch.equal(dx2, dx[:, :n])


# ---- cache policy of the forward's read of x ------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_cache_policies_give_the_same_bits(dtype):
    """The keep-x and stream-x forwards differ in a hint on their loads of x and in nothing else: y, mean and rstd
    must be bit-identical, through the per-call flag, through the process-wide default and through the modules
    (training keeps, torch.no_grad() streams, set_cache_policy forces)."""
    announce(f"cache policies {dtype}")
    lib = _native.lib()
    p = _native.ptr
    code = _native.dtype_code(dtype)
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(5)
    # 128-bit path (several launch shapes), rows off it, rows shorter than a vector, an activation epilogue
    for m, n in ((3000, 4096), (777, 6000), (5000, 256), (64, 16384), (1500, 4099), (300, 3), (900, 1288)):
        x = (torch.randn(m, n, generator=g) * 2 + 0.5).to(dtype).cuda()
        w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype).cuda()
        b = (0.1 * torch.randn(n, generator=g)).to(dtype).cuda()
        for ln in (True, False):
            for act in (-1, _native.ACT_SILU):
                outs = []
                for how in ("keep flag", "stream flag", "default keep", "default stream"):
                    y = torch.full_like(x, 9.0)
                    mean = torch.full((m,), 9.0, device="cuda") if ln else None
                    rstd = torch.full((m,), 9.0, device="cuda")
                    flag = {"keep flag": _native.X_KEEP, "stream flag": _native.X_STREAM}.get(how, 0)
                    assert lib.thn_norm_set_cache_policy(1 if how == "default stream" else 0) == 0
                    try:
                        if act < 0:
                            rc = lib.thn_norm_fwd(p(x), n, p(y), n, p(w), p(b) if ln else 0, p(mean), p(rstd), m, n, 1e-6,
                                                  code | flag, code, st)
                        else:
                            rc = lib.thn_norm_act_fwd(p(x), n, p(y), n, p(w), p(b) if ln else 0, p(mean), p(rstd), m, n,
                                                      1e-6, act, code | flag, code, st)
                    finally:
                        lib.thn_norm_set_cache_policy(0)
                    assert rc == 0, (_native.strerror(rc), how, m, n, ln, act)
                    torch.cuda.synchronize()
                    outs.append((y, mean, rstd))
                for y, mean, rstd in outs[1:]:
                    assert torch.equal(y.view(torch.uint8), outs[0][0].view(torch.uint8)), (m, n, ln, act)
                    assert torch.equal(rstd, outs[0][2]) and (not ln or torch.equal(mean, outs[0][1]))
                assert not bool((outs[0][2] == 9.0).any())
    # the modules: the same bits whichever policy the Python layer picks
    x = torch.randn(4, 500, 2048, generator=g).to(dtype).cuda()
    for mod in (LayerNorm(2048, device="cuda", dtype=dtype), RMSNorm(2048, device="cuda", dtype=dtype)):
        ys = []
        with torch.no_grad():
            ys.append(mod(x))                                 # 'auto': no backward follows, x is streamed
        ys.append(mod(x.clone().requires_grad_(True)).detach())    # 'auto': x is kept
        for forced in ("keep", "stream"):
            _launch.set_cache_policy(forced)
            try:
                ys.append(mod(x.clone().requires_grad_(True)).detach())
            finally:
                _launch.set_cache_policy("auto")
        for y in ys[1:]:
            assert torch.equal(y.view(torch.uint8), ys[0].view(torch.uint8))


# ---- every compiled kernel shape ---------------------------------------------------------------------------------
def compiled_shapes():
    import os, re
    from conftest import ROOT
    text = open(os.path.join(ROOT, "triton-hub_amd", "csrc", "thn_dispatch.h")).read()

    def expand(macro, block=None):
        body = re.search(r"#define " + macro + r"\(X(?:, B)?\)(.*?)\n\n", text, re.S).group(1)
        shapes = []
        for k, t, b in re.findall(r"X\((\d+), (\d+), (\w+)\)", body):
            shapes.append((int(k), int(t), block if b == "B" else int(b)))
        return shapes
    fwd = expand("THN_FWD_SHAPES") + expand("THN_FWD_SHAPES_TWO_ROWS") + expand("THN_FWD_SHAPES_THREE")
    fwd += expand("THN_FWD_SHAPES_AS_BACKWARD")
    bwd = [s for blk in (256, 512) for s in expand("THN_BWD_SHAPES_B", blk)]
    tail = re.search(r"#define THN_BWD_SHAPES\(X\)(.*?)\n\n", text, re.S).group(1)
    bwd += [(int(k), int(t), int(b)) for k, t, b in re.findall(r"X\((\d+), (\d+), (\d+)\)", tail)]
    bwd += expand("THN_BWD_SHAPES_THREE")
    return fwd, bwd, expand("THN_BWD_SHAPES_LN16")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("kind", ["ln", "rms"])
def test_every_compiled_launch_shape(kind, dtype):
    """Forces each kernel instance in turn through the launch override and checks it against the oracle, at a
    row width that fills the shape exactly and at one that leaves vector slots without work."""
    lib = _native.lib()
    fwd_shapes, bwd_shapes, ln16_shapes = compiled_shapes()
    assert len(fwd_shapes) >= 20 and len(bwd_shapes) >= 40 and len(ln16_shapes) == 4
    if kind == "ln" and dtype == torch.bfloat16:
        bwd_shapes = bwd_shapes + ln16_shapes       # instances that only the LayerNorm backward of 16-bit rows has
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    g = torch.Generator().manual_seed(23)
    pairs = sorted(set((k, t) for k, t, _ in fwd_shapes + bwd_shapes))
    try:
        for k, tpr in pairs:
            widths = []
            for n_vecs in sorted({k * tpr, max((k - 1) * tpr + 1, k * tpr - tpr // 2 - 1)}):
                widths.append(n_vecs * vec)
                # ... and the same number of slots off the 128-bit path: the last one ragged, its window overlapping
                # the slot before it by 1 to vec - 1 columns
                widths.append(n_vecs * vec - 1 - n_vecs % (vec - 1))
            for n in widths:
                if n * (16 // vec) > 65536 or n < vec or (n % vec and k >= 5):      # (5 to 8 vectors: 128-bit path only)
                    continue
                f_blocks = [b for kk, tt, b in fwd_shapes if (kk, tt) == (k, tpr)]
                b_blocks = [b for kk, tt, b in bwd_shapes if (kk, tt) == (k, tpr)]
                for fb, bb in zip(f_blocks + [0] * len(b_blocks), b_blocks + [0] * len(f_blocks)):
                    if fb == 0 and bb == 0:
                        break
                    rows_per_block = max(fb, bb, 256) // tpr
                    m = 2 * rows_per_block + max(1, rows_per_block // 2)
                    announce(f"shape K={k} TPR={tpr} fwd block={fb} bwd block={bb} N={n} M={m} {kind} {dtype}")
                    x = torch.randn(m, n, generator=g).to(dtype); dy = torch.randn(m, n, generator=g).to(dtype)
                    w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype)
                    b = (0.1 * torch.randn(n, generator=g)).to(dtype) if kind == "ln" else None
                    assert lib.thn_norm_set_launch_override(0, k if fb else 0, tpr if fb else 0, fb, 0) == 0
                    assert lib.thn_norm_set_launch_override(1, k if bb else 0, tpr if bb else 0, bb, 0) == 0
                    if fb:
                        assert _launch.query_launch(0, kind == "ln", m, n, dtype)[:3] == (k, tpr, fb)
                    if bb:
                        assert _launch.query_launch(1, kind == "ln", m, n, dtype)[:3] == (k, tpr, bb)
                    run_and_compare(kind, x, dy, w, b, 1e-5, f"K={k} TPR={tpr} blocks=({fb},{bb}) N={n}")
    finally:
        lib.thn_norm_set_launch_override(0, 0, 0, 0, 0)
        lib.thn_norm_set_launch_override(1, 0, 0, 0, 0)


@pytest.mark.parametrize("dtype,n,want", [
    (torch.bfloat16, 2560, (3, 128, 512)), (torch.bfloat16, 2800, (3, 128, 512)), (torch.bfloat16, 2501, (3, 128, 512)),
    (torch.float16, 2304, (3, 128, 512)), (torch.float32, 1280, (3, 128, 512)), (torch.float32, 1301, (3, 128, 512)),
    (torch.bfloat16, 1280, (3, 64, 512)), (torch.float16, 1100, (3, 64, 512)),
    (torch.bfloat16, 256, (2, 16, 256)), (torch.float16, 512, (2, 32, 256)), (torch.bfloat16, 450, (2, 32, 256)),
    (torch.bfloat16, 320, (3, 16, 512)), (torch.float16, 768, (3, 32, 512)), (torch.bfloat16, 701, (3, 32, 512))])
def test_forward_takes_the_row_groups_of_the_backward(dtype, n, want):
    """Rows of 257 to 351 vectors (16-bit LayerNorm: also 17 to 96 and 129 to 160): the forward runs as many rows per
    workgroup as the backward, so that a row meets the same XCD -- and its L2 -- in both directions; the 3-vector
    512-thread shapes of narrow rows only while x fits the L2s.  Checked against the oracle."""
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    n_vecs = -(-n // vec)
    g = torch.Generator().manual_seed(n)
    for kind in ("rms", "ln"):
        if n_vecs <= 160 and kind == "rms":
            continue
        for m in (37, 4096):
            f = _launch.query_launch(0, kind == "ln", m, n, dtype)
            b = _launch.query_launch(1, kind == "ln", m, n, dtype)
            announce(f"row groups N={n} M={m} {kind} {dtype} fwd={f} bwd={b}")
            assert f[:3] == want, f
            assert f[2] // f[1] == b[2] // b[1], (f, b)
        if want[0] == 3 and n_vecs <= 96:
            big = (32 << 20) // (n * (16 // vec))
            assert _launch.query_launch(0, kind == "ln", big, n, dtype)[:3] == (3, want[1], 256)
        x = torch.randn(37, n, generator=g).to(dtype); dy = torch.randn(37, n, generator=g).to(dtype)
        w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype)
        b = (0.1 * torch.randn(n, generator=g)).to(dtype) if kind == "ln" else None
        run_and_compare(kind, x, dy, w, b, 1e-5, f"row groups N={n} {kind}")
