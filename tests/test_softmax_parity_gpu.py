"""GPU parity tests of Softmax / Softmin / LogSoftmax: the HIP path, called through the operator interface and
the C ABI, against the float64 CPU oracle on the same seeded inputs.

Tolerances (as for the norm path): float32 storage max(1e-5, 4 float32 ulp); float16 / bfloat16 1 ulp of the
output type at the oracle's value plus 4 * 2^-24 * (magnitude of the operands that were subtracted to form
the result); float64 softmax / softmin are computed in float64 (as the reference does) and held to 1e-13,
float64 log-softmax is float32 arithmetic (logsoftmax.py:19) and held to the float32 bound.
The backward is a function of the SAVED OUTPUT (softmax.py:86-97): its expected value is the oracle's backward
evaluated at the very output tensor the GPU saved, so forward rounding does not leak into the comparison.
"""
import os
import re

import numpy as np
import pytest
import torch

from conftest import ROOT, check_elementwise, f64
from oracle import softmax_oracle as so
from TritonHub import _native
from TritonHub.Activations import LogSoftmax, Softmax, Softmin, _launch
from TritonHub.Activations.logsoftmax import logsoftmax
from TritonHub.Activations.softmax import softmax
from TritonHub.Activations.softmin import softmin

pytestmark = pytest.mark.gpu
KINDS = ["softmax", "softmin", "logsoftmax"]
MODULE = {"softmax": Softmax, "softmin": Softmin, "logsoftmax": LogSoftmax}
CODE = {"softmax": _native.SOFTMAX, "softmin": _native.SOFTMIN, "logsoftmax": _native.LOGSOFTMAX}


def announce(msg):
    print(f"\n[case] {msg}", flush=True)


def check(got, ref, scale, dtype, kind, what):
    if dtype == torch.float64 and kind != "logsoftmax":
        err = np.abs(f64(got) - ref)
        bound = 1e-13 * np.maximum(1.0, np.abs(ref))
        assert (err <= bound).all(), f"{what}: float64 error {err.max():.3e}"
        return
    check_elementwise(f64(got), ref, scale, dtype, what)


def run_and_compare(kind, x, dy, what, chunk_rows=4096, x_gpu=None, dy_gpu=None):
    """x, dy: CPU tensors in the storage dtype.  Forward + backward through the callable, compared in row chunks.
    `x_gpu` / `dy_gpu`: the same values already on the device (to keep a view's strides)."""
    dtype = x.dtype
    xg = (x.cuda() if x_gpu is None else x_gpu).requires_grad_(True)
    y = MODULE[kind]()(xg)
    y.backward(dy.cuda() if dy_gpu is None else dy_gpu)
    torch.cuda.synchronize()
    assert y.dtype == dtype and y.shape == x.shape and xg.grad.dtype == dtype and xg.grad.shape == x.shape
    n = x.shape[-1]
    x2, dy2 = x.reshape(-1, n), dy.reshape(-1, n)
    y2, dx2 = y.detach().reshape(-1, n).cpu(), xg.grad.reshape(-1, n).cpu()
    for s in range(0, x2.shape[0], chunk_rows):
        e = min(s + chunk_rows, x2.shape[0])
        xc, gc = f64(x2[s:e]), f64(dy2[s:e])
        yo = so.FWD[kind](xc)
        if kind == "logsoftmax":
            z = (xc - xc.max(1, keepdims=True))
            # y = z - log(sum): the two cancel near the row maximum; and the float32 sum of exponentials (>= 1) carries
            # a RELATIVE rounding error per addition, which is an ABSOLUTE error of that size in its logarithm (the "+ 1":
            # a row whose maximum dominates has log(sum) ~ 1e-4, far below the error of the sum it is the logarithm of)
            scale = np.abs(z) + np.abs(yo - z) + 1.0
        else:
            scale = np.abs(yo)
        check(y2[s:e], yo, scale, dtype, kind, f"{what} y rows {s}:{e}")
        ys = f64(y2[s:e])                               # the saved output, as stored
        dxo = so.BWD[kind](ys, gc)
        if kind == "logsoftmax":
            scale = np.abs(gc) + np.exp(ys) * np.abs(gc).sum(1, keepdims=True)
        else:
            scale = np.abs(ys) * (np.abs(gc) + np.abs(ys * gc).sum(1, keepdims=True))
        check(dx2[s:e], dxo, scale, dtype, kind, f"{what} dx rows {s}:{e}")
    return y.detach(), xg.grad


def make(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(shape, generator=g) * scale).to(dtype)
    dy = torch.randn(shape, generator=g).to(dtype)
    return x, dy


# ---- the reference's unit-test matrix (UnitTests/Activations/softmax_unittest.py:57-65 and twins) ---------------
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.float64])
@pytest.mark.parametrize("dim", [32, 64, 128, 256, 512, 1024, 2048])
@pytest.mark.parametrize("kind", KINDS)
def test_reference_unit_test_matrix(kind, dim, dtype):
    announce(f"reference matrix {kind} D={dim} {dtype}")
    torch.manual_seed(42)
    data = torch.randn(1, 256, 256, dim, device="cuda", dtype=dtype)
    theirs = {"softmax": torch.nn.Softmax(dim=-1), "softmin": torch.nn.Softmin(dim=-1),
              "logsoftmax": torch.nn.LogSoftmax(dim=-1)}[kind]
    a = data.clone().requires_grad_(True)
    r = data.clone().requires_grad_(True)
    rtol, atol = (3e-4, 1e-3) if dtype == torch.float32 else (5e-3, 1e-2)      # softmax_unittest.py:30-32
    if dtype == torch.float16:
        rtol, atol = 1e-2, 5e-2
    ya, yr = MODULE[kind]()(a), theirs(r)
    assert torch.allclose(ya, yr, atol=atol, rtol=rtol), "Error in forward pass"
    g = torch.randn_like(ya)
    ya.backward(g); yr.backward(g)
    assert torch.allclose(a.grad, r.grad, atol=atol, rtol=rtol), "Error in backward pass"
    # and the real bar, on a slice of the same data, against the oracle
    x = data[0, :16].cpu()
    run_and_compare(kind, x, g[0, :16].cpu(), f"{kind} D={dim} {dtype}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize("n", [1, 2, 7, 33, 100, 257, 1000, 4099, 6001])
@pytest.mark.parametrize("kind", KINDS)
def test_ragged_row_widths(kind, n, dtype):
    announce(f"ragged {kind} N={n} {dtype}")
    x, dy = make((37, n), dtype, seed=n, scale=3.0)
    run_and_compare(kind, x, dy, f"{kind} N={n} {dtype}")


@pytest.mark.parametrize("dtype,n_max", [(torch.float32, 16384), (torch.bfloat16, 32768), (torch.float16, 32768),
                                         (torch.float64, 8192)])
@pytest.mark.parametrize("kind", KINDS)
def test_row_width_limit(kind, dtype, n_max):
    announce(f"row limit {kind} {dtype} N={n_max}")
    x, dy = make((6, n_max), dtype, seed=5, scale=2.0)
    run_and_compare(kind, x, dy, f"{kind} N={n_max}")
    # one vector beyond what the row engine holds: the looping kernels, still one softmax of the whole row
    x, dy = make((6, n_max + 8), dtype, seed=6, scale=2.0)
    run_and_compare(kind, x, dy, f"{kind} N={n_max + 8}")


@pytest.mark.parametrize("dtype,widths", [(torch.float32, (32000, 50257, 128256)), (torch.bfloat16, (50257, 128256)),
                                          (torch.float16, (65536 + 3,)), (torch.float64, (8192 + 5, 20001))])
@pytest.mark.parametrize("kind", KINDS)
def test_rows_wider_than_64_kib(kind, dtype, widths):
    """Vocabulary-sized rows: more rows than workgroups at the narrowest width, ragged and misaligned rows, -inf
    entries (masked logits) at the start of a row, where the running maximum is still -inf."""
    for n in widths:
        announce(f"wide rows {kind} {dtype} N={n}")
        m = 300 if n <= 50257 else 5
        x, dy = make((m, n), dtype, seed=n, scale=3.0)
        if kind == "softmax":
            x[:, :17] = float("-inf")
            x[0, 100:n - 5] = float("-inf")
        elif kind == "softmin":
            x[:, :17] = float("inf")
        else:
            x[:, :17] = -3.0e4                  # log-softmax of -inf is -inf: keep the outputs finite
        run_and_compare(kind, x, dy, f"{kind} wide N={n}")


@pytest.mark.parametrize("kind", KINDS)
def test_large_logits_and_saturated_rows(kind):
    """Rows whose entries span hundreds of units (exp underflows for most columns), a row with one dominant entry,
    a constant row: the maximum is subtracted first, so nothing overflows and the closed forms hold."""
    announce(f"large logits {kind}")
    g = torch.Generator().manual_seed(8)
    x = torch.randn(64, 512, generator=g) * 60.0
    x[0] = 0.25
    x[1] = -1000.0; x[1, 17] = 1000.0
    dy = torch.randn(64, 512, generator=g)
    y, _ = run_and_compare(kind, x, dy, f"{kind} large logits")
    assert bool(torch.isfinite(y[2:]).all()) or kind == "logsoftmax"
    if kind == "logsoftmax":
        assert torch.allclose(y[0].cpu(), torch.full((512,), -float(np.log(512.0))), atol=2e-6)
        assert float(y[1, 17]) == 0.0
    else:
        assert torch.allclose(y[0].cpu(), torch.full((512,), 1.0 / 512), rtol=1e-6)
        hot = 17 if kind == "softmax" else None
        if hot is not None:
            assert float(y[1, hot]) == 1.0 and float(y[1].sum()) == 1.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [8, 100, 333, 2048, 4104])
@pytest.mark.parametrize("kind", ["softmax", "logsoftmax"])
def test_masked_logits(kind, n, dtype):
    """Attention-style masks: row i keeps its first i % n + 1 logits and has -inf in the rest; one row is masked
    completely.  Masked columns come out as exactly 0 (softmax) or -inf (log-softmax) and receive exactly 0 / the
    upstream gradient; a row without any finite logit is NaN, as exp(-inf - -inf) makes it in the reference
    (softmax.py:33-37) and in torch; the columns that are kept match the float64 values."""
    announce(f"masked logits {kind} n={n} {dtype}")
    rows = min(n, 257) + 3
    g = torch.Generator().manual_seed(n)
    x = torch.randn(rows, n, generator=g).to(dtype)
    dy = torch.randn(rows, n, generator=g).to(dtype)
    keep = (torch.arange(rows) % n + 1)[:, None]
    masked = torch.arange(n)[None, :] >= keep
    x[masked] = float("-inf")
    x[rows - 2] = float("-inf")
    dead = torch.zeros(rows, dtype=torch.bool); dead[rows - 2] = True
    xg = x.cuda().requires_grad_(True)
    y = MODULE[kind]()(xg)
    y.backward(dy.cuda())
    torch.cuda.synchronize()
    y, dx = y.detach().cpu(), xg.grad.cpu()
    assert bool(torch.isnan(y[dead]).all()) and bool(torch.isnan(dx[dead]).all())
    live = ~dead
    m_live = masked[live]
    y_l, dx_l, dy_l = y[live], dx[live], dy[live]
    if kind == "softmax":
        assert bool((y_l[m_live] == 0).all()) and bool((dx_l[m_live] == 0).all())
    else:
        assert bool((y_l[m_live] == float("-inf")).all()) and bool((dx_l[m_live] == dy_l[m_live]).all())
    xr = x[live].double()
    fn = torch.softmax if kind == "softmax" else torch.log_softmax
    yr = fn(xr, -1)
    ys, gd = y_l.double(), dy_l.double()        # the backward is a function of the saved output (softmax.py:86-97)
    if kind == "softmax":
        dxr = ys * (gd - (ys * gd).sum(-1, keepdim=True))
    else:
        dxr = gd - torch.exp(ys) * gd.sum(-1, keepdim=True)
    eps = {torch.float32: 2.0 ** -19, torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}[dtype]     # loose: the mask pattern is the point
    kept = ~m_live
    for got, ref, what in ((y_l, yr.detach(), "y"), (dx_l, dxr, "dx")):
        err = (got.double() - ref)[kept].abs()
        scale = ref[kept].abs() + 1.0
        assert bool((err <= eps * scale + 1e-30).all()), f"{kind} masked {what}: {float((err / (scale + 1e-30)).max()):.3e}"
    assert bool(torch.isfinite(y_l[kept]).all()) and bool(torch.isfinite(dx_l).all())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64])
@pytest.mark.parametrize("kind", KINDS)
def test_strides_views_and_batch_shapes(kind, dtype):
    announce(f"strides {kind} {dtype}")
    g = torch.Generator().manual_seed(12)
    base = (torch.randn(40, 640, generator=g) * 2).to(dtype)
    gbase = torch.randn(40, 640, generator=g).to(dtype)
    bg, gg = base.cuda(), gbase.cuda()
    for i, view in enumerate((lambda t: t[:, :512], lambda t: t[:, 3:515], lambda t: t[::2, 64:576],
                              lambda t: t.t()[:600, :32], lambda t: t[:, :512].reshape(5, 8, 512),
                              lambda t: t[0, :512], lambda t: t[:, 5:6], lambda t: t[3:4].expand(6, 640))):
        xv, gv = view(base), view(gbase)
        y, dx = run_and_compare(kind, xv.contiguous(), gv.contiguous(), f"{kind} view {i}", x_gpu=view(bg).detach(),
                                dy_gpu=view(gg))
        assert y.shape == xv.shape and dx.shape == xv.shape and y.is_contiguous()


def test_empty_input_and_single_element_rows():
    announce("softmax empty / N=1")
    for kind in KINDS:
        mod = MODULE[kind]()
        x = torch.empty(0, 64, device="cuda", requires_grad=True)
        y = mod(x)
        y.sum().backward()
        assert y.shape == (0, 64) and x.grad.shape == (0, 64)
        one = torch.randn(9, 1, device="cuda", requires_grad=True)
        y1 = mod(one)
        y1.backward(torch.randn(9, 1, device="cuda"))
        expect = 0.0 if kind == "logsoftmax" else 1.0
        assert bool((y1 == expect).all()) and bool((one.grad == 0).all())


def test_softmin_function_and_callable_follow_the_reference():
    """softmin.apply(z) is softmax(z) (softmin.py:86-97); Softmin()(x) is softmin.apply(-x) (softmin.py:103):
    values and gradients of the fused callable equal those of the explicit negation bit for bit."""
    announce("softmin semantics")
    g = torch.Generator().manual_seed(77)
    for dtype in (torch.float32, torch.bfloat16, torch.float64):
        x = (torch.randn(300, 777, generator=g) * 4).to(dtype).cuda()
        dy = torch.randn(300, 777, generator=g).to(dtype).cuda()
        a = x.clone().requires_grad_(True)
        b = x.clone().requires_grad_(True)
        c = x.clone().requires_grad_(True)
        ya = Softmin()(a); ya.backward(dy)
        yb = softmin.apply(-b); yb.backward(dy)
        yc = softmax.apply(-c); yc.backward(dy)
        assert torch.equal(ya, yb) and torch.equal(a.grad, b.grad)
        assert torch.equal(yb, yc) and torch.equal(b.grad, c.grad)
        assert torch.equal(softmin.apply(x), softmax.apply(x))
        assert Softmin().softmin_fn is not None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_properties_at_large_size(dtype):
    """Size-independent properties on 65536 x 4096: rows sum to one, shift invariance, exp(log-softmax) = softmax,
    gradients sum to zero over each row, determinism."""
    announce(f"softmax properties {dtype}")
    m, n = 65536, 4096
    g = torch.Generator(device="cuda").manual_seed(3)
    x = (torch.randn(m, n, device="cuda", generator=g) * 3).to(dtype)
    dy = torch.randn(m, n, device="cuda", generator=g).to(dtype)
    p = softmax.apply(x)
    tol = 2e-6 if dtype == torch.float32 else 4e-3          # half an ulp of bfloat16 is up to 2^-8 relative
    assert float((p.double().sum(1) - 1).abs().max()) < tol
    assert torch.equal(softmax.apply(x), p)
    small = ((x.float().clamp(-7, 7) * 4).round() / 4).to(dtype)      # multiples of 1/4: small + 8 is exact in bfloat16
    assert torch.equal((small + 8.0).float() - 8.0, small.float())
    assert torch.equal(softmax.apply(small + 8.0), softmax.apply(small))        # x - max(x) is the same float32 value
    lp = logsoftmax.apply(x)
    rel = ((lp.double().exp() - p.double()).abs() / p.double().clamp_min(1e-30)).max()
    assert float(rel) < (2e-5 if dtype == torch.float32 else 0.09)    # bfloat16: |lp| up to ~25, half an ulp is 0.06
    dx = _launch.softmax_bwd(p, dy, _native.SOFTMAX)
    ref_scale = float((p.double() * dy.double().abs()).sum(1).max())
    assert float(dx.double().sum(1).abs().max()) < (1e-5 if dtype == torch.float32 else 4e-3) * max(1.0, ref_scale) * 4
    dl = _launch.softmax_bwd(lp, dy, _native.LOGSOFTMAX)
    assert dl.shape == x.shape and bool(torch.isfinite(dl).all())
    assert torch.equal(_launch.softmax_bwd(p, dy, _native.SOFTMIN), -dx)
    # spot rows against the oracle
    idx = torch.tensor([0, 1, 31337, m - 1], device="cuda")
    for kind in KINDS:
        run_and_compare(kind, x[idx].cpu(), dy[idx].cpu(), f"{kind} spot rows")


def test_c_abi_direct_calls_and_errors():
    announce("softmax C ABI direct")
    lib = _native.lib()
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(19)
    m, n, pitch = 129, 768, 1024
    xb = (torch.randn(m, pitch, generator=g) * 2).cuda()
    gb = torch.randn(m, pitch, generator=g).cuda()
    for kind in KINDS:
        y = torch.full((m, pitch), 7.0, device="cuda"); dx = torch.full((m, pitch), 7.0, device="cuda")
        assert lib.thn_softmax_fwd(xb.data_ptr(), pitch, y.data_ptr(), pitch, m, n, CODE[kind], _native.F32, st) == 0
        assert lib.thn_softmax_bwd(y.data_ptr(), pitch, gb.data_ptr(), pitch, dx.data_ptr(), pitch, m, n, CODE[kind],
                                   _native.F32, st) == 0
        torch.cuda.synchronize()
        assert bool((y[:, n:] == 7.0).all()) and bool((dx[:, n:] == 7.0).all())        # padding untouched
        yo = so.FWD[kind](f64(xb[:, :n]))
        check_elementwise(f64(y[:, :n]), yo, np.abs(yo), torch.float32, f"C ABI {kind} y")
        dxo = so.BWD[kind](f64(y[:, :n]), f64(gb[:, :n]))
        check_elementwise(f64(dx[:, :n]), dxo, np.abs(dxo), torch.float32, f"C ABI {kind} dx")
    y = torch.empty(m, n, device="cuda")
    assert lib.thn_softmax_fwd(xb.data_ptr(), n - 1, y.data_ptr(), n, m, n, 0, _native.F32, st) == _native.E_SHAPE
    assert lib.thn_softmax_fwd(xb.data_ptr(), pitch, 0, n, m, n, 0, _native.F32, st) == _native.E_NULL
    assert lib.thn_softmax_fwd(xb.data_ptr(), pitch, y.data_ptr(), n, m, n, 5, _native.F32, st) == _native.E_SHAPE
    assert lib.thn_softmax_bwd(y.data_ptr(), n, 0, n, y.data_ptr(), n, m, n, 0, _native.F32, st) == _native.E_NULL


def compiled_forward_shapes():
    text = open(os.path.join(ROOT, "triton-hub_amd", "csrc", "thn_dispatch.h")).read()
    body = re.search(r"#define THN_FWD_SHAPES\(X\)(.*?)\n\n", text, re.S).group(1)
    body += re.search(r"#define THN_FWD_SHAPES_THREE\(X\)(.*?)\n\n", text, re.S).group(1)     # 3 x 16, 3 x 32
    text = open(os.path.join(ROOT, "triton-hub_amd", "csrc", "thn_softmax_dispatch.h")).read()
    five = re.search(r"#define THN_SM_SHAPES_FIVE\(X\)(.*?)\n\n", text, re.S).group(1)          # 5 x 32 ... 5 x 256
    assert len(re.findall(r"X\(5, ", five)) == 4
    body += five
    return [(int(k), int(t), int(b)) for k, t, b in re.findall(r"X\((\d+), (\d+), (\d+)\)", body)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float64])
def test_every_compiled_launch_shape(dtype):
    """Forces each softmax kernel instance through the launch override (forward: family 2, backward: family 3): on the
    128-bit path, and off it (one column short of a whole number of vectors: the unaligned-window instances, the last
    window overlapping its neighbour)."""
    from TritonHub.Normalization._launch import query_launch
    lib = _native.lib()
    shapes = compiled_forward_shapes()
    assert len(shapes) >= 20
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    g = torch.Generator().manual_seed(29)
    try:
        for k, tpr, block in shapes:
            for n_vecs in sorted({k * tpr, max((k - 1) * tpr + 1, k * tpr - tpr // 2 - 1)}):
                for n in (n_vecs * vec, n_vecs * vec - 1):
                    if n_vecs * 16 > 65536 or n < vec:
                        continue
                    on_path = n % vec == 0
                    rows_per_block = block // tpr
                    m = 2 * rows_per_block + max(1, rows_per_block // 2)
                    announce(f"softmax shape K={k} TPR={tpr} block={block} N={n} M={m} {dtype}")
                    assert lib.thn_norm_set_launch_override(2, k, tpr, block, 0) == 0
                    assert lib.thn_norm_set_launch_override(3, k, tpr, block, 0) == 0
                    for which in (2, 3):
                        q = query_launch(which, False, m, n, dtype)
                        assert q[:3] == (k, tpr, block) and q[4] == (1 if on_path else 0), q
                    x = (torch.randn(m, n, generator=g) * 2).to(dtype); dy = torch.randn(m, n, generator=g).to(dtype)
                    for kind in ("softmax", "logsoftmax"):
                        run_and_compare(kind, x, dy, f"{kind} K={k} TPR={tpr} block={block} N={n}")
    finally:
        lib.thn_norm_set_launch_override(2, 0, 0, 0, 0)
        lib.thn_norm_set_launch_override(3, 0, 0, 0, 0)


def test_launch_rules_of_rows_off_the_128_bit_path_and_of_the_backward():
    """The backward takes the forward's launch shape for rows of up to 512 vectors (the same rows per workgroup in
    both directions); off the 128-bit path in 16-bit storage the forward over 769 to 1024 vectors runs 2 x 512 in 512
    threads and the backward one workgroup per compute unit.  Each shape against the oracle."""
    from TritonHub.Normalization._launch import query_launch
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    bf16, f32 = torch.bfloat16, torch.float32
    for n, dt in ((512, bf16), (1792, bf16), (2048, bf16), (4096, bf16), (4095, bf16), (224, f32), (1024, f32), (2048, f32)):
        f = query_launch(2, False, 1 << 16, n, dt); b = query_launch(3, False, 1 << 16, n, dt)
        assert f[:3] == b[:3], (n, dt, f, b)
    assert query_launch(3, False, 8192, 8192, bf16)[:3] == (2, 512, 512)            # wider rows: 2 vectors per thread
    assert query_launch(2, False, 8192, 8191, bf16)[:4] == (2, 512, 512, cus)
    assert query_launch(2, False, 8192, 8191, f32)[:3] != (2, 512, 512)
    for n in (1025, 2050, 4098, 6001, 8191):
        assert query_launch(3, False, 1 << 16, n, bf16)[3] <= cus, n
        assert query_launch(2, False, 1 << 16, n, bf16)[3] == (cus if n == 8191 else 2 * cus), n
    for kind in KINDS:
        for n, dt in ((8191, bf16), (7001, torch.float16), (1792, bf16), (4095, bf16), (896, f32)):
            announce(f"launch rules {kind} N={n} {dt}")
            x, dy = make((21, n), dt, seed=n, scale=3.0)
            run_and_compare(kind, x, dy, f"{kind} N={n} {dt}")


def test_five_vector_shapes_for_rows_just_above_a_power_of_two_of_vectors():
    """Rows of 4 t + 1 to 5 t vectors (t = 32 ... 256) take 5 x t vectors per row in the forward; the backward follows
    where measured to pay.  The launches the library picks, each against the oracle."""
    from TritonHub.Normalization._launch import query_launch
    bf16, f16, f32 = torch.bfloat16, torch.float16, torch.float32
    want = {(1032, bf16): ((5, 32, 256), (5, 32, 256)), (1152, f16): ((5, 32, 256), (5, 32, 256)),
            (1280, bf16): ((5, 32, 256), (3, 64, 256)), (2056, bf16): ((5, 64, 256), (5, 64, 256)),
            (4104, f16): ((5, 128, 256), (5, 128, 256)), (5120, bf16): ((5, 128, 256), (3, 256, 256)),
            (8200, bf16): ((5, 256, 256), (5, 256, 256)), (10240, bf16): ((5, 256, 256), (3, 512, 512)),
            (516, f32): ((5, 32, 256), (5, 32, 256)), (2052, f32): ((5, 128, 256), (3, 256, 256)),
            (1025, bf16): ((5, 32, 256), (3, 64, 256)), (5001, bf16): ((5, 128, 256), (5, 128, 256)),
            (1024, bf16): ((4, 32, 256), (4, 32, 256)), (1288, bf16): ((3, 64, 256), (3, 64, 256))}
    for (n, dt), (f, b) in want.items():
        assert query_launch(2, False, 1 << 14, n, dt)[:3] == f, (n, dt)
        assert query_launch(3, False, 1 << 14, n, dt)[:3] == b, (n, dt)
    for kind in KINDS:
        for n, dt in ((1032, bf16), (1280, f16), (2056, bf16), (4104, f16), (8200, bf16), (516, f32), (2052, f32),
                      (1025, bf16), (5001, f16), (4098, bf16)):
            announce(f"five-vector shapes {kind} N={n} {dt}")
            x, dy = make((19, n), dt, seed=n, scale=3.0)
            run_and_compare(kind, x, dy, f"{kind} N={n} {dt}")
