"""GPU parity of the lane-per-row kernels for rows shorter than one 16-byte vector (csrc/thn_tiny.h): LayerNorm / RMSNorm,
softmax / softmin / log-softmax and row p-norm / normalize over 1 to 3 float32 columns and 1 to 7 columns of a 16-bit type, against the CPU
oracle with the tolerances of the families' parity tests; row counts around a wave, a workgroup and a grid step (dense
rows behind aligned pointers go through LDS in whole vectors, the last incomplete batch of 64 rows by element accesses);
rows that are columns of a wider buffer and rows behind a misaligned pointer (element accesses); masked logits; tensors whose batches do not fold (the row kernels' element-wise
instance takes those, as it does under a launch override); run-to-run identical results."""
import pytest
import torch

import test_softmax_parity_gpu as sm
from test_pnorm_parity_gpu import compare_norm, compare_normalize, make
from TritonHub import _native
from TritonHub.Normalization._launch import query_launch
from TritonHub.Ops import _launch as ops_launch

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def announce(msg):
    print(f"\n[tiny rows] {msg}", flush=True)


def widths(dtype):
    return range(1, 16 // torch.empty(0, dtype=dtype).element_size())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["softmax", "softmin", "logsoftmax"])
def test_softmax_family_over_every_short_width(kind, dtype):
    for n in widths(dtype):
        for m in (1, 63, 257, 4 * 256 + 3, 70001):
            announce(f"{kind} {dtype} N={n} M={m}")
            for which in (2, 3):
                q = query_launch(which, False, m, n, dtype)
                assert q[:3] == (4, 1, 256) and q[4] == 0, q
            x, dy = sm.make((m, n), dtype, 31 * n + m % 97, scale=3.0)
            sm.run_and_compare(kind, x, dy, f"tiny {kind} N={n} M={m}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_pnorm_family_over_every_short_width(dtype):
    for n in widths(dtype):
        # (a few hundred rows: among many thousand random rows of two or three columns some are nearly one-dimensional,
        # where the normalize backward cancels and the float32 bound of the parity tests, 4 ulp of the RESULT, no longer
        # describes float32 arithmetic; the row count classes are covered by the softmax test and the property test)
        for m in (1, 63, 4 * 256 + 3):
            for which in (4, 5, 6):
                q = query_launch(which, False, m, n, dtype)
                assert q[:3] == (4, 1, 256) and q[4] == 0, (which, q)
            for p in (1, 2, 3, 4, 5, 6) if m == 63 else (1, 2, 3):
                announce(f"pnorm {dtype} K={n} rows={m} p={p}")
                x, gn, gy = make((1, m, n), dtype, seed=n * 100 + p)
                compare_norm(x, gn, p, 1e-6, f"tiny norm K={n} M={m} p={p}")
                if n > 1 or p == 2:
                    compare_normalize(x, gy, p, 1e-6, f"tiny normalize K={n} M={m} p={p}")
                    continue
                # One column and p != 2: the normalize backward is g / |x| - sign(x) |x|^(p-1) (y g) / |x|^p, an exact 0
                # reached as the difference of two roundings of g / |x| -- the absolute bound of the parity tests does
                # not apply; the bound here is a few float32 roundings of that magnitude.
                xg = x.cuda()
                y, nrm = ops_launch.normalize_fwd(xg, p, 1e-6)
                dx = ops_launch.normalize_bwd(xg, y, nrm, gy.cuda(), p)
                bound = 16 * 2.0 ** -24 * gy.float().abs() / x.float().abs().clamp_min(1e-6)
                assert bool((dx.float().cpu().abs() <= bound + 1e-30).all()), f"tiny normalize K=1 p={p}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["ln", "rms"])
def test_norm_kernels_over_every_short_width(kind, dtype):
    """LayerNorm / RMSNorm over fewer columns than a vector holds: y, the saved statistics, dx, dW and dB against the
    oracle (eps = 1e-2: rows of a few elements are often nearly constant, and with a tiny eps rstd multiplies the float32
    rounding of x - mean beyond any fixed bound); 16-bit and float32 parameters; rows as columns of a wider buffer."""
    from parity_util import compare_with_oracle, run_and_compare
    from TritonHub.Normalization.layernorm import layernorm
    from TritonHub.Normalization.rmsnorm import rmsnorm
    g = torch.Generator().manual_seed(41)
    for n in widths(dtype):
        for m in (1, 63, 4 * 256 + 3, 70001):
            announce(f"{kind} {dtype} N={n} M={m}")
            for which in (0, 1):
                q = query_launch(which, kind == "ln", m, n, dtype)
                assert q[:3] == (4, 1, 256) and q[4] == 0, q
            x = (torch.randn(m, n, generator=g) * 2 + 0.5).to(dtype)
            dy = torch.randn(m, n, generator=g).to(dtype)
            w = 1 + 0.1 * torch.randn(n, generator=g)
            b = 0.1 * torch.randn(n, generator=g) if kind == "ln" else None
            run_and_compare(kind, x, dy, w.to(dtype), None if b is None else b.to(dtype), 1e-2, f"tiny {kind} N={n} M={m}")
            if m == 63 and dtype != torch.float32:
                run_and_compare(kind, x, dy, w, b, 1e-2, f"tiny {kind} N={n} M={m}, float32 parameters")
        # columns 2 .. 2 + n of a buffer of n + 5 columns
        m = 3001
        xb = (torch.randn(m, n + 5, generator=g) * 2 + 0.5).to(dtype)
        gb = torch.randn(m, n + 5, generator=g).to(dtype)
        x, dy = xb[:, 2:2 + n].contiguous(), gb[:, 2:2 + n].contiguous()
        w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype)
        b = (0.1 * torch.randn(n, generator=g)).to(dtype) if kind == "ln" else None
        xg = xb.cuda()[:, 2:2 + n].detach().requires_grad_(True)
        wg = w.cuda().requires_grad_(True)
        bg = None if b is None else b.cuda().requires_grad_(True)
        if kind == "ln":
            y = layernorm.apply(xg, wg, bg, 1e-2)
            mean, rstd = y.grad_fn.saved_tensors[3], y.grad_fn.saved_tensors[4]
        else:
            y = rmsnorm.apply(xg, wg, 1e-2)
            mean, rstd = None, y.grad_fn.saved_tensors[2]
        y.backward(gb.cuda()[:, 2:2 + n])
        torch.cuda.synchronize()
        out = dict(y=y.detach(), dx=xg.grad, dw=wg.grad, db=None if bg is None else bg.grad, mean=mean, rstd=rstd)
        compare_with_oracle(kind, x, dy, w, b, 1e-2, out, f"tiny {kind} N={n} column block")


def test_norm_kernels_short_rows_bits():
    """Run-to-run identical (dW / dB are summed in a fixed order); dense rows (through LDS in whole vectors) and the same
    rows behind a misaligned pointer (element accesses) agree to float32 rounding."""
    from TritonHub.Normalization import _launch as nl
    g = torch.Generator().manual_seed(8)
    m, n = 300001, 3
    x = torch.randn(m, n, generator=g).cuda(); dy = torch.randn(m, n, generator=g).cuda()
    w = (1 + 0.1 * torch.randn(n, generator=g)).cuda(); b = (0.1 * torch.randn(n, generator=g)).cuda()

    def run(xx, gg):
        y, mean, rstd = nl.norm_fwd(xx, w, b, 1e-5, True)
        dx, dw, db = nl.norm_bwd(xx, gg, w, b, mean, rstd, True)
        torch.cuda.synchronize()
        return y, mean, rstd, dx, dw, db

    first = run(x, dy)
    for u, v in zip(first, run(x, dy)):
        assert torch.equal(u, v)
    store = torch.empty(m * n + 1, device="cuda"); gstore = torch.empty(m * n + 1, device="cuda")
    xm = store[1:].view(m, n); gm = gstore[1:].view(m, n)
    xm.copy_(x); gm.copy_(dy)
    assert xm.data_ptr() % 16 != 0
    for u, v in zip(first, run(xm, gm)):
        assert torch.allclose(u, v, rtol=2e-5, atol=2e-5)      # two compiled forms of one formula: float32 roundings apart


@pytest.mark.parametrize("dtype", DTYPES)
def test_normalize_properties_over_many_short_rows(dtype):
    """2^20 + 3 rows of 3 columns: unit norms, the fused forward stores the norms of the norm-only forward, the gradient
    is orthogonal to x (p = 2), run-to-run identical, a row's result does not depend on where it sits."""
    g = torch.Generator(device="cuda").manual_seed(5)
    m = (1 << 20) + 3
    x = (torch.randn(1, m, 3, device="cuda", generator=g) + 0.5).to(dtype)
    gy = torch.randn(1, m, 3, device="cuda", generator=g).to(dtype)
    y, n = ops_launch.normalize_fwd(x, 2, 1e-12)
    assert torch.equal(ops_launch.norm_fwd(x, 2, 1e-12), n)
    unit = y.float().pow(2).sum(-1).sqrt()
    assert float((unit - 1).abs().max()) < (1e-6 if dtype == torch.float32 else 2.0 ** -7)
    dx = ops_launch.normalize_bwd(x, y, n, gy, 2)
    scale = (gy.float().abs().sum(-1) / n.float()).clamp_min(1e-30)
    dot = (dx.double() * y.double()).sum(-1).abs().float()
    assert bool((dot <= (1e-5 if dtype == torch.float32 else 3e-2) * scale).all())
    y2, n2 = ops_launch.normalize_fwd(x, 2, 1e-12)
    assert torch.equal(y, y2) and torch.equal(n, n2) and torch.equal(ops_launch.normalize_bwd(x, y, n, gy, 2), dx)
    idx = torch.tensor([0, 1, 255, 256, 4095, m // 2, m - 2, m - 1], device="cuda")
    ys, ns = ops_launch.normalize_fwd(x[:, idx].contiguous(), 2, 1e-12)
    assert torch.equal(ys, y[:, idx]) and torch.equal(ns, n[:, idx])
    assert torch.equal(ops_launch.normalize_bwd(x[:, idx].contiguous(), ys, ns, gy[:, idx].contiguous(), 2), dx[:, idx])


def test_views_batches_masks_override_and_determinism():
    g = torch.Generator().manual_seed(3)
    # columns 5..7 of a buffer of 11 columns: a row pitch wider than the row; the padding must stay untouched
    announce("softmax f32 on a column block")
    buf = torch.randn(3000, 11, generator=g).cuda()
    view = buf[:, 5:8]
    x = view.cpu().contiguous()
    dy = torch.randn(3000, 3, generator=g)
    before = buf.clone()
    sm.run_and_compare("softmax", x, dy, "tiny softmax column block", x_gpu=view.detach())
    assert torch.equal(buf, before)
    # a (B, M, K) tensor whose batches fold (dense) and one whose batches do not (the element-wise row kernel)
    announce("normalize f32 batches")
    x, gn, gy = make((6, 500, 3), torch.float32, seed=9)
    compare_norm(x, gn, 2, 1e-6, "tiny norm dense batches")
    compare_normalize(x, gy, 2, 1e-6, "tiny normalize dense batches")
    big = torch.randn(6, 520, 3, generator=g).cuda()
    sub = big[:, :500]
    compare_norm(sub.cpu(), gn, 3, 1e-6, "tiny norm unfolded batches", x_gpu=sub.detach())
    compare_normalize(sub.cpu(), gy, 3, 1e-6, "tiny normalize unfolded batches", x_gpu=sub.detach())
    # masked logits: exact zeros, a fully masked row is NaN
    announce("masked logits bf16 N=5")
    from TritonHub.Activations import Softmax
    xm = torch.randn(1000, 5, generator=g)
    xm[torch.rand(1000, 5, generator=g) < 0.3] = float("-inf")
    xm[11] = float("-inf")
    y = Softmax()(xm.bfloat16().cuda()).float().cpu()
    ref = torch.softmax(xm.bfloat16().double(), -1)
    keep = ~torch.isnan(ref).any(-1)
    assert bool(torch.isnan(y[11]).all()) and bool((y[keep][xm[keep] == float("-inf")] == 0).all())
    assert torch.allclose(y[keep].double(), ref[keep], atol=4e-3)
    # dense rows behind a pointer one element off 16 bytes: the element accesses instead of the staged vectors
    announce("misaligned base")
    for dtype, n in ((torch.bfloat16, 5), (torch.float32, 3)):
        m = 5000
        x, dy = sm.make((m, n), dtype, 17, scale=2.0)
        store = torch.empty(m * n + 1, dtype=dtype, device="cuda")
        xg = store[1:].view(m, n)
        xg.copy_(x)
        assert xg.data_ptr() % 16 != 0
        sm.run_and_compare("softmax", x, dy, f"tiny softmax misaligned {dtype}", x_gpu=xg)
    # a launch override keeps the row kernels' element-wise instance reachable; both give the oracle's results
    announce("override")
    lib = _native.lib()
    try:
        for which in (2, 3):
            assert lib.thn_norm_set_launch_override(which, 4, 8, 256, 0) == 0
            assert query_launch(which, False, 999, 3, torch.float32)[:3] == (4, 8, 256)
        x, dy = sm.make((999, 3), torch.float32, 5, scale=2.0)
        sm.run_and_compare("logsoftmax", x, dy, "element-wise row kernel N=3")
    finally:
        for which in (2, 3):
            lib.thn_norm_set_launch_override(which, 0, 0, 0, 0)
    # run to run
    announce("determinism")
    x, dy = sm.make((200003, 3), torch.float32, 6, scale=2.0)
    y1, dx1 = sm.run_and_compare("softmax", x, dy, "tiny determinism")
    y2, dx2 = sm.run_and_compare("softmax", x, dy, "tiny determinism again")
    assert torch.equal(y1, y2) and torch.equal(dx1, dx2)
