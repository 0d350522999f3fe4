"""GPU parity of the flat mapping for the row p-norm / normalize family over narrow rows (csrc/thn_pnorm_flat.h):
rows of 1, 2 and 4 vectors and of up to 32 vectors whose count is not a power of two, float32 / float16 / bfloat16,
every integer p from 1 to 6, against the float64 CPU oracle with the tolerances of test_pnorm_parity_gpu.py; row counts
that end in the middle of a wave, a workgroup and a grid step; the launch query confirms which kernels ran; batched and
strided tensors (which the row kernels take when the batches do not fold); non-finite rows; bit-level determinism and
independence of a row's position."""
import pytest
import torch

from test_pnorm_parity_gpu import compare_norm, compare_normalize, make
from TritonHub import _native
from TritonHub.Normalization._launch import query_launch
from TritonHub.Ops import _launch as ops_launch
from TritonHub.Ops import norm, normalize

pytestmark = pytest.mark.gpu
FLAT_WIDTHS = [n for n in range(1, 33) if n <= 4 or n & (n - 1)]


def announce(msg):
    print(f"\n[pnorm flat] {msg}", flush=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_every_row_width_and_p(dtype):
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    for n_vecs in FLAT_WIDTHS:
        n = n_vecs * vec
        rows_per_block = 4 * (64 // n_vecs) * 2
        for m in sorted({1, rows_per_block - 1, 3 * rows_per_block + 5, 1000 + n_vecs}):
            for which in (4, 5, 6):
                q = query_launch(which, False, m, n, dtype)
                assert q[:3] == (2, n_vecs, 256) and q[4] == 1, (which, q)
            for p in (1, 2, 3, 4, 5, 6) if m > 1000 else (1, 2, 3):
                announce(f"{dtype} L={n_vecs} K={n} rows={m} p={p}")
                x, gn, gy = make((1, m, n), dtype, seed=n_vecs * 100 + p)
                compare_norm(x, gn, p, 1e-6, f"flat norm L={n_vecs} M={m} p={p}")
                compare_normalize(x, gy, p, 1e-6, f"flat normalize L={n_vecs} M={m} p={p}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_row_widths_off_the_128_bit_path(dtype):
    """Rows that are not a whole number of vectors: the flat kernels' unaligned-window instances (the last window
    overlaps its neighbour; its leading columns count once in the row sum)."""
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    for n_vecs in range(1, 33):           # powers of two included: off the path the flat kernels take those too
        rows_per_block = 4 * (64 // n_vecs) * 2
        for n in sorted({(n_vecs - 1) * vec + 1, n_vecs * vec - 1}):
            if n < vec:
                continue
            for m in sorted({1, rows_per_block - 1, 3 * rows_per_block + 5}):
                for which in (4, 5, 6):
                    q = query_launch(which, False, m, n, dtype)
                    assert q[:3] == (2, n_vecs, 256) and q[4] == 0, (which, q)
                for p in (1, 2, 3):
                    announce(f"{dtype} L={n_vecs} ragged K={n} rows={m} p={p}")
                    x, gn, gy = make((1, m, n), dtype, seed=n_vecs * 100 + p + n)
                    compare_norm(x, gn, p, 1e-6, f"flat ragged norm K={n} M={m} p={p}")
                    compare_normalize(x, gy, p, 1e-6, f"flat ragged normalize K={n} M={m} p={p}")


def test_override_keeps_the_row_kernels_reachable():
    lib = _native.lib()
    try:
        for which in (4, 5, 6):
            assert lib.thn_norm_set_launch_override(which, 1, 8, 256, 0) == 0
            assert query_launch(which, False, 5000, 24, torch.float32)[:3] == (1, 8, 256)
            assert lib.thn_norm_set_launch_override(which, 2, 6, 0, 3) == 0
            assert query_launch(which, False, 5000, 24, torch.float32)[:3] == (2, 6, 256)
    finally:
        for which in (4, 5, 6):
            lib.thn_norm_set_launch_override(which, 0, 0, 0, 0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_batches_views_and_many_rows(dtype):
    """(B, M, K) tensors: dense ones fold into one run of rows (flat kernels); a view whose batches do not fold goes to
    the row kernels; a view of column blocks with a uniform row pitch stays flat and must leave the padding alone."""
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    k = 3 * vec
    announce(f"{dtype} dense (7, 333, {k})")
    x, gn, gy = make((7, 333, k), dtype, seed=1)
    compare_norm(x, gn, 2, 1e-6, "dense batches")
    compare_normalize(x, gy, 2, 1e-6, "dense batches")
    announce(f"{dtype} batches that do not fold")
    big = torch.randn(5, 40, k, generator=torch.Generator().manual_seed(2)).to(dtype).cuda()
    view = big[:, :33]                                   # batch stride 40 rows, 33 rows each
    compare_norm(view.cpu(), gn[:5, :33], 3, 1e-6, "unfolded batches", x_gpu=view.detach())
    compare_normalize(view.cpu(), gy[:5, :33], 3, 1e-6, "unfolded batches", x_gpu=view.detach())
    announce(f"{dtype} column blocks")
    wide = torch.randn(1, 2000, 4 * k, generator=torch.Generator().manual_seed(3)).to(dtype).cuda()
    block = wide[:, :, k:2 * k]
    gyb = torch.randn(1, 2000, k, generator=torch.Generator().manual_seed(4)).to(dtype)
    compare_norm(block.cpu(), torch.rand(1, 2000).to(dtype), 2, 1e-6, "column block", x_gpu=block.detach())
    compare_normalize(block.cpu(), gyb, 1, 1e-6, "column block", x_gpu=block.detach())
    announce(f"{dtype} 2^21 rows of {k}")
    g = torch.Generator(device="cuda").manual_seed(5)
    m = (1 << 21) + 3
    xl = torch.randn(1, m, k, device="cuda", generator=g).to(dtype)
    gl = torch.randn(1, m, k, device="cuda", generator=g).to(dtype)
    y, n = ops_launch.normalize_fwd(xl, 2, 1e-12)
    assert torch.equal(ops_launch.norm_fwd(xl, 2, 1e-12), n)
    unit = y.float().pow(2).sum(-1).sqrt()
    # bfloat16: the stored norm and every stored element carry up to 2^-9 of relative rounding each, and over 24
    # elements the element roundings do not average out
    assert float((unit - 1).abs().max()) < (1e-6 if dtype == torch.float32 else 2.0 ** -7)
    dx = ops_launch.normalize_bwd(xl, y, n, gl, 2)
    idx = torch.tensor([0, 1, 4095, 4096, m // 2, m - 2, m - 1], device="cuda")
    compare_normalize(xl[:, idx].cpu(), gl[:, idx].cpu(), 2, 1e-12, "spot rows of 2^21")
    y_s, n_s = ops_launch.normalize_fwd(xl[:, idx].contiguous(), 2, 1e-12)
    assert torch.equal(y_s, y[:, idx]) and torch.equal(n_s, n[:, idx])       # a row's result does not depend on its place
    dx_s = ops_launch.normalize_bwd(xl[:, idx].contiguous(), y_s, n_s, gl[:, idx].contiguous(), 2)
    assert torch.equal(dx_s, dx[:, idx])
    y2, n2 = ops_launch.normalize_fwd(xl, 2, 1e-12)
    assert torch.equal(y2, y) and torch.equal(n2, n)
    assert torch.equal(ops_launch.normalize_bwd(xl, y, n, gl, 2), dx)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_non_finite_zero_and_overflowing_rows(dtype):
    """As test_non_finite_and_overflowing_rows of the row kernels, on rows of 3 vectors."""
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    n = 3 * vec
    announce(f"flat pnorm non-finite K={n} {dtype}")
    x = torch.randn(1, 6, n, generator=torch.Generator().manual_seed(n)).to(dtype)
    x[0, 1, 1] = float("inf"); x[0, 2, 2] = float("nan"); x[0, 3, 3] = float("-inf")
    x[0, 4] = 0.0
    x[0, 5] = 1e30
    eps = 1e-6
    eps_st = float(torch.tensor(eps).to(dtype))
    inf = float("inf")
    for p in (1, 2, 3):
        xg = x.cuda().requires_grad_(True)
        nrm = norm(p=p, eps=eps)(xg)
        nrm.backward(torch.ones_like(nrm))
        got = nrm.detach().float().cpu()[0]
        assert float(got[1]) == inf and float(got[3]) == inf, f"p={p}: {got}"
        assert float(got[2]) == eps_st and float(got[4]) == eps_st, f"p={p}: {got}"
        if p != 1:
            assert float(got[5]) == inf
            if p == 2:
                assert bool((xg.grad[0, 5] == 0).all())
        assert bool(torch.isfinite(xg.grad[0, 0]).all())
        xg = x.cuda().requires_grad_(True)
        y = normalize(p=p, eps=eps)(xg)
        y.backward(torch.ones_like(y))
        yc = y.detach().float().cpu()[0]
        assert bool((yc[4] == 0).all())
        for r in (1, 3):
            hit = torch.zeros(n, dtype=torch.bool); hit[r] = True
            assert bool(torch.isnan(yc[r][hit]).all()) and bool((yc[r][~hit] == 0).all()), f"p={p} row {r}"
        if p != 1:
            assert bool((yc[5] == 0).all())
            if p == 2:
                assert bool((xg.grad[0, 5] == 0).all())
        assert bool(torch.isfinite(yc[0]).all()) and bool(torch.isfinite(xg.grad[0, 0]).all())
