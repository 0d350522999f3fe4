"""GPU parity tests of the row p-norm / normalize operators: the HIP path, called through the operator interface
and the C ABI, against the float64 CPU oracle on the same seeded inputs.

Every stage is compared as a function of what the reference's stage reads: the norms against the oracle's norms
of x; y against x divided by the norms THE GPU STORED (the reference's second kernel reads them back rounded to the
storage type, normalize.py:27); the backward passes against the oracle's backward at the saved tensors.
Tolerances: float32 / float64 storage max(1e-5, 4 float32 ulp); float16 / bfloat16 1 ulp of the output type plus
4 * 2^-24 * (magnitude of the operands that cancel).
"""
import os
import re

import numpy as np
import pytest
import torch

from conftest import ROOT, check_elementwise, f64
from oracle import pnorm_oracle as po
from TritonHub import _native
from TritonHub.Normalization._launch import query_launch
from TritonHub.Ops import norm, normalize
from TritonHub.Ops import _launch as ops_launch

pytestmark = pytest.mark.gpu
PS = [1, 2, 3, 4, 5, 6]


def announce(msg):
    print(f"\n[case] {msg}", flush=True)


def make(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(shape, generator=g) * scale).to(dtype)
    gn = torch.rand(shape[:-1], generator=g).to(dtype)
    gy = torch.randn(shape, generator=g).to(dtype)
    return x, gn, gy


def compare_norm(x, gn, p, eps, what, x_gpu=None):
    """norm forward + backward through the callable.  x, gn: CPU tensors in the storage dtype."""
    dtype = x.dtype
    xg = (x.cuda() if x_gpu is None else x_gpu).requires_grad_(True)
    n = norm(p=p, eps=eps)(xg)
    n.backward(gn.cuda())
    torch.cuda.synchronize()
    assert n.dtype == dtype and n.shape == x.shape[:-1] and n.is_contiguous()
    assert xg.grad.dtype == dtype and xg.grad.shape == x.shape
    x64 = f64(x)
    n_ref = po.norm_fwd(x64, p, eps)
    check_elementwise(f64(n), n_ref, n_ref, dtype, f"{what} norms")
    dx_ref = po.norm_bwd(x64, f64(n), f64(gn), p)                     # at the saved (stored) norms
    check_elementwise(f64(xg.grad), dx_ref, np.abs(dx_ref), dtype, f"{what} norm dx")
    return n.detach(), xg.grad


def compare_normalize(x, gy, p, eps, what, x_gpu=None, gy_gpu=None):
    dtype = x.dtype
    xg = (x.cuda() if x_gpu is None else x_gpu).requires_grad_(True)
    y = normalize(p=p, eps=eps)(xg)
    saved_x, saved_y, saved_n = y.grad_fn.saved_tensors
    y.backward(gy.cuda() if gy_gpu is None else gy_gpu)
    torch.cuda.synchronize()
    assert y.dtype == dtype and y.shape == x.shape and y.is_contiguous()
    assert saved_n.dtype == dtype and saved_n.shape == x.shape[:-1] and saved_y.data_ptr() == y.data_ptr()
    x64, g64 = f64(x), f64(gy)
    n_ref = po.norm_fwd(x64, p, eps)
    check_elementwise(f64(saved_n), n_ref, n_ref, dtype, f"{what} saved norms")
    n_st = f64(saved_n)
    y_ref = po.normalize_fwd(x64, n_st)                               # at the stored norms
    check_elementwise(f64(y), y_ref, np.abs(y_ref), dtype, f"{what} y")
    y_st = f64(y)
    dx_ref = po.normalize_bwd(x64, y_st, n_st, g64, p)
    nn = n_st[..., None]
    if p == 1:
        scale = np.abs(g64) / nn + np.abs(x64 * g64).sum(-1, keepdims=True) / (nn * nn)
    elif p == 2:
        scale = (np.abs(g64) + np.abs(y_st) * np.abs(y_st * g64).sum(-1, keepdims=True)) / nn
    else:
        scale = np.abs(g64) / nn + np.abs(x64) ** (p - 1) * np.abs(y_st * g64).sum(-1, keepdims=True) / nn ** p
    check_elementwise(f64(xg.grad), dx_ref, scale, dtype, f"{what} normalize dx")
    return y.detach(), xg.grad


# ---- the reference's unit-test matrix (UnitTests/Ops/norm_unittest.py:78-88, normalize_unittest.py alike) --------
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("dim", [32, 64, 128, 256, 512, 1024])
def test_reference_unit_test_matrix(dim, dtype):
    announce(f"reference matrix norm / normalize D={dim} {dtype}")
    torch.manual_seed(42)
    data = torch.randn(1, 1000, dim, device="cuda", dtype=dtype)
    rtol, atol = (3e-4, 1e-3) if dtype == torch.float32 else (1e-2, 5e-2)       # norm_unittest.py:27
    a = data.clone().requires_grad_(True)
    r = data.clone().requires_grad_(True)
    out = norm(p=2, eps=1e-12)(a)
    ref = torch.norm(r, p=2, dim=-1, keepdim=True)
    assert torch.allclose(out, ref.squeeze(-1), atol=atol, rtol=rtol), "Error in forward pass"
    g = torch.rand_like(ref)
    out.backward(g.squeeze(-1)); ref.backward(g)
    assert torch.allclose(a.grad, r.grad, atol=atol, rtol=rtol), "Error in backward pass"
    a = data.clone().requires_grad_(True)
    r = data.clone().requires_grad_(True)
    out = normalize(p=2, eps=1e-12)(a)
    ref = torch.nn.functional.normalize(r, p=2, dim=-1, eps=1e-12)
    assert torch.allclose(out, ref, atol=atol, rtol=rtol), "Error in forward pass"
    g = torch.rand_like(ref)
    out.backward(g); ref.backward(g)
    assert torch.allclose(a.grad, r.grad, atol=atol, rtol=rtol), "Error in backward pass"
    x = data[:, :64].cpu()
    compare_norm(x, torch.rand(1, 64).to(dtype), 2, 1e-12, f"norm D={dim}")
    compare_normalize(x, torch.randn(1, 64, dim).to(dtype), 2, 1e-12, f"normalize D={dim}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize("p", PS)
def test_every_integer_p(p, dtype):
    announce(f"p={p} {dtype}")
    for shape in ((3, 50, 256), (2, 33, 1000), (1, 9, 4100)):
        x, gn, gy = make(shape, dtype, seed=p + shape[-1])
        compare_norm(x, gn, p, 1e-6, f"norm p={p} {shape}")
        compare_normalize(x, gy, p, 1e-6, f"normalize p={p} {shape}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("p", [1.5, 2.5, 3.7])
def test_real_p(p, dtype):
    announce(f"real p={p} {dtype}")
    x, gn, gy = make((2, 40, 300), dtype, seed=3)
    compare_norm(x, gn, p, 1e-6, f"norm p={p}")
    compare_normalize(x, gy, p, 1e-6, f"normalize p={p}")


@pytest.mark.parametrize("dtype,decades", [(torch.float32, 6.0), (torch.float64, 6.0), (torch.bfloat16, 6.0),
                                           (torch.float16, 1.5)])
@pytest.mark.parametrize("p", [1.5, 2.5, 3.7])
def test_real_p_over_many_magnitudes(p, dtype, decades):
    """|x|^p and |x|^(p-1) with |x| spread over many powers of ten: every binary exponent passes through the
    exponent-splitting power, and the element-wise relative bound on dx checks each of them."""
    announce(f"real p={p} {dtype} magnitudes")
    g = torch.Generator().manual_seed(41)
    shape = (3, 50, 700)
    mag = 10.0 ** ((torch.rand(shape, generator=g) * 2 - 1) * decades)
    x = (torch.randn(shape, generator=g) * mag).to(dtype)
    gn = torch.rand(shape[:-1], generator=g).to(dtype)
    gy = torch.randn(shape, generator=g).to(dtype)
    compare_norm(x, gn, p, 1e-6, f"norm p={p} magnitudes")
    compare_normalize(x, gy, p, 1e-6, f"normalize p={p} magnitudes")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize("k", [1, 2, 7, 33, 100, 257, 1000, 4099, 6001])
def test_ragged_row_widths(k, dtype):
    announce(f"ragged K={k} {dtype}")
    x, gn, gy = make((2, 19, k), dtype, seed=k)
    for p in (1, 2, 3):
        compare_norm(x, gn, p, 1e-6, f"norm K={k} p={p}")
        compare_normalize(x, gy, p, 1e-6, f"normalize K={k} p={p}")


@pytest.mark.parametrize("dtype,k", [(torch.float32, 16384), (torch.bfloat16, 32768), (torch.float32, 16392),
                                     (torch.bfloat16, 70001), (torch.float16, 131072), (torch.float64, 9000)])
def test_rows_at_and_beyond_64_kib(dtype, k):
    """There is no row-width limit (the reference loops over K, norm.py:25): 64 KiB rows still use the row engine,
    wider ones the looping kernels."""
    announce(f"wide rows K={k} {dtype}")
    x, gn, gy = make((2, 5, k), dtype, seed=11, scale=0.05 if dtype == torch.float16 else 1.0)   # float16: sum |x| < 65504
    for p in (1, 2, 4):
        compare_norm(x, gn, p, 1e-6, f"norm K={k} p={p}")
        compare_normalize(x, gy, p, 1e-6, f"normalize K={k} p={p}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_strides_views_and_batch_shapes(dtype):
    announce(f"pnorm strides {dtype}")
    g = torch.Generator().manual_seed(12)
    base = torch.randn(6, 40, 640, generator=g).to(dtype)
    gbase = torch.randn(6, 40, 640, generator=g).to(dtype)
    bg, gg = base.cuda(), gbase.cuda()
    views = (lambda t: t[:, :, :512], lambda t: t[:, :33, :512], lambda t: t[:, ::2, 64:576], lambda t: t[::2, 1:, 3:515],
             lambda t: t.transpose(1, 2)[:, :600, :32], lambda t: t[:, :1, :], lambda t: t[:1, :, 8:], lambda t: t[:, 5:6, :640],
             lambda t: t[2:3, :, :256].expand(4, 40, 256), lambda t: t[:, 7:8, :128].expand(6, 10, 128))
    for i, view in enumerate(views):
        xv, gv = view(base), view(gbase)
        gn = torch.rand(xv.shape[:2], generator=g).to(dtype)
        for p in (2, 3):
            compare_norm(xv.contiguous(), gn, p, 1e-6, f"norm view {i} p={p}", x_gpu=view(bg).detach())
            compare_normalize(xv.contiguous(), gv.contiguous(), p, 1e-6, f"normalize view {i} p={p}",
                              x_gpu=view(bg).detach(), gy_gpu=view(gg))


def test_eps_clamp_zero_rows_and_empty_input():
    announce("pnorm eps / empty")
    x = torch.randn(2, 6, 64)
    x[0, 1] = 0.0
    x[1, 4] = 1e-9
    gn = torch.rand(2, 6); gy = torch.randn(2, 6, 64)
    for p in (1, 2, 3):
        n, _ = compare_norm(x, gn, p, 1e-4, f"clamped norm p={p}")
        assert float(n[0, 1]) == pytest.approx(1e-4, rel=1e-6) and float(n[1, 4]) == pytest.approx(1e-4, rel=1e-6)
        y, dx = compare_normalize(x, gy, p, 1e-4, f"clamped normalize p={p}")
        assert bool((y[0, 1] == 0).all()) and bool(torch.isfinite(dx).all())
    for shape in ((0, 5, 16), (3, 0, 16)):
        e = torch.empty(shape, device="cuda", requires_grad=True)
        n = norm()(e)
        n.sum().backward()
        assert n.shape == shape[:2] and e.grad.shape == shape
        e = torch.empty(shape, device="cuda", requires_grad=True)
        y = normalize()(e)
        y.sum().backward()
        assert y.shape == shape and e.grad.shape == shape


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [64, 1000, 40000])
def test_non_finite_and_overflowing_rows(n, dtype):
    """Rows that hold an infinity, a NaN, only zeros, or entries whose squares overflow float32 (the reference
    computes these types in float32, norm.py:24): the norm is inf / eps / eps / inf -- eps for the NaN row because
    tl.maximum(out, eps) returns eps for a NaN (norm.py:40) -- and x / norm follows from the stored norm
    (normalize.py:30): 0 for a row with an infinite norm (NaN where x itself is infinite), x / eps for the NaN row.
    For p = 2 the gradients of an overflowed row are 0 (a finite numerator over an infinite norm)."""
    announce(f"pnorm non-finite N={n} {dtype}")
    g = torch.Generator().manual_seed(n)
    x = torch.randn(1, 6, n, generator=g).to(dtype)
    spoiled = {1: float("inf"), 2: float("nan"), 3: float("-inf")}
    for r, v in spoiled.items():
        x[0, r, r * 7] = v
    x[0, 4] = 0.0
    x[0, 5] = 1e30
    eps = 1e-6
    eps_st = float(torch.tensor(eps).to(dtype))
    inf = float("inf")
    for p in (1, 2, 3, 2.5):
        xg = x.cuda().requires_grad_(True)
        nrm = norm(p=p, eps=eps)(xg)
        nrm.backward(torch.ones_like(nrm))
        got = nrm.detach().float().cpu()[0]
        assert float(got[1]) == inf and float(got[3]) == inf, f"p={p}: {got}"
        assert float(got[2]) == eps_st and float(got[4]) == eps_st, f"p={p}: {got}"
        if p == 1:
            assert float(got[5]) == pytest.approx(n * 1e30, rel=1e-2)
        else:
            assert float(got[5]) == inf
            if p == 2:                   # p > 2: |x|^(p-1) overflows as well, inf / inf (norm.py:86-90)
                assert bool((xg.grad[0, 5] == 0).all()), f"p={p}: norm dx of the overflowed row"
        assert bool(torch.isfinite(got[0])) and bool(torch.isfinite(xg.grad[0, 0]).all())
        xg = x.cuda().requires_grad_(True)
        y = normalize(p=p, eps=eps)(xg)
        y.backward(torch.ones_like(y))
        yc = y.detach().float().cpu()[0]
        assert bool((yc[4] == 0).all())
        for r in (1, 3):
            hit = torch.zeros(n, dtype=torch.bool); hit[r * 7] = True
            assert bool(torch.isnan(yc[r][hit]).all()) and bool((yc[r][~hit] == 0).all()), f"p={p} row {r}"
        hit = torch.zeros(n, dtype=torch.bool); hit[14] = True
        expect = (x[0, 2].float() / eps_st)[~hit]
        assert bool(torch.isnan(yc[2][hit]).all())
        assert torch.allclose(yc[2][~hit], expect.to(dtype).float(), rtol=2.0 ** -6 if dtype == torch.bfloat16 else 1e-5)
        if p != 1:
            assert bool((yc[5] == 0).all()), f"p={p}: y of the overflowed row"
            if p == 2:                   # p > 2: |x|^(p-1) * (0 / inf) = inf * 0 (normalize.py:113)
                assert bool((xg.grad[0, 5] == 0).all()), f"p={p}: normalize dx of the overflowed row"
        assert bool(torch.isfinite(yc[0]).all()) and bool(torch.isfinite(xg.grad[0, 0]).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_properties_at_large_size(dtype):
    """Size-independent properties on 16 x 4096 x 4096: unit norm of the output, homogeneity (a power-of-two scale
    is exact), gradient orthogonal to x (p = 2), determinism."""
    announce(f"pnorm properties {dtype}")
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(16, 4096, 4096, device="cuda", generator=g).to(dtype)
    gy = torch.randn(16, 4096, 4096, device="cuda", generator=g).to(dtype)
    y, n = ops_launch.normalize_fwd(x, 2, 1e-12)
    y2, n2 = ops_launch.normalize_fwd(x, 2, 1e-12)
    assert torch.equal(y, y2) and torch.equal(n, n2)
    assert torch.equal(ops_launch.norm_fwd(x, 2, 1e-12), n)          # the fused forward stores the same norms
    unit = y.float().pow(2).sum(-1).sqrt()
    assert float((unit - 1).abs().max()) < (1e-6 if dtype == torch.float32 else 6e-3)
    y4, n4 = ops_launch.normalize_fwd(x * 4, 2, 1e-12)
    assert torch.equal(n4, n * 4) and torch.equal(y4, y)
    dx = ops_launch.normalize_bwd(x, y, n, gy, 2)
    dot = (dx.double() * x.double()).sum(-1).abs().max()
    assert float(dot) < (2e-4 if dtype == torch.float32 else 0.5)     # sum of 4096 terms of size ~|g||x|/n rounded to dtype
    idx = torch.tensor([0, 7, 15], device="cuda")
    compare_normalize(x[idx, :3].cpu(), gy[idx, :3].cpu(), 2, 1e-12, "spot rows")


def test_c_abi_direct_calls_and_errors():
    announce("pnorm C ABI direct")
    lib = _native.lib()
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(23)
    B, M, K, pitch = 3, 50, 200, 256
    xb = torch.randn(B, M + 4, pitch, generator=g).cuda()          # batch stride != M * row stride
    gyb = torch.randn(B, M + 4, pitch, generator=g).cuda()
    gn = torch.rand(B, M, generator=g).cuda()
    x, gy = xb[:, :M, :K], gyb[:, :M, :K]
    sb, sm = xb.stride(0), xb.stride(1)
    for p in (1.0, 2.0, 3.0, 2.5):
        norms = torch.empty(B, M, device="cuda"); norms2 = torch.empty(B, M, device="cuda")
        y = torch.full((B, M + 4, pitch), 7.0, device="cuda"); dx = torch.full((B, M + 4, pitch), 7.0, device="cuda")
        dxn = torch.full((B, M + 4, pitch), 7.0, device="cuda")
        assert lib.thn_pnorm_fwd(x.data_ptr(), sb, sm, norms.data_ptr(), B, M, K, p, 1e-6, _native.F32, st) == 0
        assert lib.thn_normalize_fwd(x.data_ptr(), sb, sm, y.data_ptr(), sb, sm, norms2.data_ptr(), B, M, K, p, 1e-6,
                                     _native.F32, st) == 0
        assert lib.thn_pnorm_bwd(x.data_ptr(), sb, sm, norms.data_ptr(), gn.data_ptr(), dxn.data_ptr(), sb, sm, B, M, K,
                                 p, _native.F32, st) == 0
        assert lib.thn_normalize_bwd(x.data_ptr(), sb, sm, y.data_ptr(), sb, sm, norms2.data_ptr(), gy.data_ptr(), sb, sm,
                                     dx.data_ptr(), sb, sm, B, M, K, p, _native.F32, st) == 0
        torch.cuda.synchronize()
        assert torch.equal(norms, norms2)
        for t in (y, dx, dxn):
            assert bool((t[:, M:] == 7.0).all()) and bool((t[:, :, K:] == 7.0).all())      # padding untouched
        pp = int(p) if p == int(p) else p
        x64 = f64(x)
        n_ref = po.norm_fwd(x64, pp, 1e-6)
        check_elementwise(f64(norms), n_ref, n_ref, torch.float32, f"C ABI norms p={p}")
        check_elementwise(f64(y[:, :M, :K]), po.normalize_fwd(x64, f64(norms)), 1.0, torch.float32, f"C ABI y p={p}")
        check_elementwise(f64(dxn[:, :M, :K]), po.norm_bwd(x64, f64(norms), f64(gn), pp), 1.0, torch.float32, f"C ABI norm dx p={p}")
        check_elementwise(f64(dx[:, :M, :K]), po.normalize_bwd(x64, f64(y[:, :M, :K]), f64(norms), f64(gy), pp), 1.0,
                          torch.float32, f"C ABI normalize dx p={p}")
    # operands that a formula does not read may be NULL
    assert lib.thn_pnorm_bwd(x.data_ptr(), sb, sm, 0, gn.data_ptr(), dxn.data_ptr(), sb, sm, B, M, K, 1.0, _native.F32, st) == 0
    assert lib.thn_normalize_bwd(0, 0, 0, y.data_ptr(), sb, sm, norms.data_ptr(), gy.data_ptr(), sb, sm, dx.data_ptr(), sb, sm,
                                 B, M, K, 2.0, _native.F32, st) == 0
    assert lib.thn_normalize_bwd(x.data_ptr(), sb, sm, 0, 0, 0, norms.data_ptr(), gy.data_ptr(), sb, sm, dx.data_ptr(), sb, sm,
                                 B, M, K, 1.0, _native.F32, st) == 0
    torch.cuda.synchronize()
    # errors
    assert lib.thn_pnorm_fwd(x.data_ptr(), sb, K - 1, norms.data_ptr(), B, M, K, 2.0, 1e-6, _native.F32, st) == _native.E_SHAPE
    assert lib.thn_pnorm_bwd(x.data_ptr(), sb, sm, 0, gn.data_ptr(), dxn.data_ptr(), sb, sm, B, M, K, 2.0, _native.F32, st) == _native.E_NULL
    assert lib.thn_normalize_bwd(0, 0, 0, y.data_ptr(), sb, sm, norms.data_ptr(), gy.data_ptr(), sb, sm, dx.data_ptr(), sb, sm,
                                 B, M, K, 3.0, _native.F32, st) == _native.E_NULL


def row_shapes():
    text = open(os.path.join(ROOT, "triton-hub_amd", "csrc", "thn_pnorm_dispatch.h")).read()
    body = re.search(r"#define THN_ROW_SHAPES\(X\)(.*?)\n\n", text, re.S).group(1)
    five = re.search(r"#define THN_PN_SHAPES_FIVE\(X\)(.*?)\n\n", text, re.S).group(1)    # forward, normalize backward
    assert len(re.findall(r"X\(5, ", five)) == 4
    return [(int(k), int(t), int(b)) for k, t, b in re.findall(r"X\((\d+), (\d+), (\d+)\)", body + five)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_every_compiled_launch_shape(dtype):
    """Forces each kernel instance of the three families (4 forward, 5 norm backward, 6 normalize backward) through
    the launch override, for the three p modes: on the 128-bit path, and off it (one column short of a whole number of
    vectors: the unaligned-window instances, the last window overlapping its neighbour)."""
    lib = _native.lib()
    shapes = row_shapes()
    assert len(shapes) >= 20
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    try:
        for k, tpr, block in shapes:
            for n_vecs in sorted({k * tpr, max((k - 1) * tpr + 1, k * tpr - tpr // 2 - 1)}):
                for n in (n_vecs * vec, n_vecs * vec - 1):
                    if n_vecs * 16 > 65536 or n < vec:
                        continue
                    on_path = n % vec == 0
                    rows_per_block = block // tpr
                    m = 2 * rows_per_block + max(1, rows_per_block // 2)
                    announce(f"pnorm shape K={k} TPR={tpr} block={block} cols={n} rows={m} {dtype}")
                    for which in (4, 5, 6):
                        assert lib.thn_norm_set_launch_override(which, k, tpr, block, 0) == 0
                        q = query_launch(which, False, m, n, dtype)
                        if k == 5 and which == 5:       # the norm backward has no 5-vector instances: keeps its own shape
                            assert q[0] != 5
                            continue
                        assert q[:3] == (k, tpr, block) and q[4] == (1 if on_path else 0), q
                    x, gn, gy = make((1, m, n), dtype, seed=k * 1000 + tpr)
                    for p in (1, 2, 3):
                        compare_norm(x, gn, p, 1e-6, f"norm shape {k},{tpr},{block} p={p} cols={n}")
                        compare_normalize(x, gy, p, 1e-6, f"normalize shape {k},{tpr},{block} p={p} cols={n}")
    finally:
        for which in (4, 5, 6):
            lib.thn_norm_set_launch_override(which, 0, 0, 0, 0)


def test_launch_rules_of_16_bit_rows_off_the_128_bit_path():
    """normalize: the forward over 769 to 1024 vectors runs 2 x 512 in 512 threads (the p-norm by itself keeps 4 x 256),
    the backward takes its forward's 3-vector shape for rows of 129 to 191 and 257 to 383 vectors (on the path up to 144
    and 288),
    4 x 128 for 385 to 512 vectors, and one workgroup per compute unit in 512 threads.  Each against the oracle."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    bf16, f16, f32 = torch.bfloat16, torch.float16, torch.float32
    assert query_launch(4, True, 8192, 8191, bf16)[:4] == (2, 512, 512, cus)
    assert query_launch(4, False, 8192, 8191, bf16)[:3] == (4, 256, 256)
    assert query_launch(4, True, 8192, 8192, bf16)[:3] == (4, 256, 256)
    # (rows of 4 t + 1 to 5 t vectors off the path take 5 x t, below)
    for n, want in ((1152, (3, 64, 256)), (1288, (2, 128, 256)), (1500, (3, 64, 256)), (2304, (3, 128, 256)),
                    (2900, (3, 128, 256)), (1280, (2, 128, 256)), (2560, (2, 256, 256)), (3072, (2, 256, 256)),
                    (1536, (2, 128, 256)), (3999, (4, 128, 256))):
        assert query_launch(6, False, 1 << 15, n, bf16)[:3] == want, n
        assert query_launch(6, False, 1 << 15, n, f16)[:3] == want, n
    assert query_launch(6, False, 1 << 15, 516, f32)[:3] == (2, 128, 256)
    for n in (5400, 6001, 8191):
        assert query_launch(6, False, 1 << 15, n, bf16)[2:4] == (512, cus), n
    # rows of 33 to 48 and 65 to 96 vectors: the forward 3 x 16 / 3 x 32 in every storage type, the 16-bit normalize
    # backward up to 40 and 80 vectors
    for which_fwd in (False, True):
        assert query_launch(4, which_fwd, 1 << 15, 264, bf16)[:3] == (3, 16, 256)
        assert query_launch(4, which_fwd, 1 << 15, 576, f16)[:3] == (3, 32, 256)
        assert query_launch(4, which_fwd, 1 << 15, 132, f32)[:3] == (3, 16, 256)
        assert query_launch(4, which_fwd, 1 << 15, 301, f32)[:3] == (3, 32, 256)
    assert query_launch(6, False, 1 << 15, 264, bf16)[:3] == (3, 16, 256) and query_launch(6, False, 1 << 15, 320, f16)[:3] == (3, 16, 256)
    assert query_launch(6, False, 1 << 15, 384, bf16)[:3] == (2, 32, 256) and query_launch(6, False, 1 << 15, 132, f32)[:3] == (2, 32, 256)
    assert query_launch(6, False, 1 << 15, 577, bf16)[:3] == (3, 32, 256) and query_launch(6, False, 1 << 15, 768, bf16)[:3] == (2, 64, 256)
    for n, dt in ((264, bf16), (301, f16), (577, bf16), (640, f16), (132, f32), (301, f32)):
        announce(f"three-vector shapes K={n} {dt}")
        x, gn, gy = make((3, 37, n), dt, seed=n)
        for p in (1, 2, 3):
            compare_norm(x, gn, p, 1e-6, f"norm K={n} p={p}")
            compare_normalize(x, gy, p, 1e-6, f"normalize K={n} p={p}")
    # rows of 4 t + 1 to 5 t vectors: the normalize forward 5 x t with one workgroup per compute unit (t up to 128), the
    # 16-bit backward 5 x t off the path and just above 4 t vectors on it
    for n, dt, f, b in ((1032, bf16, (5, 32, 256), (3, 64, 256)), (2056, bf16, (5, 64, 256), (5, 64, 256)),
                        (4104, f16, (5, 128, 256), (5, 128, 256)), (5120, bf16, (5, 128, 256), (2, 512, 512)),
                        (8200, bf16, (5, 256, 256), (5, 256, 256)), (10240, bf16, (3, 512, 512), (2, 1024, 1024)),
                        (516, f32, (5, 32, 256), (2, 128, 256)), (2052, f32, (5, 128, 256), (2, 512, 512)),
                        (1025, bf16, (5, 32, 256), (5, 32, 256)), (2050, f16, (5, 64, 256), (5, 64, 256)),
                        (5001, bf16, (5, 128, 256), (5, 128, 256))):
        q = query_launch(4, True, 1 << 15, n, dt)
        assert q[:3] == f and (q[3] <= cus or f[0] != 5), (n, dt, q)
        assert query_launch(6, False, 1 << 15, n, dt)[:3] == b, (n, dt)
        assert query_launch(4, False, 1 << 15, n, dt)[0] != 5, (n, dt)         # the p-norm by itself keeps its shapes
    for n, dt in ((8191, bf16), (7001, f16), (1025, bf16), (1152, f16), (2050, bf16), (2304, bf16), (3999, f16),
                  (1032, bf16), (2056, f16), (4104, bf16), (8200, f16), (516, f32), (2052, f32), (5001, bf16)):
        announce(f"launch rules K={n} {dt}")
        x, gn, gy = make((2, 11, n), dt, seed=n)
        for p in (1, 2, 3):
            compare_norm(x, gn, p, 1e-6, f"norm K={n} p={p}")
            compare_normalize(x, gy, p, 1e-6, f"normalize K={n} p={p}")
