"""GPU parity on seeded random problems: random family, storage type, row count and row width (log-uniform up to the
widest row each family accepts), sometimes through a column-offset view.  The per-family tests pin chosen widths;
this one walks the launch heuristics (vectors per thread, threads per row, workgroups per compute unit, the forms
for wide, narrow, ragged and misaligned rows) at widths nobody chose.  Same oracles and tolerances as the per-family
tests, whose comparison helpers it reuses."""
import math

import numpy as np
import pytest
import torch

import parity_util
import test_act_parity_gpu as act_t
import test_fused_parity_gpu as fused_t
import test_pnorm_parity_gpu as pnorm_t
import test_softmax_parity_gpu as softmax_t

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16, torch.float64]
FAMILIES = ["ln", "rms", "softmax", "softmin", "logsoftmax", "norm", "normalize", "act", "ln+act", "rms+act"]
MAX_ELEMS = 3_000_000


def log_uniform(rng, lo, hi):
    return int(round(math.exp(rng.uniform(math.log(lo), math.log(hi)))))


def draw(seed):
    rng = np.random.default_rng(1000 + seed)
    family = FAMILIES[seed % len(FAMILIES)]
    dtype = DTYPES[int(rng.integers(len(DTYPES)))]
    size = torch.empty(0, dtype=dtype).element_size()
    row_cap = 65536 // size if family in ("ln", "rms", "ln+act", "rms+act") else 200_000
    n = log_uniform(rng, 1, row_cap)
    m = max(1, min(log_uniform(rng, 1, 5000), MAX_ELEMS // n))
    offset = int(rng.integers(0, 4)) if rng.random() < 0.3 else 0       # a view that starts `offset` columns in
    return family, dtype, m, n, offset, rng


@pytest.mark.parametrize("seed", range(200))
def test_random_problem(seed):
    family, dtype, m, n, offset, rng = draw(seed)
    print(f"\n[case] random seed={seed} {family} {dtype} M={m} N={n} offset={offset}", flush=True)
    g = torch.Generator().manual_seed(seed)
    pad = offset + int(rng.integers(0, 3)) if offset else 0
    xb = (torch.randn(m, n + pad, generator=g) * 2).to(dtype)
    gb = torch.randn(m, n + pad, generator=g).to(dtype)
    x, dy = xb[:, offset:offset + n].contiguous(), gb[:, offset:offset + n].contiguous()
    x_gpu = xb.cuda()[:, offset:offset + n] if pad else None
    dy_gpu = gb.cuda()[:, offset:offset + n] if pad else None
    what = f"random {seed} {family} {m}x{n}"
    # Rows of a few elements are often nearly constant; with a tiny eps rstd then reaches hundreds and multiplies the
    # float32 rounding of (x - mean) beyond any fixed bound, for every implementation that saves a float32 mean.
    eps = 1e-5 if n >= 16 else 1e-2
    if family in ("ln", "rms"):
        w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype)
        b = (0.1 * torch.randn(n, generator=g)).to(dtype) if family == "ln" else None
        parity_util.run_and_compare(family, x, dy, w, b, eps, what)
    elif family in ("softmax", "softmin", "logsoftmax"):
        softmax_t.run_and_compare(family, x, dy, what, x_gpu=None if x_gpu is None else x_gpu.detach(), dy_gpu=dy_gpu)
    elif family == "norm":
        p = [1, 2, 3, 2.5][int(rng.integers(4))]
        gn = torch.rand(1, m, generator=g).to(dtype)
        pnorm_t.compare_norm(x.view(1, m, n), gn, p, 1e-6, f"{what} p={p}")
    elif family == "normalize":
        p = [1, 2, 4, 1.5][int(rng.integers(4))]
        pnorm_t.compare_normalize(x.view(1, m, n), dy.view(1, m, n), p, 1e-6, f"{what} p={p}")
    elif family == "act":
        name = ["gelu", "gelu_tanh", "silu", "relu", "sigmoid", "tanh", "mish", "softplus"][int(rng.integers(8))]
        act_t.run_and_compare(name, x, dy, f"{what} {name}", x_gpu=None if x_gpu is None else x_gpu.detach(), dy_gpu=dy_gpu)
    else:
        kind = family.split("+")[0]
        act = ["gelu", "gelu_tanh", "silu", "relu"][int(rng.integers(4))]
        w = (1 + 0.2 * torch.randn(n, generator=g)).to(dtype)
        b = (0.2 * torch.randn(n, generator=g)).to(dtype) if kind == "ln" else None
        fused_t.run_and_compare(kind, act, x, dy, w, b, eps, f"{what} {act}")


def draw_large(seed):
    """LayerNorm / RMSNorm problems of up to 40 M elements: 200 to 150000 rows, 64 elements to 64 KiB per row; half
    of the widths whole 16-byte vectors, a quarter whole 128-byte lines."""
    rng = np.random.default_rng(7000 + seed)
    dtype = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(3))]
    size = torch.empty(0, dtype=dtype).element_size()
    n = log_uniform(rng, 64, 65536 // size)
    r = rng.random()
    if r < 0.5:
        n = max(8, n // 8 * 8)
    elif r < 0.75:
        n = max(64, n // 64 * 64)
    m = max(1, min(log_uniform(rng, 200, 150000), 40_000_000 // n))
    kind = "ln" if rng.random() < 0.5 else "rms"
    return kind, dtype, m, n


@pytest.mark.parametrize("seed", range(32))
def test_random_large_norm_problem(seed):
    """The launch rules that depend on the row count (workgroups per compute unit, more workgroups than the chip
    holds for the widest rows, half a grid for few rows, rows off 128-byte lines) at sizes nobody chose."""
    from TritonHub.Normalization import _launch
    kind, dtype, m, n = draw_large(seed)
    fwd = tuple(_launch.query_launch(0, kind == "ln", m, n, dtype))[:4]
    bwd = tuple(_launch.query_launch(1, kind == "ln", m, n, dtype))[:4]
    print(f"\n[case] random large seed={seed} {kind} {dtype} M={m} N={n} forward{fwd} backward{bwd}", flush=True)
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(m, n, generator=g) * 2 + 0.5).to(dtype)
    dy = torch.randn(m, n, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype)
    b = (0.1 * torch.randn(n, generator=g)).to(dtype) if kind == "ln" else None
    parity_util.run_and_compare(kind, x, dy, w, b, 1e-5, f"random large {seed}",
                                sample_chunks=8 if m * n > 8_000_000 else None)


def draw_narrow(seed):
    """LayerNorm / RMSNorm over rows of 1 to 100 16-byte vectors (the staged kernels, the flat mapping, the 3-vector
    shapes and the row kernels' narrow-row rules, each by the library's own choice), 1 to 300000 rows, a third of them
    as column blocks of a wider buffer."""
    rng = np.random.default_rng(9000 + seed)
    dtype = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(3))]
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    n_vecs = int(rng.integers(1, 101)) if seed % 4 else int(rng.integers(1, 33))
    n = n_vecs * vec
    m = max(1, min(log_uniform(rng, 1, 300000), 12_000_000 // n))
    kind = "ln" if rng.random() < 0.5 else "rms"
    pad = vec * int(rng.integers(1, 5)) if rng.random() < 0.33 else 0
    return kind, dtype, m, n, pad


@pytest.mark.parametrize("seed", range(80))
def test_random_narrow_norm_problem(seed):
    from TritonHub.Normalization import _launch
    kind, dtype, m, n, pad = draw_narrow(seed)
    fwd = tuple(_launch.query_launch(0, kind == "ln", m, n, dtype))[:4]
    bwd = tuple(_launch.query_launch(1, kind == "ln", m, n, dtype))[:4]
    print(f"\n[case] random narrow seed={seed} {kind} {dtype} M={m} N={n} pad={pad} forward{fwd} backward{bwd}", flush=True)
    g = torch.Generator().manual_seed(seed)
    xb = (torch.randn(m, n + pad, generator=g) * 2 + 0.5).to(dtype)
    gb = torch.randn(m, n + pad, generator=g).to(dtype)
    x, dy = xb[:, :n].contiguous(), gb[:, :n].contiguous()
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype)
    b = (0.1 * torch.randn(n, generator=g)).to(dtype) if kind == "ln" else None
    eps = 1e-5 if n >= 16 else 1e-2
    sample = 8 if m * n > 8_000_000 else None
    if not pad:
        parity_util.run_and_compare(kind, x, dy, w, b, eps, f"random narrow {seed}", sample_chunks=sample)
        return
    # rows that are column blocks of a wider buffer: the same call on strided device views
    from TritonHub.Normalization.layernorm import layernorm
    from TritonHub.Normalization.rmsnorm import rmsnorm
    xg = xb.cuda()[:, :n].detach().requires_grad_(True)
    wg = w.cuda().requires_grad_(True)
    bg = None if b is None else b.cuda().requires_grad_(True)
    assert xg.stride(0) == n + pad
    if kind == "ln":
        y = layernorm.apply(xg, wg, bg, eps)
        mean, rstd = y.grad_fn.saved_tensors[3], y.grad_fn.saved_tensors[4]
    else:
        y = rmsnorm.apply(xg, wg, eps)
        mean, rstd = None, y.grad_fn.saved_tensors[2]
    y.backward(gb.cuda()[:, :n])
    torch.cuda.synchronize()
    out = dict(y=y.detach(), dx=xg.grad, dw=wg.grad, db=None if bg is None else bg.grad, mean=mean, rstd=rstd)
    parity_util.compare_with_oracle(kind, x, dy, w, b, eps, out, f"random narrow {seed} (strided)", sample_chunks=sample)


SHORT_FAMILIES = ["ln", "rms", "softmax", "softmin", "logsoftmax", "norm", "normalize"]


def draw_short(seed):
    """Every row family over rows of 1 to 280 columns, any width -- shorter than a vector (a lane per row), not a whole
    number of vectors (unaligned windows: the flat kernels' other instances, the row kernels' narrow shapes), whole
    vectors (the flat and staged kernels) -- 1 to 200000 rows, a third of them as column blocks of a wider buffer that
    start 0 to 3 columns in (rows behind pointers and pitches off 16 bytes)."""
    rng = np.random.default_rng(31000 + seed)
    family = SHORT_FAMILIES[seed % len(SHORT_FAMILIES)]
    dtype = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(3))]
    n = int(rng.integers(1, 281)) if seed % 3 else int(rng.integers(1, 40))
    m = max(1, min(log_uniform(rng, 1, 200000), 6_000_000 // n))
    if family in ("norm", "normalize") and n < 8:
        m = min(m, 2000)        # nearly one-dimensional rows among many thousand: see test_tiny_rows_gpu.py
    offset = int(rng.integers(0, 4)) if rng.random() < 0.33 else -1
    return family, dtype, m, n, offset, rng


@pytest.mark.parametrize("seed", range(140))
def test_random_short_row_problem(seed):
    family, dtype, m, n, offset, rng = draw_short(seed)
    print(f"\n[case] random short seed={seed} {family} {dtype} M={m} N={n} offset={offset}", flush=True)
    g = torch.Generator().manual_seed(seed)
    pad = 0 if offset < 0 else offset + int(rng.integers(1, 6))
    off = max(offset, 0)
    xb = (torch.randn(m, n + pad, generator=g) * 2 + 0.25).to(dtype)
    gb = torch.randn(m, n + pad, generator=g).to(dtype)
    x, dy = xb[:, off:off + n].contiguous(), gb[:, off:off + n].contiguous()
    what = f"random short {seed} {family} {m}x{n}"
    eps = 1e-5 if n >= 16 else 1e-2
    sample = 8 if m * n > 4_000_000 else None
    if family in ("ln", "rms"):
        w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype)
        b = (0.1 * torch.randn(n, generator=g)).to(dtype) if family == "ln" else None
        if not pad:
            parity_util.run_and_compare(family, x, dy, w, b, eps, what, sample_chunks=sample)
            return
        from TritonHub.Normalization.layernorm import layernorm
        from TritonHub.Normalization.rmsnorm import rmsnorm
        xg = xb.cuda()[:, off:off + n].detach().requires_grad_(True)
        wg = w.cuda().requires_grad_(True)
        bg = None if b is None else b.cuda().requires_grad_(True)
        if family == "ln":
            y = layernorm.apply(xg, wg, bg, eps)
            mean, rstd = y.grad_fn.saved_tensors[3], y.grad_fn.saved_tensors[4]
        else:
            y = rmsnorm.apply(xg, wg, eps)
            mean, rstd = None, y.grad_fn.saved_tensors[2]
        y.backward(gb.cuda()[:, off:off + n])
        torch.cuda.synchronize()
        out = dict(y=y.detach(), dx=xg.grad, dw=wg.grad, db=None if bg is None else bg.grad, mean=mean, rstd=rstd)
        parity_util.compare_with_oracle(family, x, dy, w, b, eps, out, what + " (strided)", sample_chunks=sample)
    elif family in ("softmax", "softmin", "logsoftmax"):
        x_gpu = xb.cuda()[:, off:off + n].detach() if pad else None
        dy_gpu = gb.cuda()[:, off:off + n] if pad else None
        softmax_t.run_and_compare(family, x, dy, what, x_gpu=x_gpu, dy_gpu=dy_gpu)
    else:
        p = [1, 2, 3, 2, 4, 2][int(rng.integers(6))]
        x_gpu = xb.cuda()[:, off:off + n].unsqueeze(0).detach() if pad else None
        if family == "norm":
            gn = torch.rand(1, m, generator=g).to(dtype)
            pnorm_t.compare_norm(x.view(1, m, n), gn, p, 1e-6, f"{what} p={p}", x_gpu=x_gpu)
        else:
            gy_gpu = gb.cuda()[:, off:off + n].unsqueeze(0) if pad else None
            pnorm_t.compare_normalize(x.view(1, m, n), dy.view(1, m, n), p, 1e-6, f"{what} p={p}", x_gpu=x_gpu, gy_gpu=gy_gpu)
