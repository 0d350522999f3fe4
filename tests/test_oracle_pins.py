"""CPU tests that pin the oracle (oracle/norm_oracle.py and the C restatement oracle/norm_oracle.c).

A test here never re-types the oracle's formula.  Each one compares against something independent:
PyTorch's float64 CPU kernels, the frozen vectors under tests/golden/, central finite differences of the
oracle's own forward, closed forms, or invariants that a dropped term / wrong sign / transposed operand breaks.
"""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import norm_oracle as no

RT = dict(rtol=1e-11, atol=1e-12)


# ---- golden vectors (written by tests/golden/make_golden.py from torch's float64 CPU kernels) -----------
def test_golden_vectors_numpy_oracle(golden):
    assert len(golden) == 8
    for name, c in golden.items():
        w, b, eps = c.get("w"), c.get("b"), float(c["eps"])
        if name.startswith("ln"):
            y, mean, rstd = no.layernorm_fwd(c["x"], w, b, eps)
            dx, dw, db = no.layernorm_bwd(c["x"], c["dy"], w, mean, rstd, has_bias=b is not None)
            np.testing.assert_allclose(mean, c["mean"], **RT)
            if b is not None:
                np.testing.assert_allclose(db, c["db"], **RT)
            else:
                assert db is None
        else:
            y, rstd = no.rmsnorm_fwd(c["x"], w, eps)
            dx, dw = no.rmsnorm_bwd(c["x"], c["dy"], w, rstd)
        # the hostile case (mean 1000, std 1) loses ~3 digits to cancellation in any float64 evaluation
        tol = dict(rtol=1e-8, atol=1e-9) if name == "ln_hostile" else RT
        np.testing.assert_allclose(y, c["y"], **tol)
        np.testing.assert_allclose(rstd, c["rstd"], **tol)
        np.testing.assert_allclose(dx, c["dx"], **tol)
        if w is not None:
            np.testing.assert_allclose(dw, c["dw"], **tol)
        else:
            assert dw is None


def test_golden_vectors_c_oracle(golden):
    for name, c in golden.items():
        t = lambda a: None if a is None else torch.from_numpy(np.ascontiguousarray(a))
        x, dy, w, b, eps = t(c["x"]), t(c["dy"]), t(c.get("w")), t(c.get("b")), float(c["eps"])
        tol = dict(rtol=1e-8, atol=1e-9) if name == "ln_hostile" else RT
        if name.startswith("ln"):
            y, mean, rstd = co.layernorm_fwd(x, w, b, eps)
            dx, dw, db = co.layernorm_bwd(x, dy, w, mean, rstd, has_bias=b is not None)
            np.testing.assert_allclose(mean, c["mean"], **RT)
            if b is not None:
                np.testing.assert_allclose(db, c["db"], **RT)
        else:
            y, rstd = co.rmsnorm_fwd(x, w, eps)
            dx, dw = co.rmsnorm_bwd(x, dy, w, rstd)
        np.testing.assert_allclose(y, c["y"], **tol)
        np.testing.assert_allclose(dx, c["dx"], **tol)
        if w is not None:
            np.testing.assert_allclose(dw, c["dw"], **tol)


# ---- live library pins (float64 CPU kernels of the installed torch) ---------------------------------------
@pytest.mark.parametrize("shape,has_w,has_b", [((2, 100, 128), True, True), ((37, 6000), True, True),
                                               ((9, 32), False, False), ((5, 3, 48), True, False)])
def test_layernorm_against_torch_float64(shape, has_w, has_b):
    g = torch.Generator().manual_seed(11)
    n = shape[-1]
    x = torch.randn(shape, generator=g, dtype=torch.float64)
    dy = torch.randn(shape, generator=g, dtype=torch.float64)
    w = 1 + 0.1 * torch.randn(n, generator=g, dtype=torch.float64) if has_w else None
    b = 0.1 * torch.randn(n, generator=g, dtype=torch.float64) if has_b else None
    ty, tmean, trstd = torch.native_layer_norm(x, [n], w, b, 1e-6)
    tdx, tdw, tdb = torch.ops.aten.native_layer_norm_backward(dy, x, [n], tmean, trstd, w, b, [True, has_w, has_b])
    for impl, conv in ((no, lambda t: None if t is None else t.numpy()), (co, lambda t: t)):
        y, mean, rstd = impl.layernorm_fwd(conv(x), conv(w), conv(b), 1e-6)
        dx, dw, db = impl.layernorm_bwd(conv(x), conv(dy), conv(w), mean, rstd, has_bias=has_b)
        np.testing.assert_allclose(y, ty.numpy(), **RT)
        np.testing.assert_allclose(mean, tmean.reshape(-1).numpy(), **RT)
        np.testing.assert_allclose(rstd, trstd.reshape(-1).numpy(), **RT)
        np.testing.assert_allclose(dx, tdx.numpy(), **RT)
        if has_w:
            np.testing.assert_allclose(dw, tdw.numpy(), **RT)
        if has_b:
            np.testing.assert_allclose(db, tdb.numpy(), **RT)


@pytest.mark.parametrize("shape,has_w", [((8, 64, 256), True), ((13, 1000), True), ((4, 40), False)])
def test_rmsnorm_against_torch_float64_autograd(shape, has_w):
    g = torch.Generator().manual_seed(12)
    n = shape[-1]
    x = torch.randn(shape, generator=g, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(shape, generator=g, dtype=torch.float64)
    w = (1 + 0.1 * torch.randn(n, generator=g, dtype=torch.float64)).requires_grad_() if has_w else None
    ty = torch.nn.functional.rms_norm(x, [n], w, 1e-6)
    ty.backward(dy)
    for impl, conv in ((no, lambda t: None if t is None else t.detach().numpy()), (co, lambda t: None if t is None else t.detach())):
        y, rstd = impl.rmsnorm_fwd(conv(x), conv(w), 1e-6)
        dx, dw = impl.rmsnorm_bwd(conv(x), conv(dy), conv(w), rstd)
        np.testing.assert_allclose(y, ty.detach().numpy(), **RT)
        np.testing.assert_allclose(dx, x.grad.numpy(), **RT)
        if has_w:
            np.testing.assert_allclose(dw, w.grad.numpy(), **RT)


# ---- finite differences: backward must be the gradient of forward ---------------------------------------
@pytest.mark.parametrize("kind", ["ln", "rms"])
def test_backward_is_gradient_of_forward(kind):
    rng = np.random.default_rng(3)
    m, n = 3, 7
    x = rng.normal(size=(m, n)); w = 1 + 0.3 * rng.normal(size=n); b = rng.normal(size=n); dy = rng.normal(size=(m, n))
    eps = 1e-3

    def loss(xv, wv, bv):
        y = no.layernorm_fwd(xv, wv, bv, eps)[0] if kind == "ln" else no.rmsnorm_fwd(xv, wv, eps)[0]
        return float((y * dy).sum())

    if kind == "ln":
        _, mean, rstd = no.layernorm_fwd(x, w, b, eps)
        dx, dw, db = no.layernorm_bwd(x, dy, w, mean, rstd)
    else:
        _, rstd = no.rmsnorm_fwd(x, w, eps)
        dx, dw = no.rmsnorm_bwd(x, dy, w, rstd)
        db = None
    h = 1e-6
    num_dx = np.zeros_like(x)
    for i in range(m):
        for j in range(n):
            xp = x.copy(); xp[i, j] += h; xm = x.copy(); xm[i, j] -= h
            num_dx[i, j] = (loss(xp, w, b) - loss(xm, w, b)) / (2 * h)
    np.testing.assert_allclose(dx, num_dx, rtol=1e-6, atol=1e-8)
    num_dw = np.zeros(n); num_db = np.zeros(n)
    for j in range(n):
        wp = w.copy(); wp[j] += h; wm = w.copy(); wm[j] -= h
        num_dw[j] = (loss(x, wp, b) - loss(x, wm, b)) / (2 * h)
        bp = b.copy(); bp[j] += h; bm = b.copy(); bm[j] -= h
        num_db[j] = (loss(x, w, bp) - loss(x, w, bm)) / (2 * h)
    np.testing.assert_allclose(dw, num_dw, rtol=1e-6, atol=1e-8)
    if db is not None:
        np.testing.assert_allclose(db, num_db, rtol=1e-6, atol=1e-8)


# ---- closed forms and invariants -------------------------------------------------------------------------
def test_closed_forms():
    # LayerNorm of (-1, +1) with eps = 0: mean 0, var 1, y = x.  With eps = 3: rstd = 1/2.
    x = np.array([[-1.0, 1.0]])
    y, mean, rstd = no.layernorm_fwd(x, None, None, 0.0)
    assert mean[0] == 0.0 and rstd[0] == 1.0 and (y == x).all()
    assert no.layernorm_fwd(x, None, None, 3.0)[2][0] == 0.5
    # biased (1/N) variance: rows (0, 2): var = 1, not 2
    assert no.layernorm_fwd(np.array([[0.0, 2.0]]), None, None, 0.0)[2][0] == 1.0
    # RMSNorm of (3, 4): mean square 12.5
    y, rstd = no.rmsnorm_fwd(np.array([[3.0, 4.0]]), None, 0.0)
    np.testing.assert_allclose(rstd[0], 1 / np.sqrt(12.5), rtol=1e-15)
    # constant row: LayerNorm output is the bias exactly, rstd = 1/sqrt(eps)
    y, mean, rstd = no.layernorm_fwd(np.full((1, 9), 5.0), np.arange(9.0), np.arange(9.0) * 2, 0.25)
    assert mean[0] == 5.0 and rstd[0] == 2.0 and (y == np.arange(9.0) * 2).all()
    # weight is applied per column, bias added after: y[:, j] = xhat*w[j] + b[j]
    x = np.array([[1.0, 2.0, 3.0, 6.0]])
    y0 = no.layernorm_fwd(x, None, None, 1e-5)[0]
    w = np.array([2.0, -1.0, 0.5, 3.0]); b = np.array([0.1, 0.2, 0.3, 0.4])
    np.testing.assert_allclose(no.layernorm_fwd(x, w, b, 1e-5)[0], y0 * w + b, rtol=1e-15)


def test_invariants():
    rng = np.random.default_rng(5)
    m, n = 11, 96
    x = rng.normal(size=(m, n)) * 3 + 2; dy = rng.normal(size=(m, n)); w = 1 + 0.2 * rng.normal(size=n)
    eps = 1e-6
    y, mean, rstd = no.layernorm_fwd(x, None, None, eps)
    np.testing.assert_allclose(y.sum(1), 0, atol=1e-12)                       # sum xhat = 0
    var = x.var(axis=1)
    np.testing.assert_allclose((y * y).mean(1), var / (var + eps), rtol=1e-12)  # mean xhat^2 = var/(var+eps)
    dx, dw, db = no.layernorm_bwd(x, dy, w, mean, rstd)
    np.testing.assert_allclose(dx.sum(1), 0, atol=1e-12)                      # dx is orthogonal to 1 ...
    y0, mean0, rstd0 = no.layernorm_fwd(x, None, None, 0.0)
    dx0 = no.layernorm_bwd(x, dy, w, mean0, rstd0)[0]
    np.testing.assert_allclose((dx0 * y0).sum(1), 0, atol=1e-11)              # ... and, at eps = 0, to xhat
    np.testing.assert_allclose(db, dy.sum(0), rtol=1e-13)
    yr, rr = no.rmsnorm_fwd(x, None, eps)
    ms = (x * x).mean(1)
    np.testing.assert_allclose((yr * yr).mean(1), ms / (ms + eps), rtol=1e-12)
    yr0, rr0 = no.rmsnorm_fwd(x, None, 0.0)
    dxr0, _ = no.rmsnorm_bwd(x, dy, w, rr0)
    np.testing.assert_allclose((dxr0 * yr0).sum(1), 0, atol=1e-11)            # at eps = 0, dx is orthogonal to xhat
    # shifting a row by a constant does not change LayerNorm; scaling it does not change RMSNorm (eps = 0)
    np.testing.assert_allclose(no.layernorm_fwd(x + 7.5, None, None, eps)[0], y, atol=1e-11)
    np.testing.assert_allclose(no.rmsnorm_fwd(x * 3.0, None, 0.0)[0], no.rmsnorm_fwd(x, None, 0.0)[0], rtol=1e-13)
    # dW / dB are linear in the rows: the sum over two halves equals the whole
    h = m // 2
    _, dwa, dba = no.layernorm_bwd(x[:h], dy[:h], w, mean[:h], rstd[:h])
    _, dwb, dbb = no.layernorm_bwd(x[h:], dy[h:], w, mean[h:], rstd[h:])
    np.testing.assert_allclose(dwa + dwb, dw, rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(dba + dbb, db, rtol=1e-12, atol=1e-13)


# ---- the two oracles agree; storage decoding in the C oracle is exact -----------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64])
def test_c_oracle_matches_numpy_oracle(dtype):
    g = torch.Generator().manual_seed(21)
    m, n = 33, 200
    x = (torch.randn(m, n, generator=g) * 2 + 1).to(dtype); dy = torch.randn(m, n, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype); b = (0.1 * torch.randn(n, generator=g)).to(dtype)
    d = lambda t: t.double().numpy()
    y, mean, rstd = no.layernorm_fwd(d(x), d(w), d(b), 1e-6)
    cy, cmean, crstd = co.layernorm_fwd(x, w, b, 1e-6)
    np.testing.assert_allclose(cy, y, **RT); np.testing.assert_allclose(cmean, mean, **RT); np.testing.assert_allclose(crstd, rstd, **RT)
    dx, dw, db = no.layernorm_bwd(d(x), d(dy), d(w), mean, rstd)
    cdx, cdw, cdb = co.layernorm_bwd(x, dy, w, mean, rstd)
    np.testing.assert_allclose(cdx, dx, **RT); np.testing.assert_allclose(cdw, dw, **RT); np.testing.assert_allclose(cdb, db, **RT)
    y, rstd = no.rmsnorm_fwd(d(x), d(w), 1e-6)
    cy, crstd = co.rmsnorm_fwd(x, w, 1e-6)
    np.testing.assert_allclose(cy, y, **RT); np.testing.assert_allclose(crstd, rstd, **RT)
    dx, dw = no.rmsnorm_bwd(d(x), d(dy), d(w), rstd)
    cdx, cdw = co.rmsnorm_bwd(x, dy, w, rstd)
    np.testing.assert_allclose(cdx, dx, **RT); np.testing.assert_allclose(cdw, dw, **RT)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_c_oracle_narrowing_is_round_to_nearest_even(dtype):
    g = torch.Generator().manual_seed(22)
    x = torch.cat([torch.randn(4, 512, generator=g) * s for s in (1e-6, 1e-3, 1.0, 300.0)]).to(dtype)
    y = co.rmsnorm_fwd(x, None, 1e-6, out_dtype=dtype)[0]
    y64, _ = co.rmsnorm_fwd(x, None, 1e-6)
    want = torch.from_numpy(y64).to(torch.float32).to(dtype)       # torch's own RTNE narrowing
    assert torch.equal(y, want)


def test_ulp_helper():
    assert no.ulp(1.0, "fp32") == 2.0 ** -23 and no.ulp(1.5, "bf16") == 2.0 ** -7 and no.ulp(1000.0, "fp16") == 0.5
    assert no.ulp(0.0, "fp16") == 2.0 ** -24 and no.ulp(1e-9, "fp16") == 2.0 ** -24      # subnormal spacing
    got = torch.tensor([1.0 + 2.0 ** -7], dtype=torch.bfloat16).double().numpy()
    assert no.ulp_error(got, np.array([1.0]), "bf16")[0] == 1.0


def test_host_wrapper_rules():
    # rows wider than 64 KiB are refused with the reference's message (layernorm.py:69-72)
    no.check_feature_dim(16384, 4); no.check_feature_dim(32768, 2); no.check_feature_dim(8192, 8)
    for n, es in ((16385, 4), (32769, 2), (8193, 8), (70000, 2)):
        with pytest.raises(RuntimeError, match="doesn't support feature dim >= 64KB"):
            no.check_feature_dim(n, es)
    assert no.flatten_rows(np.zeros((2, 3, 4))).shape == (6, 4)
