"""CPU tests that pin oracle/pnorm_oracle.py against independent evidence: torch's float64 CPU kernels (live
and frozen), finite differences, closed forms, invariants."""
import os

import numpy as np
import pytest
import torch

from conftest import ROOT
from oracle import pnorm_oracle as po

PS = [1, 2, 3, 4, 5, 6, 1.5, 2.5]


def test_golden_vectors():
    data = np.load(os.path.join(ROOT, "tests", "golden", "pnorm_golden.npz"), allow_pickle=False)
    names = sorted({k.split("/")[0] for k in data.files})
    assert len(names) == 8
    for name in names:
        c = {k.split("/")[1]: data[k] for k in data.files if k.startswith(name + "/")}
        p = float(c["p"])
        p = int(p) if p == int(p) else p
        n = po.norm_fwd(c["x"], p, 1e-12)
        np.testing.assert_allclose(n, c["norms"], rtol=1e-13)
        np.testing.assert_allclose(po.norm_bwd(c["x"], n, c["gn"], p), c["dx_norm"], rtol=1e-11, atol=1e-14)
        y = po.normalize_fwd(c["x"], n)
        np.testing.assert_allclose(y, c["y"], rtol=1e-13, atol=1e-16)
        np.testing.assert_allclose(po.normalize_bwd(c["x"], y, n, c["gy"], p), c["dx_normalize"], rtol=1e-10, atol=1e-13)


@pytest.mark.parametrize("p", PS)
@pytest.mark.parametrize("shape", [(2, 3, 16), (1, 5, 333), (3, 1, 1)])
def test_against_torch_float64(p, shape):
    g = torch.Generator().manual_seed(41)
    x = torch.randn(shape, generator=g, dtype=torch.float64).requires_grad_(True)
    gn = torch.rand(shape[:-1], generator=g, dtype=torch.float64)
    gy = torch.randn(shape, generator=g, dtype=torch.float64)
    tn = torch.norm(x, p=p, dim=-1)
    tn.backward(gn)
    n = po.norm_fwd(x.detach().numpy(), p, 1e-12)
    np.testing.assert_allclose(n, tn.detach().numpy(), rtol=1e-13)
    np.testing.assert_allclose(po.norm_bwd(x.detach().numpy(), n, gn.numpy(), p), x.grad.numpy(), rtol=1e-11, atol=1e-14)
    x.grad = None
    ty = torch.nn.functional.normalize(x, p=p, dim=-1, eps=1e-12)
    ty.backward(gy)
    y = po.normalize_fwd(x.detach().numpy(), n)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-13)
    np.testing.assert_allclose(po.normalize_bwd(x.detach().numpy(), y, n, gy.numpy(), p), x.grad.numpy(),
                               rtol=1e-10, atol=1e-13)


@pytest.mark.parametrize("p", [1, 2, 3, 2.5])
def test_backward_is_gradient_of_forward(p):
    rng = np.random.default_rng(6)
    x = rng.normal(size=(2, 7)) + 0.3
    gn = rng.uniform(size=(2,))
    gy = rng.normal(size=(2, 7))
    n = po.norm_fwd(x, p, 0.0)
    y = po.normalize_fwd(x, n)
    h = 1e-6
    num_n = np.zeros_like(x)
    num_y = np.zeros_like(x)
    for i in range(x.shape[0]):
        for j in range(x.shape[1]):
            xp = x.copy(); xp[i, j] += h; xm = x.copy(); xm[i, j] -= h
            num_n[i, j] = ((po.norm_fwd(xp, p, 0.0) - po.norm_fwd(xm, p, 0.0)) * gn).sum() / (2 * h)
            yp = po.normalize_fwd(xp, po.norm_fwd(xp, p, 0.0)); ym = po.normalize_fwd(xm, po.norm_fwd(xm, p, 0.0))
            num_y[i, j] = ((yp - ym) * gy).sum() / (2 * h)
    np.testing.assert_allclose(po.norm_bwd(x, n, gn, p), num_n, rtol=1e-6, atol=1e-9)
    np.testing.assert_allclose(po.normalize_bwd(x, y, n, gy, p), num_y, rtol=1e-6, atol=1e-9)


def test_closed_forms_and_invariants():
    x = np.array([[3.0, -4.0, 0.0]])
    assert po.norm_fwd(x, 1)[0] == 7.0 and po.norm_fwd(x, 2)[0] == 5.0
    np.testing.assert_allclose(po.norm_fwd(x, 3), (27 + 64) ** (1 / 3), rtol=1e-15)
    np.testing.assert_allclose(po.norm_fwd(np.ones((1, 16)), 4), 2.0, rtol=1e-15)           # 16^(1/4)
    assert po.norm_fwd(np.zeros((2, 8)), 2, 1e-6).tolist() == [1e-6, 1e-6]                 # clamped from below by eps
    np.testing.assert_array_equal(po.norm_bwd(x, po.norm_fwd(x, 1), np.array([2.0]), 1), [[2.0, -2.0, 0.0]])
    np.testing.assert_allclose(po.norm_bwd(x, po.norm_fwd(x, 2), np.array([1.0]), 2), [[0.6, -0.8, 0.0]], rtol=1e-15)
    rng = np.random.default_rng(2)
    x = rng.normal(size=(5, 40))
    gy = rng.normal(size=(5, 40))
    for p in (1, 2, 3, 2.5, 6):
        n = po.norm_fwd(x, p, 1e-12)
        y = po.normalize_fwd(x, n)
        np.testing.assert_allclose(po.norm_fwd(y, p, 0.0), 1.0, rtol=1e-13)                 # unit p-norm
        np.testing.assert_allclose(po.norm_fwd(3.5 * x, p, 0.0), 3.5 * n, rtol=1e-13)       # homogeneity
        # normalize is invariant to positive scaling, so its gradient is orthogonal to x (Euler)
        dx = po.normalize_bwd(x, y, n, gy, p)
        np.testing.assert_allclose((dx * x).sum(-1), 0.0, atol=1e-12)
        # the gradient of the norm has unit dual norm pairing: <dnorm/dx, x> = norm (Euler, degree 1)
        np.testing.assert_allclose((po.norm_bwd(x, n, np.ones(5), p) * x).sum(-1), n, rtol=1e-12)
