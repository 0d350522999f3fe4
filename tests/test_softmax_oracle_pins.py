"""CPU tests that pin oracle/softmax_oracle.py against independent evidence: torch's float64 CPU kernels
(live and frozen), finite differences, closed forms, invariants."""
import os

import numpy as np
import pytest
import torch

from conftest import ROOT
from oracle import softmax_oracle as so

RT = dict(rtol=1e-12, atol=1e-14)
KINDS = ["softmax", "softmin", "logsoftmax"]
TORCH = {"softmax": lambda x: torch.softmax(x, -1), "softmin": lambda x: torch.nn.functional.softmin(x, -1),
         "logsoftmax": lambda x: torch.log_softmax(x, -1)}


def test_golden_vectors():
    data = np.load(os.path.join(ROOT, "tests", "golden", "softmax_golden.npz"), allow_pickle=False)
    names = sorted({k.split("/")[0] for k in data.files})
    assert len(names) == 6
    for name in names:
        kind = name.split("_")[0]
        y = so.FWD[kind](data[f"{name}/x"])
        np.testing.assert_allclose(y, data[f"{name}/y"], **RT)
        np.testing.assert_allclose(so.BWD[kind](y, data[f"{name}/dy"]), data[f"{name}/dx"], rtol=1e-11, atol=1e-13)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("shape,scale", [((7, 33), 1.0), ((2, 3, 1000), 20.0), ((5, 1), 1.0), ((4, 4096), 3.0)])
def test_against_torch_float64(kind, shape, scale):
    g = torch.Generator().manual_seed(31)
    x = (torch.randn(shape, generator=g, dtype=torch.float64) * scale).requires_grad_(True)
    dy = torch.randn(shape, generator=g, dtype=torch.float64)
    ty = TORCH[kind](x)
    ty.backward(dy)
    y = so.FWD[kind](x.detach().numpy())
    np.testing.assert_allclose(y, ty.detach().numpy(), **RT)
    np.testing.assert_allclose(so.BWD[kind](y, dy.numpy()), x.grad.numpy(), rtol=1e-11, atol=1e-13)


@pytest.mark.parametrize("kind", KINDS)
def test_backward_is_gradient_of_forward(kind):
    rng = np.random.default_rng(4)
    x = rng.normal(size=(3, 6)) * 2
    dy = rng.normal(size=(3, 6))
    dx = so.BWD[kind](so.FWD[kind](x), dy)
    h = 1e-6
    num = np.zeros_like(x)
    for i in range(x.shape[0]):
        for j in range(x.shape[1]):
            xp = x.copy(); xp[i, j] += h; xm = x.copy(); xm[i, j] -= h
            num[i, j] = ((so.FWD[kind](xp) - so.FWD[kind](xm)) * dy).sum() / (2 * h)
    np.testing.assert_allclose(dx, num, rtol=1e-6, atol=1e-9)


def test_closed_forms_and_invariants():
    # a constant row is uniform; log-softmax of it is -log N
    np.testing.assert_allclose(so.softmax_fwd(np.full((2, 8), 3.5)), 0.125, rtol=1e-15)
    np.testing.assert_allclose(so.logsoftmax_fwd(np.zeros((1, 10))), -np.log(10.0), rtol=1e-15)
    # two elements: a logistic function of the difference
    y = so.softmax_fwd(np.array([[0.0, np.log(3.0)]]))
    np.testing.assert_allclose(y, [[0.25, 0.75]], rtol=1e-15)
    np.testing.assert_allclose(so.softmin_fwd(np.array([[0.0, np.log(3.0)]])), [[0.75, 0.25]], rtol=1e-15)
    rng = np.random.default_rng(9)
    x = rng.normal(size=(6, 50)) * 30
    dy = rng.normal(size=(6, 50))
    p = so.softmax_fwd(x)
    np.testing.assert_allclose(p.sum(1), 1.0, rtol=1e-14)
    np.testing.assert_allclose(so.softmax_fwd(x + 123.0), p, rtol=1e-12)            # shift invariance
    np.testing.assert_allclose(np.exp(so.logsoftmax_fwd(x)), p, rtol=1e-12)          # log-softmax = log(softmax)
    np.testing.assert_allclose(so.softmin_fwd(x), so.softmax_fwd(-x), rtol=0)
    np.testing.assert_allclose(so.softmax_bwd(p, dy).sum(1), 0, atol=1e-14)          # gradients sum to zero per row
    np.testing.assert_allclose(so.logsoftmax_bwd(np.log(p), dy).sum(1), 0, atol=1e-12)
    np.testing.assert_allclose(so.softmax_bwd(p, np.ones_like(dy)), 0, atol=1e-15)   # constant upstream gradient
    # no overflow for large inputs (the max is subtracted first)
    assert np.isfinite(so.softmax_fwd(np.array([[1e4, 1e4 - 1.0]]))).all()
