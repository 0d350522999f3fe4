"""CPU tests that pin oracle/act_oracle.py against independent evidence: torch's float64 CPU functional ops and
autograd (live and frozen), finite differences, closed forms."""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import ROOT
from oracle import act_oracle as ao

TORCH = {
    "gelu": lambda x, p0, p1: F.gelu(x), "gelu_tanh": lambda x, p0, p1: F.gelu(x, approximate="tanh"),
    "silu": lambda x, p0, p1: F.silu(x), "relu": lambda x, p0, p1: F.relu(x),
    "leaky_relu": lambda x, p0, p1: F.leaky_relu(x, p0), "relu6": lambda x, p0, p1: F.relu6(x),
    "sigmoid": lambda x, p0, p1: torch.sigmoid(x), "tanh": lambda x, p0, p1: torch.tanh(x),
    "mish": lambda x, p0, p1: F.mish(x), "softplus": lambda x, p0, p1: F.softplus(x, beta=p0, threshold=p1),
    "threshold": lambda x, p0, p1: F.threshold(x, p0, p1),
}
PARAMS = {"leaky_relu": (0.01, 0.0), "softplus": (1.0, 20.0), "threshold": (0.5, 0.25)}


# mish and softplus follow the reference's log(1 + exp(x)) (mish.py:19, softplus.py:21); torch uses log1p, which keeps
# relative accuracy where exp(x) < 1e-16: an absolute difference of at most |x| * 2e-16 there.
ATOL = {"mish": 1e-13, "softplus": 1e-13}


def saved_for(name, x, y):
    return y if name in ao.SAVES_OUTPUT else x


def test_names_cover_the_reference_modules():
    assert sorted(ao.NAMES) == sorted(TORCH)


def test_golden_vectors():
    data = np.load(os.path.join(ROOT, "tests", "golden", "act_golden.npz"), allow_pickle=False)
    names = sorted({k.split("/")[0] for k in data.files})
    assert names == sorted(ao.NAMES)
    for name in names:
        p0, p1 = data[f"{name}/params"]
        x, dy = data[f"{name}/x"], data[f"{name}/dy"]
        y = ao.fwd(name, x, p0, p1)
        np.testing.assert_allclose(y, data[f"{name}/y"], rtol=1e-12, atol=ATOL.get(name, 1e-15), err_msg=name)
        np.testing.assert_allclose(ao.bwd(name, saved_for(name, x, y), dy, p0, p1), data[f"{name}/dx"], rtol=1e-11,
                                   atol=ATOL.get(name, 1e-14), err_msg=name)


@pytest.mark.parametrize("name", ao.NAMES)
@pytest.mark.parametrize("scale", [1.0, 12.0])
def test_against_torch_float64(name, scale):
    p0, p1 = PARAMS.get(name, (0.0, 0.0))
    g = torch.Generator().manual_seed(7)
    x = (torch.randn(5, 333, generator=g, dtype=torch.float64) * scale).requires_grad_(True)
    dy = torch.randn(5, 333, generator=g, dtype=torch.float64)
    ty = TORCH[name](x, p0, p1)
    ty.backward(dy)
    xn = x.detach().numpy()
    y = ao.fwd(name, xn, p0, p1)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-12, atol=ATOL.get(name, 1e-15))
    np.testing.assert_allclose(ao.bwd(name, saved_for(name, xn, y), dy.numpy(), p0, p1), x.grad.numpy(), rtol=1e-10,
                               atol=ATOL.get(name, 1e-14))


@pytest.mark.parametrize("name", ["gelu", "gelu_tanh", "silu", "sigmoid", "tanh", "mish", "softplus"])
def test_backward_is_derivative_of_forward(name):
    p0, p1 = PARAMS.get(name, (0.0, 0.0))
    x = np.linspace(-6, 6, 97)
    h = 1e-6
    num = (ao.fwd(name, x + h, p0, p1) - ao.fwd(name, x - h, p0, p1)) / (2 * h)
    y = ao.fwd(name, x, p0, p1)
    np.testing.assert_allclose(ao.bwd(name, saved_for(name, x, y), np.ones_like(x), p0, p1), num, rtol=1e-7, atol=1e-9)


def test_closed_forms():
    x = np.array([-3.0, -0.0, 0.0, 2.0, 6.0, 7.5])
    np.testing.assert_array_equal(ao.fwd("relu", x), [0, 0, 0, 2, 6, 7.5])
    np.testing.assert_array_equal(ao.fwd("relu6", x), [0, 0, 0, 2, 6, 6])
    np.testing.assert_array_equal(ao.bwd("relu6", x, np.ones(6)), [0, 0, 0, 1, 0, 0])       # 6 itself is outside (x < 6)
    np.testing.assert_allclose(ao.fwd("leaky_relu", x, 0.1), [-0.3, 0, 0, 2, 6, 7.5])
    np.testing.assert_array_equal(ao.fwd("threshold", x, 2.0, -1.0), [-1, -1, -1, -1, 6, 7.5])   # x > threshold, strictly
    np.testing.assert_array_equal(ao.bwd("threshold", x, np.ones(6), 2.0, -1.0), [0, 0, 0, 0, 1, 1])
    assert ao.fwd("sigmoid", np.array([0.0]))[0] == 0.5 and ao.fwd("gelu", np.array([0.0]))[0] == 0.0
    np.testing.assert_allclose(ao.fwd("softplus", np.array([0.0]), 2.0, 20.0), np.log(2.0) / 2.0, rtol=1e-15)
    np.testing.assert_array_equal(ao.fwd("softplus", np.array([30.0]), 1.0, 20.0), [30.0])       # linear above the threshold
    np.testing.assert_allclose(ao.fwd("silu", np.array([1.0])), 1.0 / (1.0 + np.exp(-1.0)), rtol=1e-15)
    # large arguments stay finite (the overflow-free form of tanh)
    for name in ("tanh", "mish", "gelu_tanh", "silu", "sigmoid", "softplus"):
        big = np.array([-200.0, 200.0])
        y = ao.fwd(name, big, 1.0, 20.0)
        assert np.isfinite(y).all() and np.isfinite(ao.bwd(name, y if name in ao.SAVES_OUTPUT else big, np.ones(2), 1.0, 20.0)).all()
