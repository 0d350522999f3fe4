"""Writes tests/golden/act_golden.npz: frozen vectors for oracle/act_oracle.py.

Expected values come from PyTorch's float64 CPU functional ops and autograd (the routines the reference's own tests
compare against, e.g. UnitTests/Activations/gelu_unittest.py:17); neither the oracle nor the reference package
produces them.  Run from the repository root:   python tests/golden/make_act_golden.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = {
    "gelu": (lambda x: F.gelu(x), 0.0, 0.0),
    "gelu_tanh": (lambda x: F.gelu(x, approximate="tanh"), 0.0, 0.0),
    "silu": (F.silu, 0.0, 0.0),
    "relu": (F.relu, 0.0, 0.0),
    "leaky_relu": (lambda x: F.leaky_relu(x, 0.07), 0.07, 0.0),
    "relu6": (F.relu6, 0.0, 0.0),
    "sigmoid": (torch.sigmoid, 0.0, 0.0),
    "tanh": (torch.tanh, 0.0, 0.0),
    "mish": (F.mish, 0.0, 0.0),
    "softplus": (lambda x: F.softplus(x, beta=1.5, threshold=6.0), 1.5, 6.0),
    "threshold": (lambda x: F.threshold(x, 0.3, -2.0), 0.3, -2.0),
}


def main():
    out = {}
    for i, (name, (fn, p0, p1)) in enumerate(CASES.items()):
        g = torch.Generator().manual_seed(100 + i)
        x = (torch.randn(6, 257, generator=g, dtype=torch.float64) * 4.0).requires_grad_(True)
        dy = torch.randn(6, 257, generator=g, dtype=torch.float64)
        y = fn(x)
        y.backward(dy)
        out[f"{name}/x"] = x.detach().numpy()
        out[f"{name}/dy"] = dy.numpy()
        out[f"{name}/y"] = y.detach().numpy()
        out[f"{name}/dx"] = x.grad.numpy()
        out[f"{name}/params"] = np.array([p0, p1])
    path = os.path.join(HERE, "act_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
