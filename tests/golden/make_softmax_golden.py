"""Writes tests/golden/softmax_golden.npz: frozen vectors for oracle/softmax_oracle.py.

Expected values come from PyTorch's float64 CPU kernels (torch.softmax / torch.log_softmax and autograd), the
routine the reference's own tests compare against (UnitTests/Activations/softmax_unittest.py:16-47); neither the
oracle nor the reference package produces them.  Run from the repository root:
    python tests/golden/make_softmax_golden.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = [("softmax", (3, 5, 32), 1.0, 1), ("softmax", (4, 257), 8.0, 2), ("softmin", (2, 6, 48), 1.0, 3),
         ("softmin", (5, 100), 5.0, 4), ("logsoftmax", (3, 4, 64), 1.0, 5), ("logsoftmax", (6, 333), 10.0, 6)]


def main():
    out = {}
    for i, (kind, shape, scale, seed) in enumerate(CASES):
        g = torch.Generator().manual_seed(seed)
        x = (torch.randn(shape, generator=g, dtype=torch.float64) * scale).requires_grad_(True)
        dy = torch.randn(shape, generator=g, dtype=torch.float64)
        if kind == "softmax":
            y = torch.softmax(x, dim=-1)
        elif kind == "softmin":
            y = torch.nn.functional.softmin(x, dim=-1)
        else:
            y = torch.log_softmax(x, dim=-1)
        y.backward(dy)
        name = f"{kind}_{i}"
        out[f"{name}/x"] = x.detach().numpy()
        out[f"{name}/dy"] = dy.numpy()
        out[f"{name}/y"] = y.detach().numpy()
        out[f"{name}/dx"] = x.grad.numpy()
    path = os.path.join(HERE, "softmax_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
