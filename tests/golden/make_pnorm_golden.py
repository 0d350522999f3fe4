"""Writes tests/golden/pnorm_golden.npz: frozen vectors for oracle/pnorm_oracle.py.

Expected values come from PyTorch's float64 CPU kernels (torch.norm, torch.nn.functional.normalize and
autograd), the routines the reference's own tests compare against (UnitTests/Ops/norm_unittest.py:38,
normalize_unittest.py:38); neither the oracle nor the reference package produces them.
Run from the repository root:   python tests/golden/make_pnorm_golden.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = [(1, (2, 5, 32), 1), (2, (3, 4, 64), 2), (2, (1, 7, 257), 3), (3, (2, 3, 48), 4), (4, (1, 6, 100), 5),
         (2.5, (2, 4, 33), 6), (6, (2, 2, 40), 7), (1.5, (1, 5, 20), 8)]


def main():
    out = {}
    for i, (p, shape, seed) in enumerate(CASES):
        g = torch.Generator().manual_seed(seed)
        x = torch.randn(shape, generator=g, dtype=torch.float64).requires_grad_(True)
        gn = torch.rand(shape[:-1], generator=g, dtype=torch.float64)
        gy = torch.randn(shape, generator=g, dtype=torch.float64)
        n = torch.norm(x, p=p, dim=-1)
        n.backward(gn)
        dx_norm = x.grad.clone()
        x.grad = None
        y = torch.nn.functional.normalize(x, p=p, dim=-1, eps=1e-12)
        y.backward(gy)
        name = f"case{i}"
        out[f"{name}/p"] = np.float64(p)
        out[f"{name}/x"] = x.detach().numpy()
        out[f"{name}/gn"] = gn.numpy()
        out[f"{name}/gy"] = gy.numpy()
        out[f"{name}/norms"] = n.detach().numpy()
        out[f"{name}/dx_norm"] = dx_norm.numpy()
        out[f"{name}/y"] = y.detach().numpy()
        out[f"{name}/dx_normalize"] = x.grad.numpy()
    path = os.path.join(HERE, "pnorm_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
