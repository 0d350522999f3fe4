"""Writes tests/golden/norm_golden.npz: frozen input/expected-output vectors for the oracle.

The expected values do NOT come from the oracle and do NOT come from the reference package (whose kernels
need a GPU and whose tests hold no vectors for this path): they are produced by PyTorch's float64 CPU
kernels -- ``torch.native_layer_norm``, ``aten.native_layer_norm_backward`` and autograd through
``torch.nn.functional.rms_norm`` -- which is the same library routine the reference's own tests compare
against (UnitTests/Normalization/layernorm_unittest.py:16-47).  Freezing them makes the pin independent of the
installed torch version.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = [
    # name, shape, eps, has_weight, has_bias, offset (adds a large mean), seed
    ("ln_quickstart", (2, 5, 128), 1e-6, True, True, 0.0, 1),
    ("ln_ragged", (5, 33), 1e-5, True, True, 0.0, 2),
    ("ln_noaffine", (4, 64), 1e-5, False, False, 0.0, 3),
    ("ln_nobias", (3, 7, 24), 1e-5, True, False, 0.0, 4),
    ("ln_hostile", (4, 300), 1e-6, True, True, 1000.0, 5),
    ("rms_llm", (2, 4, 256), 1e-6, True, False, 0.0, 6),
    ("rms_noaffine", (7, 40), 1e-5, False, False, 0.0, 7),
    ("rms_outliers", (4, 256), 1e-6, True, False, 0.0, 8),
]


def main():
    out = {}
    for name, shape, eps, has_w, has_b, offset, seed in CASES:
        g = torch.Generator().manual_seed(seed)
        n = shape[-1]
        x = torch.randn(shape, generator=g, dtype=torch.float64) + offset
        if name == "rms_outliers":
            mask = torch.rand(shape, generator=g) < 0.02
            x = torch.where(mask, x * 100.0, x)
        dy = torch.randn(shape, generator=g, dtype=torch.float64)
        w = (1.0 + 0.1 * torch.randn(n, generator=g, dtype=torch.float64)) if has_w else None
        b = (0.1 * torch.randn(n, generator=g, dtype=torch.float64)) if has_b else None
        out[f"{name}/x"] = x.numpy()
        out[f"{name}/dy"] = dy.numpy()
        out[f"{name}/eps"] = np.float64(eps)
        if has_w:
            out[f"{name}/w"] = w.numpy()
        if has_b:
            out[f"{name}/b"] = b.numpy()
        if name.startswith("ln"):
            y, mean, rstd = torch.native_layer_norm(x, [n], w, b, eps)
            dx, dw, db = torch.ops.aten.native_layer_norm_backward(dy, x, [n], mean, rstd, w, b, [True, has_w, has_b])
            out[f"{name}/mean"] = mean.reshape(-1).numpy()
            if has_b:
                out[f"{name}/db"] = db.numpy()
        else:
            xr = x.clone().requires_grad_(True)
            wr = w.clone().requires_grad_(True) if has_w else None
            y = torch.nn.functional.rms_norm(xr, [n], wr, eps)
            y.backward(dy)
            dx = xr.grad
            dw = wr.grad if has_w else None
            rstd = torch.rsqrt(x.pow(2).mean(-1) + eps)
            y = y.detach()
        out[f"{name}/y"] = y.numpy()
        out[f"{name}/rstd"] = rstd.reshape(-1).numpy()
        out[f"{name}/dx"] = dx.numpy()
        if has_w:
            out[f"{name}/dw"] = dw.numpy()
    path = os.path.join(HERE, "norm_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
