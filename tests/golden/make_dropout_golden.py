"""Writes tests/golden/dropout_golden.npz: outputs of Triton's ``tl.randint`` / ``tl.rand`` (the random source of the
reference's dropout kernel, Layers/dropout.py:20) for a few seeds and offset ranges, computed by Triton's CPU
interpreter (TRITON_INTERPRET=1; Triton 3.6.0 of this image).  Nothing of the reference is imported or run: the
kernel below only calls the two library functions.  Run once: ``python tests/golden/make_dropout_golden.py``."""
import os

os.environ["TRITON_INTERPRET"] = "1"

import numpy as np
import torch
import triton
import triton.language as tl


@triton.jit
def sample(OUT_F, OUT_I, seed, first, n, BLOCK: tl.constexpr):
    idx = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    offs = first + idx                                   # int32 offsets, as the reference's `cols`
    tl.store(OUT_F + idx, tl.rand(seed, offs), mask=idx < n)
    tl.store(OUT_I + idx, tl.randint(seed, offs), mask=idx < n)


@triton.jit
def sample64(OUT_F, OUT_I, seed, first, n, BLOCK: tl.constexpr):
    idx = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    offs = first + idx.to(tl.int64)                      # 64-bit offsets: (low, high) words in the counter
    tl.store(OUT_F + idx, tl.rand(seed, offs), mask=idx < n)
    tl.store(OUT_I + idx, tl.randint(seed, offs), mask=idx < n)


def main():
    out = {}
    cases = [(0, 0, 1024), (1, 0, 512), (12345, 0, 4096), (65536, 1 << 20, 512), (40503, (1 << 31) - 300, 300),
             (2 ** 16 - 1, 123456789, 256)]
    for seed, first, n in cases:
        f = torch.empty(n, dtype=torch.float32)
        i = torch.empty(n, dtype=torch.int32)
        sample[(triton.cdiv(n, 256),)](f, i, seed, first, n, BLOCK=256)
        out[f"rand_s{seed}_o{first}"] = f.numpy()
        out[f"randint_s{seed}_o{first}"] = i.numpy()
    for seed, first, n in [(7, (1 << 32) - 100, 256), (2 ** 40 + 3, (1 << 33) + 17, 128)]:
        f = torch.empty(n, dtype=torch.float32)
        i = torch.empty(n, dtype=torch.int32)
        sample64[(triton.cdiv(n, 128),)](f, i, seed, first, n, BLOCK=128)
        out[f"rand64_s{seed}_o{first}"] = f.numpy()
        out[f"randint64_s{seed}_o{first}"] = i.numpy()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "dropout_golden.npz")
    np.savez_compressed(path, triton_version=np.array(triton.__version__), **out)
    print("wrote", path, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
