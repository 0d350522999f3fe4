"""GPU parity for rows whose pitch is a multiple of 16 but not of 128 bytes: the norm kernels then move their
vector slots so that every wave request starts on a 128-byte line (up to 7 slots to the left, the phase of the
row's first byte), where one row per workgroup, equal phases of all streams and spare slots allow it.  The cases
walk every phase (pitches of 16 mod 128 bytes), the two-phase pitch of 6000 columns, the last width that still
has the spare slots and the first that has not, and row counts whose grid does or does not keep a workgroup on
one phase.  The softmax family's row kernels do the same.  Same oracles and tolerances as the other parity tests."""
import pytest
import torch

import parity_util
import test_softmax_parity_gpu as softmax_t

pytestmark = pytest.mark.gpu

CASES = [
    ("ln", torch.float32, 700, 6000),      # phases 0 / 64, forward and backward shifted
    ("rms", torch.float32, 700, 6000),
    ("ln", torch.float32, 600, 4100),      # pitch 16400 = 16 mod 128: all eight phases
    ("rms", torch.float32, 523, 4100),
    ("ln", torch.float32, 300, 6116),      # 1529 vectors = 3 * 512 - 7: the widest row with room for the shift
    ("ln", torch.float32, 300, 6124),      # 1531 vectors: no room, unshifted
    ("ln", torch.float16, 520, 6000),      # 256-thread rows: the backward takes one-row workgroups to shift too
    ("rms", torch.bfloat16, 600, 4104),    # pitch 8208 = 16 mod 128, 256-thread rows
    ("ln", torch.bfloat16, 600, 4104),
    ("ln", torch.float32, 100, 6000),      # one workgroup per row, 100 * pitch is a multiple of 128
    ("ln", torch.float32, 101, 6000),      # 101 * pitch is not: unshifted
    ("rms", torch.float64, 300, 3000),     # float64 storage (pitch 24000)
]


@pytest.mark.parametrize("kind,dtype,m,n", CASES)
def test_rows_off_line_boundaries(kind, dtype, m, n):
    print(f"\n[case] line shift {kind} {dtype} M={m} N={n}", flush=True)
    g = torch.Generator().manual_seed(m * 7919 + n)
    x = (torch.randn(m, n, generator=g) * 2 + 0.5).to(dtype)
    dy = torch.randn(m, n, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype)
    b = (0.1 * torch.randn(n, generator=g)).to(dtype) if kind == "ln" else None
    parity_util.run_and_compare(kind, x, dy, w, b, 1e-5, f"line shift {kind} {m}x{n}")


SOFTMAX_CASES = [
    ("softmax", torch.float32, 523, 4100),       # 1025 vectors on 512 threads, all eight phases
    ("logsoftmax", torch.float32, 300, 6000),    # phases 0 / 64
    ("softmin", torch.bfloat16, 600, 4104),      # 513 vectors on 256 threads
    ("softmax", torch.float16, 520, 6000),
    ("logsoftmax", torch.float32, 300, 8180),    # 2045 vectors: 4 x 512 - 7 = 2041 < 2045, unshifted
    ("softmax", torch.float32, 101, 6000),       # 101 * pitch is not a multiple of 128: unshifted
]


@pytest.mark.parametrize("kind,dtype,m,n", SOFTMAX_CASES)
def test_softmax_rows_off_line_boundaries(kind, dtype, m, n):
    print(f"\n[case] line shift {kind} {dtype} M={m} N={n}", flush=True)
    g = torch.Generator().manual_seed(m * 7919 + n)
    x = (torch.randn(m, n, generator=g) * 3).to(dtype)
    dy = torch.randn(m, n, generator=g).to(dtype)
    softmax_t.run_and_compare(kind, x, dy, f"line shift {kind} {m}x{n}")
