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
    ("ln", torch.float32, 3100, 8100),     # 1024-thread rows (2025 vectors, pitch 32400 = 16 mod 128) and enough of them for
    ("rms", torch.float32, 3100, 8100),    # the forward to launch more workgroups than are resident (a grid that is not a
                                           # multiple of 8: unshifted); the backward's grid keeps every workgroup on one phase
    ("ln", torch.float16, 8200, 6000),     # 256-thread one-row forward with two workgroups per compute unit
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


def test_two_vector_rows_stay_two_to_a_workgroup():
    """Rows of 2 x 256 vectors at a pitch off 128-byte lines keep the two-row 512-thread workgroup (unshifted): one
    such row per 256-thread workgroup would leave a compute unit four waves with two vectors each.  Only the
    3 x 256-vector shape goes one row at a time to shift.  Also rows of 352-384 vectors and float32 rows of 704-768
    vectors, which run as 2 vectors per thread on twice the threads."""
    from TritonHub.Normalization import _launch
    bf16, f16, f32 = torch.bfloat16, torch.float16, torch.float32
    shape = lambda which, ln, m, n, dt: tuple(_launch.query_launch(which, ln, m, n, dt))[:3]
    for which in (0, 1):
        assert shape(which, False, 16384, 4000, bf16) == (2, 256, 512)       # 500 vectors, pitch 8000
        assert shape(which, True, 16384, 2000, f32) == (2, 256, 512)
        assert shape(which, True, 16384, 6000, f16) == (3, 256, 256)         # 750 vectors: one row, shifted
        assert shape(which, False, 16384, 3072, bf16) == (2, 256, 512)       # 384 vectors
        assert shape(which, False, 16384, 3072, f32) == (2, 512, 512)        # 768 vectors
    # 3 x 256 vectors with a sixth or more of the slots idle: two unshifted rows per workgroup in the forward and in the
    # 16-bit LayerNorm backward, one shifted row at a time in the other backwards
    assert shape(0, False, 16384, 4248, bf16) == (3, 256, 512) and shape(0, True, 16384, 2204, f32) == (3, 256, 512)
    assert shape(1, True, 16384, 4248, bf16) == (3, 256, 512) and shape(1, False, 16384, 4248, bf16) == (3, 256, 256)
    assert shape(1, True, 16384, 2204, f32) == (3, 256, 256)
    assert shape(0, True, 16384, 3072, bf16) == (3, 128, 256)                # the 16-bit LayerNorm forward keeps 3 x 128
    assert shape(1, True, 16384, 3072, bf16) == (2, 256, 512)
    assert shape(0, False, 16384, 2688, bf16) == (3, 128, 512)               # 336 vectors: too empty for 2 x 256;
    assert shape(1, False, 16384, 2688, bf16) == (3, 128, 512)               # four rows per workgroup in both directions
    # 16-bit forward rows of 769-1024 vectors: 2 x 512 in 512 threads up to 896 vectors, and beyond up to 32 rows per
    # compute unit; short kernels (two 256-thread workgroups per compute unit) and float32 rows keep 4 x 256
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    assert shape(0, True, 64 * cus, 6656, bf16) == (2, 512, 512) and shape(0, False, 64 * cus, 7168, f16) == (2, 512, 512)
    assert shape(0, True, 32 * cus, 8192, bf16) == (2, 512, 512) and shape(0, True, 64 * cus, 8192, bf16) == (4, 256, 256)
    assert shape(0, True, 8 * cus, 6656, bf16) == (4, 256, 256) and shape(0, True, 64 * cus, 3328, f32) == (4, 256, 256)
    g = torch.Generator().manual_seed(4000)
    for m, n, dt in ((4200, 4000, bf16), (4200, 2000, f32), (4200, 3000, bf16), (4200, 2816, f16), (4200, 2900, f32),
                     (2100, 6656, bf16), (2100, 7000, f16), (2100, 8192, bf16), (2100, 4248, bf16), (2100, 2204, f32)):
        print(f"\n[case] two-vector rows {dt} M={m} N={n}", flush=True)
        x = (torch.randn(m, n, generator=g) * 2 + 0.5).to(dt)
        dy = torch.randn(m, n, generator=g).to(dt)
        w = (1 + 0.1 * torch.randn(n, generator=g)).to(dt)
        b = (0.1 * torch.randn(n, generator=g)).to(dt)
        parity_util.run_and_compare("ln", x, dy, w, b, 1e-5, f"two-vector rows ln {m}x{n}")
        parity_util.run_and_compare("rms", x, dy, w, None, 1e-5, f"two-vector rows rms {m}x{n}")


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


# The row p-norm / normalize kernels (thn_pnorm.h) take the same shift when the (B, M, K) tensor folds into one batch
# of rows.  Same oracle and tolerances as tests/test_pnorm_parity_gpu.py.
PNORM_CASES = [
    (2.0, torch.float32, (1, 523, 4100)),     # 1025 vectors on 512 threads, pitch 16 mod 128: all eight phases
    (2.0, torch.float32, (3, 100, 6000)),     # batches fold (contiguous): phases 0 / 64
    (1.0, torch.float32, (1, 300, 6000)),
    (3.0, torch.float32, (2, 150, 6000)),
    (2.0, torch.bfloat16, (1, 600, 4104)),    # 513 vectors on 256 threads
    (2.0, torch.float16, (1, 520, 6000)),
    (2.0, torch.float32, (1, 300, 8180)),     # 2045 vectors: no room for the shift
    (2.0, torch.float32, (1, 101, 6000)),     # 101 * pitch is not a multiple of 128: unshifted
]


@pytest.mark.parametrize("p,dtype,shape", PNORM_CASES)
def test_pnorm_rows_off_line_boundaries(p, dtype, shape):
    import test_pnorm_parity_gpu as pnorm_t
    print(f"\n[case] line shift pnorm p={p} {dtype} {shape}", flush=True)
    x, gn, gy = pnorm_t.make(shape, dtype, seed=shape[1] * 31 + shape[2])
    pnorm_t.compare_norm(x, gn, p, 1e-6, f"line shift norm p={p} {shape}")
    pnorm_t.compare_normalize(x, gy, p, 1e-6, f"line shift normalize p={p} {shape}")


def test_pnorm_strided_batches_do_not_shift():
    """Batches that do not fold (a batch stride that is not M row strides) keep the unshifted slots: the result must
    still be right."""
    import test_pnorm_parity_gpu as pnorm_t
    print("\n[case] line shift pnorm, batches that do not fold", flush=True)
    big, _, gbig = pnorm_t.make((3, 140, 6000), torch.float32, seed=77)
    view = lambda t: t[:, :100, :]                   # batch stride 140 rows, 100 rows used
    _, gn, _ = pnorm_t.make((3, 100, 8), torch.float32, seed=79)
    pnorm_t.compare_norm(view(big).contiguous(), gn, 2.0, 1e-6, "non-folding batches norm", x_gpu=view(big.cuda()).detach())
    pnorm_t.compare_normalize(view(big).contiguous(), view(gbig).contiguous(), 2.0, 1e-6, "non-folding batches normalize",
                              x_gpu=view(big.cuda()).detach(), gy_gpu=view(gbig.cuda()))
