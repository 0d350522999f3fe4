"""GPU parity of the flat mapping for narrow Softmax / Softmin / LogSoftmax rows (csrc/thn_softmax_flat.h): rows of 1, 2
and 4 vectors and rows of up to 32 vectors whose vector count is not a power of two, in three storage types, with 2 and
4 rows per lane forced through the launch override (and once by the library's own choice), against the CPU oracle; row
counts that end in the middle of a wave, a workgroup and a grid step; masked (-inf) logits; rows that are column blocks
of a wider buffer; run-to-run identical results."""
import pytest
import torch

import test_softmax_parity_gpu as sm
from TritonHub import _native

pytestmark = pytest.mark.gpu

FLAT_WIDTHS = [n for n in range(1, 33) if n & (n - 1) or n <= 4]


def announce(msg):
    print(f"\n[softmax flat] {msg}", flush=True)


class forced:
    """Launch override for the softmax forward (2) and backward (3): threads_per_row = vectors per row selects the flat
    kernels, vecs_per_thread = rows per lane and step."""

    def __init__(self, n_vecs, rows_each):
        self.args = (rows_each, n_vecs, 0, 0)

    def __enter__(self):
        for which in (2, 3):
            assert _native.lib().thn_norm_set_launch_override(which, *self.args) == 0

    def __exit__(self, *exc):
        for which in (2, 3):
            _native.lib().thn_norm_set_launch_override(which, 0, 0, 0, 0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("kind", ["softmax", "softmin", "logsoftmax"])
def test_every_flat_width_against_the_oracle(kind, dtype):
    from TritonHub.Normalization import _launch
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    for n_vecs in FLAT_WIDTHS:
        n = n_vecs * vec
        for rows_each in (2, 4):
            rows_per_block = 4 * (64 // n_vecs) * rows_each
            for m in sorted({1, rows_per_block - 1, 3 * rows_per_block + 5, 1000 + n_vecs}):
                announce(f"{kind} {dtype} L={n_vecs} N={n} J={rows_each} M={m}")
                with forced(n_vecs, rows_each):
                    for which in (2, 3):
                        q = _launch.query_launch(which, False, m, n, dtype)
                        assert q[:3] == (rows_each, n_vecs, 256), q
                    x, dy = sm.make((m, n), dtype, 100 * n_vecs + rows_each, scale=3.0)
                    sm.run_and_compare(kind, x, dy, f"flat L={n_vecs} J={rows_each} M={m}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("kind", ["softmax", "softmin", "logsoftmax"])
def test_flat_widths_off_the_128_bit_path(kind, dtype):
    """Rows that are not a whole number of vectors (one column more than n_vecs - 1 vectors, one less than n_vecs): the
    flat kernels' unaligned-window instances, the last window overlapping its neighbour; and whole vectors behind a
    base pointer that is one element off 16 bytes."""
    from TritonHub.Normalization import _launch
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    for n_vecs in range(1, 33):           # powers of two included: off the path the flat kernels take those too
        rows_per_block = 4 * (64 // n_vecs) * 2
        for n in sorted({(n_vecs - 1) * vec + 1, n_vecs * vec - 1}):
            if n < vec:
                continue
            for m in sorted({1, rows_per_block - 1, 3 * rows_per_block + 5, 1000 + n_vecs}):
                announce(f"{kind} {dtype} L={n_vecs} ragged N={n} M={m}")
                for which in (2, 3):
                    q = _launch.query_launch(which, False, m, n, dtype)
                    assert q[:3] == (2, n_vecs, 256) and q[4] == 0, q
                x, dy = sm.make((m, n), dtype, 100 * n_vecs + n, scale=3.0)
                sm.run_and_compare(kind, x, dy, f"flat ragged L={n_vecs} N={n} M={m}")
        n, m = n_vecs * vec, 3 * rows_per_block + 5
        announce(f"{kind} {dtype} L={n_vecs} N={n} M={m} behind a misaligned pointer")
        x, dy = sm.make((m, n), dtype, 7 * n_vecs, scale=3.0)
        buf = torch.empty(m * n + 1, dtype=dtype, device="cuda")
        xg = buf[1:].view(m, n)
        xg.copy_(x)
        assert xg.data_ptr() % 16 != 0
        sm.run_and_compare(kind, x, dy, f"flat misaligned L={n_vecs} M={m}", x_gpu=xg)


def test_default_choice_masked_logits_strided_rows_and_determinism():
    from TritonHub.Normalization import _launch
    g = torch.Generator().manual_seed(11)
    # by the library's own choice: 72 bf16 columns (9 vectors), 2^18 rows
    m, n = 1 << 18, 72
    q = _launch.query_launch(2, False, m, n, torch.bfloat16)
    assert q[1] == 9 and q[2] == 256, q
    announce("bf16 262144 x 72 by default")
    x, dy = sm.make((m, n), torch.bfloat16, 3, scale=2.0)
    y1, dx1 = sm.run_and_compare("softmax", x, dy, "flat default bf16 2^18 x 72")
    y2, dx2 = sm.run_and_compare("softmax", x, dy, "flat default bf16 2^18 x 72 again")
    assert torch.equal(y1, y2) and torch.equal(dx1, dx2)
    # masked logits: -inf entries come out as exact 0 (softmax) / -inf (log-softmax), a fully masked row as NaN
    announce("masked logits f32 500 x 20")
    x = torch.randn(500, 20, generator=g)
    x[torch.rand(500, 20, generator=g) < 0.3] = float("-inf")
    x[7] = float("-inf")
    xg = x.cuda()
    from TritonHub.Activations import LogSoftmax, Softmax
    y = Softmax()(xg).cpu()
    ref = torch.softmax(x.double(), -1)
    keep = ~torch.isnan(ref).any(-1)
    assert bool(torch.isnan(y[7]).all()) and bool((y[keep][x[keep] == float("-inf")] == 0).all())
    assert torch.allclose(y[keep].double(), ref[keep], atol=1e-6)
    ly = LogSoftmax()(xg).cpu()
    assert bool((ly[keep][x[keep] == float("-inf")] == float("-inf")).all())
    # rows that are column blocks of a wider buffer
    announce("strided f16 777 x 88 inside rows of 128")
    xb = (torch.randn(777, 128, generator=g) * 2).half()
    gb = torch.randn(777, 128, generator=g).half()
    sm.run_and_compare("softmin", xb[:, :88].contiguous(), gb[:, :88].contiguous(), "flat strided f16 777 x 88",
                       x_gpu=xb.cuda()[:, :88].detach(), dy_gpu=gb.cuda()[:, :88])
