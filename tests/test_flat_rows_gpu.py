"""GPU parity of the flat mapping for narrow rows (csrc/thn_flat.h): consecutive lanes own consecutive vectors across
rows and the row sums are segmented reductions.  Every row width from 2 to 32 vectors is forced through the launch
override (threads_per_row = vectors per row) in three storage types, with 1, 2 and 4 rows per lane, and compared with
the CPU oracle; row counts that end in the middle of a wave, a workgroup and a grid step; strided rows; and the
bit-level properties the row kernels have (run-to-run identical, a row's result independent of where it sits)."""
import ctypes

import pytest
import torch

from parity_util import run_and_compare
from TritonHub import _native
from TritonHub.Normalization import _launch

pytestmark = pytest.mark.gpu


def announce(msg):
    print(f"\n[flat] {msg}", flush=True)


class forced_flat:
    """Launch override that selects the flat kernels for rows of `n_vecs` vectors (not a power of two)."""

    def __init__(self, n_vecs, rows_each=0, bpc=0):
        self.args = (rows_each, n_vecs, 0, bpc)

    def __enter__(self):
        lib = _native.lib()
        for which in (0, 1):
            assert lib.thn_norm_set_launch_override(which, *self.args) == 0

    def __exit__(self, *exc):
        lib = _native.lib()
        for which in (0, 1):
            lib.thn_norm_set_launch_override(which, 0, 0, 0, 0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("kind", ["ln", "rms"])
def test_every_row_width_against_the_oracle(kind, dtype):
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    g = torch.Generator().manual_seed(31)
    for n_vecs in range(2, 33):
        if n_vecs & (n_vecs - 1) == 0:
            continue                      # powers of two fill the row kernels' lane groups: not a flat shape
        n = n_vecs * vec
        for rows_each in (1, 2, 4):
            rows_per_block = 4 * (64 // n_vecs) * rows_each
            for m in sorted({1, rows_per_block - 1, 3 * rows_per_block + 5, 1000 + n_vecs}):
                announce(f"{kind} {dtype} L={n_vecs} N={n} J={rows_each} M={m}")
                with forced_flat(n_vecs, rows_each):
                    for which in (0, 1):
                        q = _launch.query_launch(which, kind == "ln", m, n, dtype)
                        assert q[:3] == (rows_each, n_vecs, 256), q
                    x = (torch.randn(m, n, generator=g) * 2 + 0.5).to(dtype)
                    dy = torch.randn(m, n, generator=g).to(dtype)
                    w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype)
                    b = (0.1 * torch.randn(n, generator=g)).to(dtype) if kind == "ln" else None
                    run_and_compare(kind, x, dy, w, b, 1e-5, f"flat L={n_vecs} J={rows_each} M={m}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("kind", ["ln", "rms"])
def test_row_widths_off_the_128_bit_path(kind, dtype):
    """Rows that are not a whole number of vectors (one column more than n_vecs - 1 vectors, one less than n_vecs), every
    vector count from 2 to 32 -- powers of two included: off the 128-bit path the flat kernels take those too -- with 1
    and 2 rows per lane: the unaligned-window instances, whose last window overlaps its neighbour (its leading columns
    are stored twice and counted once in the row sums and in dW / dB)."""
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    g = torch.Generator().manual_seed(77)
    for n_vecs in range(2, 33):
        for n in sorted({(n_vecs - 1) * vec + 1, n_vecs * vec - 1}):
            for rows_each in (1, 2):
                rows_per_block = 4 * (64 // n_vecs) * rows_each
                for m in sorted({1, rows_per_block - 1, 3 * rows_per_block + 5}):
                    announce(f"{kind} {dtype} L={n_vecs} ragged N={n} J={rows_each} M={m}")
                    with forced_flat(n_vecs, rows_each):
                        for which in (0, 1):
                            q = _launch.query_launch(which, kind == "ln", m, n, dtype)
                            assert q[:3] == (rows_each, n_vecs, 256) and q[4] == 0, q
                        x = (torch.randn(m, n, generator=g) * 2 + 0.5).to(dtype)
                        dy = torch.randn(m, n, generator=g).to(dtype)
                        w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype)
                        b = (0.1 * torch.randn(n, generator=g)).to(dtype) if kind == "ln" else None
                        run_and_compare(kind, x, dy, w, b, 1e-5, f"flat ragged L={n_vecs} N={n} J={rows_each} M={m}")


def test_many_rows_hostile_mean_and_strided_views():
    """2^20 rows of 72 bf16 columns (every workgroup takes many steps), the hostile mean in float32, and rows that
    are not dense (column blocks of a wider buffer: the flat kernels address every lane's row by itself)."""
    g = torch.Generator().manual_seed(5)
    announce("bf16 1048577 x 72")
    m, n = 1048577, 72
    x = torch.randn(m, n, generator=g).bfloat16(); dy = torch.randn(m, n, generator=g).bfloat16()
    w = (1 + 0.1 * torch.randn(n, generator=g)).bfloat16(); b = (0.1 * torch.randn(n, generator=g)).bfloat16()
    with forced_flat(9):
        run_and_compare("ln", x, dy, w, b, 1e-6, "flat bf16 2^20 x 72", sample_chunks=8)
        run_and_compare("rms", x, dy, w, None, 1e-6, "flat bf16 2^20 x 72", sample_chunks=8)
    announce("f32 hostile mean 5000 x 68")
    m, n = 5000, 68
    x = 1000.0 + torch.randn(m, n, generator=g); dy = torch.randn(m, n, generator=g)
    w = 1 + 0.1 * torch.randn(n, generator=g); b = 0.1 * torch.randn(n, generator=g)
    with forced_flat(17):
        run_and_compare("ln", x, dy, w, b, 1e-6, "flat f32 hostile 68")
    announce("strided rows")
    lib = _native.lib()
    p = _native.ptr
    st = torch.cuda.current_stream().cuda_stream
    m, n, pitch = 777, 88, 128                      # 11 vectors of bf16 inside rows of 128 elements
    xb = torch.randn(m, pitch, generator=g).bfloat16().cuda(); gb = torch.randn(m, pitch, generator=g).bfloat16().cuda()
    wv = (1 + 0.1 * torch.randn(n, generator=g)).bfloat16().cuda(); bv = (0.1 * torch.randn(n, generator=g)).bfloat16().cuda()
    outs = []
    for flat in (True, False):
        y = torch.full((m, pitch), 7.0, dtype=torch.bfloat16, device="cuda"); dx = torch.full_like(y, 7.0)
        mean = torch.empty(m, device="cuda"); rstd = torch.empty(m, device="cuda")
        dw = torch.empty(n, dtype=torch.bfloat16, device="cuda"); db = torch.empty_like(dw)
        ctx = forced_flat(11) if flat else forced_flat(0)
        with ctx:
            nbytes = lib.thn_norm_bwd_workspace_bytes(m, n, 1, 1, _native.BF16)
            ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
            assert lib.thn_norm_fwd(p(xb), pitch, p(y), pitch, p(wv), p(bv), p(mean), p(rstd), m, n, 1e-5, _native.BF16,
                                    _native.BF16, st) == 0
            assert lib.thn_norm_bwd(p(xb), pitch, p(gb), pitch, p(dx), pitch, p(wv), p(mean), p(rstd), p(dw), p(db), p(ws),
                                    nbytes, m, n, _native.BF16, _native.BF16, st) == 0
        torch.cuda.synchronize()
        assert bool((y[:, n:] == 7.0).all()) and bool((dx[:, n:] == 7.0).all())       # the padding is untouched
        outs.append((y[:, :n].float(), dx[:, :n].float(), mean, rstd, dw.float(), db.float()))
    for a, c in zip(*outs):              # flat against the row kernels: the same quantities to a storage ulp
        assert torch.allclose(a, c, rtol=2e-2, atol=2e-2)


def test_bit_level_properties():
    """Run-to-run identical; a row's y and dx do not depend on where the row sits (the segmented sums depend on the
    vector count alone); both cache policies give the same bits."""
    g = torch.Generator().manual_seed(9)
    lib = _native.lib()
    p = _native.ptr
    st = torch.cuda.current_stream().cuda_stream
    m, n = 40000, 104                                     # 13 vectors of bf16
    x = torch.randn(m, n, generator=g).bfloat16().cuda(); dy = torch.randn(m, n, generator=g).bfloat16().cuda()
    w = (1 + 0.1 * torch.randn(n, generator=g)).bfloat16().cuda(); b = (0.1 * torch.randn(n, generator=g)).bfloat16().cuda()

    def run(xx, gg, rows, flag=0):
        y = torch.empty_like(xx); dx = torch.empty_like(xx)
        mean = torch.empty(rows, device="cuda"); rstd = torch.empty(rows, device="cuda")
        dw = torch.empty(n, dtype=torch.bfloat16, device="cuda"); db = torch.empty_like(dw)
        nbytes = lib.thn_norm_bwd_workspace_bytes(rows, n, 1, 1, _native.BF16)
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        assert lib.thn_norm_fwd(p(xx), n, p(y), n, p(w), p(b), p(mean), p(rstd), rows, n, 1e-5, _native.BF16 | flag,
                                _native.BF16, st) == 0
        assert lib.thn_norm_bwd(p(xx), n, p(gg), n, p(dx), n, p(w), p(mean), p(rstd), p(dw), p(db), p(ws), nbytes, rows, n,
                                _native.BF16, _native.BF16, st) == 0
        torch.cuda.synchronize()
        return y, dx, mean, rstd, dw, db

    with forced_flat(13):
        a = run(x, dy, m)
        c = run(x, dy, m, _native.X_STREAM)
        for u, v in zip(a, c):
            assert torch.equal(u, v)
        # rows 1000 ... 1999 on their own: another lane, another wave, another workgroup for every row
        sub = run(x[1000:2000].contiguous(), dy[1000:2000].contiguous(), 1000)
        for u, v in zip(a[:4], sub[:4]):
            assert torch.equal(u[1000:2000], v)
