"""GPU test of thn_norm_bwd_static_workspace, the backward entry point that allocates nothing: its partial rows
go to a fixed array in device memory that the library owns.  It must give the bits of thn_norm_bwd (the same
kernels with a caller-supplied workspace) on two calls in a row, the second one smaller than the first, and refuse
problems whose partial rows do not fit the array.  Collected last: the file name sorts behind every other test."""
import ctypes

import pytest
import torch

from TritonHub import _native

pytestmark = pytest.mark.gpu

STATIC_BYTES = 16 * 1024 * 1024


def announce(msg):
    print(f"[no-alloc] {msg}", flush=True)          # names the case before its GPU work starts


def _case(kind, m, n, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(m, n, generator=g) * 1.5 + 0.25).to(dtype).cuda()
    dy = torch.randn(m, n, generator=g).to(dtype).cuda()
    w = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype).cuda()
    b = (0.1 * torch.randn(n, generator=g)).to(dtype).cuda() if kind == "ln" else None
    return x, dy, w, b


def _both_backwards(kind, m, n, dtype, seed, want_dw=True, want_db=True):
    lib = _native.lib()
    p = _native.ptr
    code = _native.dtype_code(dtype)
    st = torch.cuda.current_stream().cuda_stream
    ln = kind == "ln"
    x, dy, w, b = _case(kind, m, n, dtype, seed)
    y = torch.empty_like(x)
    mean = torch.empty(m, device="cuda") if ln else None
    rstd = torch.empty(m, device="cuda")
    assert lib.thn_norm_fwd(p(x), n, p(y), n, p(w), p(b), p(mean), p(rstd), m, n, 1e-6, code, code, st) == 0
    want_db = want_db and ln
    outs = []
    for static in (False, True):
        dx = torch.full_like(x, 3.0)
        dw = torch.full_like(w, 3.0) if want_dw else None
        db = torch.full_like(w, 3.0) if want_db else None
        if static:
            rc = lib.thn_norm_bwd_static_workspace(p(x), n, p(dy), n, p(dx), n, p(w), p(mean), p(rstd), p(dw), p(db), m, n,
                                                   code, code, st)
        else:
            nbytes = lib.thn_norm_bwd_workspace_bytes(m, n, int(want_dw), int(want_db), code)
            assert 0 <= nbytes <= STATIC_BYTES
            ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
            rc = lib.thn_norm_bwd(p(x), n, p(dy), n, p(dx), n, p(w), p(mean), p(rstd), p(dw), p(db), p(ws), nbytes, m, n,
                                  code, code, st)
        assert rc == 0, _native.strerror(rc)
        torch.cuda.synchronize()
        outs.append((dx, dw, db))
    (dx0, dw0, db0), (dx1, dw1, db1) = outs
    assert torch.equal(dx0, dx1)
    assert bool(torch.isfinite(dx1.float()).all())
    if want_dw:
        assert torch.equal(dw0, dw1) and not bool((dw1 == 3.0).all())
    if want_db:
        assert torch.equal(db0, db1) and not bool((db1 == 3.0).all())


def test_static_workspace_backward_matches_the_workspace_backward_twice_in_a_row():
    announce("static workspace: LayerNorm bf16 3000 x 4096, then RMSNorm f32 700 x 1024, then LayerNorm f16 513 x 520")
    _both_backwards("ln", 3000, 4096, torch.bfloat16, 1)      # 2 x 256 partial rows of 16 KiB: 8 MiB of the array
    _both_backwards("rms", 700, 1024, torch.float32, 2)       # a smaller problem right after: the array keeps stale rows
    _both_backwards("ln", 513, 520, torch.float16, 3)
    _both_backwards("ln", 300, 768, torch.float32, 4, want_dw=False)      # dB only
    _both_backwards("ln", 64, 256, torch.float32, 5, want_dw=False, want_db=False)   # no gradient: the array is not touched


def test_static_workspace_is_sized_by_the_grid_the_backward_launches():
    """512 rows of 16384 bf16 columns: the upper bound of thn_norm_bwd_workspace_bytes (one partial row per compute
    unit and gradient: 32 MiB) does not fit the array, but the backward over so few rows launches half the
    workgroups, and what those write does."""
    announce("static workspace: LayerNorm bf16 512 x 16384 (upper bound 32 MiB, 128 partial rows per gradient)")
    lib = _native.lib()
    m, n = 512, 16384
    shape = (ctypes.c_int32 * 5)()
    assert lib.thn_norm_query_launch(1, 1, m, n, _native.BF16, shape) == 0
    need = 2 * shape[3] * n * 4
    upper = lib.thn_norm_bwd_workspace_bytes(m, n, 1, 1, _native.BF16)
    if not (need <= STATIC_BYTES < upper):
        pytest.skip(f"this device launches {shape[3]} workgroups here: {need} bytes of {upper}")
    p = _native.ptr
    st = torch.cuda.current_stream().cuda_stream
    x, dy, w, b = _case("ln", m, n, torch.bfloat16, 6)
    y, mean, rstd = torch.empty_like(x), torch.empty(m, device="cuda"), torch.empty(m, device="cuda")
    code = _native.BF16
    assert lib.thn_norm_fwd(p(x), n, p(y), n, p(w), p(b), p(mean), p(rstd), m, n, 1e-6, code, code, st) == 0
    outs = []
    for static in (False, True):
        dx, dw, db = torch.full_like(x, 3.0), torch.full_like(w, 3.0), torch.full_like(w, 3.0)
        if static:
            rc = lib.thn_norm_bwd_static_workspace(p(x), n, p(dy), n, p(dx), n, p(w), p(mean), p(rstd), p(dw), p(db), m, n,
                                                   code, code, st)
        else:
            ws = torch.empty(upper, dtype=torch.uint8, device="cuda")
            rc = lib.thn_norm_bwd(p(x), n, p(dy), n, p(dx), n, p(w), p(mean), p(rstd), p(dw), p(db), p(ws), upper, m, n,
                                  code, code, st)
        assert rc == 0, _native.strerror(rc)
        torch.cuda.synchronize()
        outs.append((dx, dw, db))
    for a, c in zip(*outs):
        assert torch.equal(a, c) and not bool((c == 3.0).all())


def test_static_workspace_refuses_what_does_not_fit():
    announce("static workspace: limits")
    lib = _native.lib()
    p = _native.ptr
    st = torch.cuda.current_stream().cuda_stream
    m, n = 4096, 16384                                          # float32 LayerNorm: 2 x 256 partial rows of 64 KiB = 32 MiB
    need = lib.thn_norm_bwd_workspace_bytes(m, n, 1, 1, _native.F32)
    assert need > STATIC_BYTES
    # never read or written: the call returns before any launch (full size: the argument checks look at the spans)
    x, g, d = (torch.empty(m, n, device="cuda") for _ in range(3))
    v = torch.zeros(n, device="cuda")
    r = torch.zeros(m, device="cuda")
    rc = lib.thn_norm_bwd_static_workspace(p(x), n, p(g), n, p(d), n, p(v), p(r), p(r), p(v), p(v), m, n, _native.F32,
                                           _native.F32, st)
    assert rc == _native.E_WORKSPACE
    # the same errors as thn_norm_bwd for bad arguments
    assert lib.thn_norm_bwd_static_workspace(p(x), n, p(x), n, p(x), n, p(v), p(r), p(r), p(v), p(v), 8, n, 17,
                                             _native.F32, st) == _native.E_DTYPE
    assert lib.thn_norm_bwd_static_workspace(p(x), n, 0, n, p(x), n, p(v), p(r), p(r), p(v), p(v), 8, n, _native.F32,
                                             _native.F32, st) == _native.E_NULL
    assert lib.thn_norm_bwd_static_workspace(p(x), n, p(x), n, p(x), n, p(v), 0, p(r), p(v), p(v), 8, n, _native.F32,
                                             _native.F32, st) == _native.E_SHAPE          # RMSNorm has no dB
    torch.cuda.synchronize()
