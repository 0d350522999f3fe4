"""Outputs with a row pitch wider than the row, through the C ABI: every family writes the N columns of each row
and nothing else -- the padding behind each row (which may belong to another view of the caller's buffer) and the
elements before and after the output keep their sentinel.  Row widths on the 128-bit path, on the unaligned-window
path (whose 16-byte windows are moved back to end at the row end) and shorter than one vector; pitches that keep
rows 16-byte aligned and pitches that do not."""
import ctypes

import pytest
import torch

from TritonHub import _native

pytestmark = pytest.mark.gpu
SENTINEL = 768.0            # exact in bfloat16
WIDTHS = [1, 3, 7, 8, 100, 101, 1024, 4099, 6000]
PADS = [3, 16]


def padded(m, n, pad, dtype, lead=5):
    """A sentinel-filled buffer and the address of an (m, n) view with row pitch n + pad that starts `lead` elements in."""
    buf = torch.full((lead + m * (n + pad) + 9,), SENTINEL, device="cuda", dtype=dtype)
    return buf, buf.data_ptr() + lead * buf.element_size(), lead


def check_guards(buf, m, n, pad, lead, what):
    got = buf.cpu().float()
    assert bool((got[:lead] == SENTINEL).all()), f"{what}: wrote before the output"
    body = got[lead:lead + m * (n + pad)].reshape(m, n + pad)
    assert bool((body[:, n:] == SENTINEL).all()), f"{what}: wrote into the padding behind a row"
    assert bool((got[lead + m * (n + pad):] == SENTINEL).all()), f"{what}: wrote behind the output"
    assert bool((body[:, :n] != SENTINEL).all()), f"{what}: left output elements unwritten"
    return body[:, :n]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pad", PADS)
@pytest.mark.parametrize("n", WIDTHS)
def test_every_family_keeps_to_its_rows(n, pad, dtype):
    print(f"\n[case] output guards N={n} pad={pad} {dtype}", flush=True)
    lib = _native.lib()
    st = torch.cuda.current_stream().cuda_stream
    code = _native.dtype_code(dtype)
    m = 37
    pitch = n + pad
    g = torch.Generator(device="cuda").manual_seed(n * 31 + pad)
    x = (0.3 + torch.randn(m, n, device="cuda", generator=g)).to(dtype)
    dy = torch.randn(m, n, device="cuda", generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(n, device="cuda", generator=g)).to(dtype)
    b = (0.1 * torch.randn(n, device="cuda", generator=g)).to(dtype)
    mean = torch.empty(m, device="cuda")
    rstd = torch.empty(m, device="cuda")

    # LayerNorm forward / backward (and the same kernels with an epilogue)
    ybuf, yptr, lead = padded(m, n, pad, dtype)
    assert lib.thn_norm_fwd(x.data_ptr(), n, yptr, pitch, w.data_ptr(), b.data_ptr(), mean.data_ptr(), rstd.data_ptr(),
                            m, n, 1e-5, code, code, st) == 0
    y = check_guards(ybuf, m, n, pad, lead, "norm forward")
    ref = torch.nn.functional.layer_norm(x.float(), (n,), w.float(), b.float(), 1e-5)
    assert torch.allclose(y, ref.cpu(), atol=3e-2 if dtype == torch.bfloat16 else 1e-4, rtol=2e-2)
    nbytes = lib.thn_norm_bwd_workspace_bytes(m, n, 1, 1, code)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    dw, db = torch.empty_like(w), torch.empty_like(w)
    dxbuf, dxptr, lead = padded(m, n, pad, dtype)
    assert lib.thn_norm_bwd(x.data_ptr(), n, dy.data_ptr(), n, dxptr, pitch, w.data_ptr(), mean.data_ptr(),
                            rstd.data_ptr(), dw.data_ptr(), db.data_ptr(), ws.data_ptr(), nbytes, m, n, code, code,
                            st) == 0
    check_guards(dxbuf, m, n, pad, lead, "norm backward")
    ybuf, yptr, lead = padded(m, n, pad, dtype)
    assert lib.thn_norm_act_fwd(x.data_ptr(), n, yptr, pitch, w.data_ptr(), b.data_ptr(), mean.data_ptr(),
                                rstd.data_ptr(), m, n, 1e-5, _native.ACT_SILU, code, code, st) == 0
    check_guards(ybuf, m, n, pad, lead, "norm+act forward")
    nbytes = lib.thn_norm_act_bwd_workspace_bytes(m, n, 1, 1, _native.ACT_SILU, code)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    dxbuf, dxptr, lead = padded(m, n, pad, dtype)
    assert lib.thn_norm_act_bwd(x.data_ptr(), n, dy.data_ptr(), n, dxptr, pitch, w.data_ptr(), b.data_ptr(),
                                mean.data_ptr(), rstd.data_ptr(), dw.data_ptr(), db.data_ptr(), ws.data_ptr(), nbytes,
                                m, n, _native.ACT_SILU, code, code, st) == 0
    check_guards(dxbuf, m, n, pad, lead, "norm+act backward")

    # softmax forward / backward
    ybuf, yptr, lead = padded(m, n, pad, dtype)
    assert lib.thn_softmax_fwd(x.data_ptr(), n, yptr, pitch, m, n, _native.SOFTMAX, code, st) == 0
    y = check_guards(ybuf, m, n, pad, lead, "softmax forward")
    assert torch.allclose(y.sum(1), torch.ones(m), atol=2e-2 if dtype == torch.bfloat16 else 1e-5)
    ysaved = torch.softmax(x.float(), -1).to(dtype)
    dxbuf, dxptr, lead = padded(m, n, pad, dtype)
    assert lib.thn_softmax_bwd(ysaved.data_ptr(), n, dy.data_ptr(), n, dxptr, pitch, m, n, _native.SOFTMAX, code,
                               st) == 0
    check_guards(dxbuf, m, n, pad, lead, "softmax backward")

    # element-wise activation on strided rows
    ybuf, yptr, lead = padded(m, n, pad, dtype)
    assert lib.thn_act_fwd(x.data_ptr(), n, yptr, pitch, m, n, _native.ACT_GELU, 0.0, 0.0, code, st) == 0
    check_guards(ybuf, m, n, pad, lead, "activation forward")
    dxbuf, dxptr, lead = padded(m, n, pad, dtype)
    assert lib.thn_act_bwd(x.data_ptr(), n, dy.data_ptr(), n, dxptr, pitch, m, n, _native.ACT_GELU, 0.0, 0.0, code,
                           st) == 0
    check_guards(dxbuf, m, n, pad, lead, "activation backward")

    # normalize forward / backward, p-norm backward (one batch of m rows)
    norms = torch.empty(m, device="cuda", dtype=dtype)
    ybuf, yptr, lead = padded(m, n, pad, dtype)
    assert lib.thn_normalize_fwd(x.data_ptr(), m * n, n, yptr, m * pitch, pitch, norms.data_ptr(), 1, m, n, 2.0, 1e-6,
                                 code, st) == 0
    check_guards(ybuf, m, n, pad, lead, "normalize forward")
    yn = torch.nn.functional.normalize(x.float(), dim=-1).to(dtype)
    dxbuf, dxptr, lead = padded(m, n, pad, dtype)
    assert lib.thn_normalize_bwd(x.data_ptr(), m * n, n, yn.data_ptr(), m * n, n, norms.data_ptr(), dy.data_ptr(), m * n,
                                 n, dxptr, m * pitch, pitch, 1, m, n, 2.0, code, st) == 0
    check_guards(dxbuf, m, n, pad, lead, "normalize backward")
    dn = torch.rand(m, device="cuda", generator=g).to(dtype)
    dxbuf, dxptr, lead = padded(m, n, pad, dtype)
    assert lib.thn_pnorm_bwd(x.data_ptr(), m * n, n, norms.data_ptr(), dn.data_ptr(), dxptr, m * pitch, pitch, 1, m, n,
                             2.0, code, st) == 0
    torch.cuda.synchronize()
    check_guards(dxbuf, m, n, pad, lead, "p-norm backward")


@pytest.mark.parametrize("dtype,n", [(torch.float32, 20001), (torch.bfloat16, 40003), (torch.bfloat16, 65544)])
@pytest.mark.parametrize("pad", PADS)
def test_looping_kernels_keep_to_their_rows(n, pad, dtype):
    """Rows wider than 64 KiB (the looping kernels of the softmax and p-norm families), same guards."""
    print(f"\n[case] output guards, wide rows N={n} pad={pad} {dtype}", flush=True)
    lib = _native.lib()
    st = torch.cuda.current_stream().cuda_stream
    code = _native.dtype_code(dtype)
    m = 9
    pitch = n + pad
    g = torch.Generator(device="cuda").manual_seed(n + pad)
    x = (0.3 + torch.randn(m, n, device="cuda", generator=g)).to(dtype)
    dy = torch.randn(m, n, device="cuda", generator=g).to(dtype)
    for kind in (_native.SOFTMAX, _native.LOGSOFTMAX):
        ybuf, yptr, lead = padded(m, n, pad, dtype)
        assert lib.thn_softmax_fwd(x.data_ptr(), n, yptr, pitch, m, n, kind, code, st) == 0
        check_guards(ybuf, m, n, pad, lead, f"softmax forward kind {kind}")
        ysaved = (torch.softmax(x.float(), -1) if kind == _native.SOFTMAX else torch.log_softmax(x.float(), -1)).to(dtype)
        dxbuf, dxptr, lead = padded(m, n, pad, dtype)
        assert lib.thn_softmax_bwd(ysaved.data_ptr(), n, dy.data_ptr(), n, dxptr, pitch, m, n, kind, code, st) == 0
        check_guards(dxbuf, m, n, pad, lead, f"softmax backward kind {kind}")
    norms = torch.empty(m, device="cuda", dtype=dtype)
    for p in (2.0, 3.0, 2.5):
        ybuf, yptr, lead = padded(m, n, pad, dtype)
        assert lib.thn_normalize_fwd(x.data_ptr(), m * n, n, yptr, m * pitch, pitch, norms.data_ptr(), 1, m, n, p, 1e-6,
                                     code, st) == 0
        y = check_guards(ybuf, m, n, pad, lead, f"normalize forward p={p}")
        dxbuf, dxptr, lead = padded(m, n, pad, dtype)
        yn = y.to(dtype).cuda()
        assert lib.thn_normalize_bwd(x.data_ptr(), m * n, n, yn.data_ptr(), m * n, n, norms.data_ptr(), dy.data_ptr(),
                                     m * n, n, dxptr, m * pitch, pitch, 1, m, n, p, code, st) == 0
        check_guards(dxbuf, m, n, pad, lead, f"normalize backward p={p}")
        dn = torch.rand(m, device="cuda", generator=g).to(dtype)
        dxbuf, dxptr, lead = padded(m, n, pad, dtype)
        assert lib.thn_pnorm_bwd(x.data_ptr(), m * n, n, norms.data_ptr(), dn.data_ptr(), dxptr, m * pitch, pitch, 1, m,
                                 n, p, code, st) == 0
        torch.cuda.synchronize()
        check_guards(dxbuf, m, n, pad, lead, f"p-norm backward p={p}")
