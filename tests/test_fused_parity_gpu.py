"""GPU parity tests of LayerNorm / RMSNorm with an activation epilogue (thn_norm_act_fwd / thn_norm_act_bwd).

Expected values: the float64 oracles composed without any intermediate rounding -- z = norm(x), y = act(z);
g = dy * act'(z), then the norm backward with g as upstream gradient.  Tolerances are those of the norm path, with
the float32 error of the recomputed pre-activation carried into the backward's allowance.  The chained GPU modules
(which round z to the storage type in between) must agree to within a few storage ulp.
"""
import os
import re

import numpy as np
import pytest
import torch

from conftest import ROOT, check_elementwise, check_param_grad, check_stats, f64
from oracle import act_oracle as ao
from oracle import norm_oracle as no
from TritonHub import _native
from TritonHub.Activations import GeLU, ReLU, SiLU
from TritonHub.Normalization import LayerNorm, RMSNorm
from TritonHub.Normalization._launch import query_launch
from TritonHub.Normalization.fused import LayerNormActivation, RMSNormActivation

pytestmark = pytest.mark.gpu
ACTS = ["gelu", "gelu_tanh", "silu", "relu"]


def announce(msg):
    print(f"\n[case] {msg}", flush=True)


def make(shape, dtype, seed, affine=True, bias=True, x_shift=0.0):
    g = torch.Generator().manual_seed(seed)
    n = shape[-1]
    x = (torch.randn(shape, generator=g) + x_shift).to(dtype)
    dy = torch.randn(shape, generator=g).to(dtype)
    w = (1 + 0.3 * torch.randn(n, generator=g)).to(dtype) if affine else None
    b = (0.3 * torch.randn(n, generator=g)).to(dtype) if (affine and bias) else None
    return x, dy, w, b


def run_and_compare(kind, act, x, dy, w, b, eps, what, x_gpu=None, dy_gpu=None):
    dtype = x.dtype
    n = x.shape[-1]
    if kind == "ln":
        mod = LayerNormActivation(n, act, eps=eps, elementwise_affine=w is not None, bias=b is not None, device="cuda", dtype=dtype)
    else:
        mod = RMSNormActivation(n, act, eps=eps, elementwise_affine=w is not None, device="cuda", dtype=dtype)
    with torch.no_grad():
        if w is not None:
            mod.weight.copy_(w)
        if b is not None:
            mod.bias.copy_(b)
    xg = (x.cuda() if x_gpu is None else x_gpu).requires_grad_(True)
    y = mod(xg)
    saved = y.grad_fn.saved_tensors
    y.backward(dy.cuda() if dy_gpu is None else dy_gpu)
    torch.cuda.synchronize()
    assert y.dtype == dtype and y.shape == x.shape and xg.grad.shape == x.shape

    x64 = f64(x).reshape(-1, n); g64 = f64(dy).reshape(-1, n)
    w64 = None if w is None else f64(w); b64 = None if b is None else f64(b)
    if kind == "ln":
        z, mean, rstd = no.layernorm_fwd(x64, w64, b64, eps)
        check_stats(f64(saved[3]), mean, f"{what} mean", floor=1.0)
        check_stats(f64(saved[4]), rstd, f"{what} rstd")
    else:
        z, rstd = no.rmsnorm_fwd(x64, w64, eps)
        mean = None
        check_stats(f64(saved[2]), rstd, f"{what} rstd")
    mu = mean[:, None] if mean is not None else 0.0
    xs = (np.abs(x64) + np.abs(mu)) * rstd[:, None] + 1.0
    z_scale = xs * (np.abs(w64) if w64 is not None else 1.0) + (np.abs(b64) if b64 is not None else 0.0)
    check_elementwise(f64(y).reshape(-1, n), ao.fwd(act, z), z_scale + 1.0, dtype, f"{what} y")

    g_eff = ao.bwd(act, z, g64)                              # dy * act'(z)
    if kind == "ln":
        dx_ref, dw_ref, db_ref = no.layernorm_bwd(x64, g_eff, w64, mean, rstd, has_bias=b is not None)
    else:
        dx_ref, dw_ref = no.rmsnorm_bwd(x64, g_eff, w64, rstd)
        db_ref = None
    xhat = (x64 - mu) * rstd[:, None]
    # the recomputed z carries ~2^-24 * z_scale of float32 error; act' has slope <= ~1.2, so g_eff is uncertain by
    # about |dy| * 2^-24 * z_scale on top of its own rounding
    g_abs = np.abs(g_eff) + np.abs(g64) * z_scale
    wdy = g_abs * (np.abs(w64) if w64 is not None else 1.0)
    rms = lambda a: np.sqrt((a * a).mean(1, keepdims=True))
    dx_scale = (wdy + xs * rms(xhat * wdy) + rms(wdy) + np.abs(xhat) * rms(xhat * wdy)) * rstd[:, None]
    check_elementwise(f64(xg.grad).reshape(-1, n), dx_ref, dx_scale, dtype, f"{what} dx")
    if w is not None:
        check_param_grad(f64(mod.weight.grad), dw_ref, ((g_abs * xhat) ** 2).sum(0), dtype, f"{what} dW")
    if b is not None:
        check_param_grad(f64(mod.bias.grad), db_ref, (g_abs ** 2).sum(0), dtype, f"{what} dB")
    return mod, y.detach(), xg.grad


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("kind", ["ln", "rms"])
def test_against_composed_oracles(kind, act, dtype):
    for shape in ((2, 100, 128), (300, 1024), (64, 4096), (17, 6000)):
        announce(f"fused {kind} {act} {dtype} {shape}")
        x, dy, w, b = make(shape, dtype, seed=shape[-1], bias=kind == "ln")
        run_and_compare(kind, act, x, dy, w, b, 1e-5, f"{kind}+{act} {shape} {dtype}")


@pytest.mark.parametrize("dtype,widths", [(torch.bfloat16, (16384, 20480, 24576, 28672, 32768)), (torch.float16, (26632,)),
                                          (torch.float32, (12288, 16384))])
def test_wide_rows_many_per_workgroup(dtype, widths):
    # rows of 32-64 KiB (1024-thread workgroups; LayerNorm over 16-bit rows: 512 threads with 5-8 vectors each), with
    # more rows than the grid has workgroups
    for n in widths:
        for kind, act in (("ln", "gelu_tanh"), ("rms", "silu")):
            announce(f"fused wide {kind} {act} {dtype} N={n}")
            x, dy, w, b = make((520, n), dtype, seed=n, bias=kind == "ln")
            run_and_compare(kind, act, x, dy, w, b, 1e-5, f"{kind}+{act} wide N={n} {dtype}")


@pytest.mark.parametrize("affine,bias", [(True, True), (True, False), (False, False)])
@pytest.mark.parametrize("kind", ["ln", "rms"])
def test_constructor_variants_and_hostile_mean(kind, affine, bias):
    if kind == "rms" and bias:
        pytest.skip("RMSNorm has no bias")
    announce(f"fused variants {kind} affine={affine} bias={bias}")
    for dtype in (torch.float32, torch.bfloat16):
        x, dy, w, b = make((200, 768), dtype, seed=5, affine=affine, bias=bias and kind == "ln")
        run_and_compare(kind, "gelu", x, dy, w, b, 1e-6, f"{kind} affine={affine} bias={bias} {dtype}")
    # rows whose mean dwarfs their spread: the backward must rebuild z from the corrected xhat
    x, dy, w, b = make((256, 6000), torch.float32, seed=6, affine=affine, bias=bias and kind == "ln", x_shift=1000.0 if kind == "ln" else 0.0)
    run_and_compare(kind, "silu", x, dy, w, b, 1e-6, f"{kind} hostile")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64])
@pytest.mark.parametrize("n", [1, 2, 7, 33, 100, 257, 1000, 4099])
def test_ragged_hidden_sizes(n, dtype):
    announce(f"fused ragged N={n} {dtype}")
    for kind, act in (("ln", "gelu_tanh"), ("rms", "silu"), ("ln", "relu")):
        x, dy, w, b = make((37, n), dtype, seed=n, bias=kind == "ln")
        run_and_compare(kind, act, x, dy, w, b, 1e-5, f"{kind}+{act} N={n}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_strided_and_misaligned_views(dtype):
    announce(f"fused strides {dtype}")
    g = torch.Generator().manual_seed(12)
    base = torch.randn(40, 640, generator=g).to(dtype); gbase = torch.randn(40, 640, generator=g).to(dtype)
    bg, gg = base.cuda(), gbase.cuda()
    for i, view in enumerate((lambda t: t[:, :512], lambda t: t[:, 3:515], lambda t: t[::2, 64:576], lambda t: t[:, :512].reshape(5, 8, 512))):
        xv, gv = view(base), view(gbase)
        n = xv.shape[-1]
        w = (1 + 0.2 * torch.randn(n, generator=g)).to(dtype); b = (0.2 * torch.randn(n, generator=g)).to(dtype)
        run_and_compare("ln", "gelu", xv.contiguous(), gv.contiguous(), w, b, 1e-5, f"view {i}", x_gpu=view(bg).detach(), dy_gpu=view(gg))
        run_and_compare("rms", "silu", xv.contiguous(), gv.contiguous(), w, None, 1e-5, f"view {i}", x_gpu=view(bg).detach(), dy_gpu=view(gg))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_agrees_with_the_chained_modules(dtype):
    """act(norm(x)) through the fused module against Activation()(Norm()(x)) on the GPU: the chained path rounds the
    intermediate to the storage type, so the two agree to a few storage ulp, not bit for bit (exactly for ReLU's
    forward in float32, where the intermediate rounding is the identity)."""
    announce(f"fused vs chained {dtype}")
    torch.manual_seed(3)
    x = torch.randn(4096, 2048, device="cuda", dtype=dtype); dy = torch.randn_like(x)
    tol = dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    for kind, act, chain_act in (("ln", "gelu", GeLU()), ("ln", "gelu_tanh", GeLU("tanh")), ("rms", "silu", SiLU()), ("ln", "relu", ReLU())):
        if kind == "ln":
            fused = LayerNormActivation(2048, act, device="cuda", dtype=dtype); plain = LayerNorm(2048, device="cuda", dtype=dtype)
        else:
            fused = RMSNormActivation(2048, act, device="cuda", dtype=dtype); plain = RMSNorm(2048, device="cuda", dtype=dtype)
        with torch.no_grad():
            fused.weight.normal_(1.0, 0.2); plain.weight.copy_(fused.weight)
            if kind == "ln":
                fused.bias.normal_(0.0, 0.2); plain.bias.copy_(fused.bias)
        a = x.clone().requires_grad_(True); c = x.clone().requires_grad_(True)
        ya = fused(a); ya.backward(dy)
        yc = chain_act(plain(c)); yc.backward(dy)
        assert torch.allclose(ya, yc, **tol)
        if act == "relu":
            # where the pre-activation is within rounding of 0 the two paths can land on different sides of it: the
            # gradient of that element (and, through c1 / c2, a trace of its row) differs; such elements are rare
            far = (a.grad - c.grad).abs() > tol["atol"] + tol["rtol"] * c.grad.abs()
            assert float(far.any(dim=1).float().mean()) < 5e-3          # a handful of the 4096 rows
        else:
            assert torch.allclose(a.grad, c.grad, **tol)
        wt = dict(rtol=1e-4, atol=2e-3) if dtype == torch.float32 else dict(rtol=3e-2, atol=1.0)
        if act == "relu":
            wt["atol"] = 8.0             # one flipped element moves its column's sum by a whole term dy*xhat
        assert torch.allclose(fused.weight.grad, plain.weight.grad, **wt)
        if act == "relu" and dtype == torch.float32:
            assert torch.equal(ya, yc)


def test_empty_input_and_c_abi_errors():
    announce("fused empty / errors")
    m = LayerNormActivation(64, "gelu", device="cuda")
    x = torch.empty(0, 64, device="cuda", requires_grad=True)
    y = m(x); y.sum().backward()
    assert y.shape == (0, 64) and x.grad.shape == (0, 64) and bool((m.weight.grad == 0).all())
    lib = _native.lib()
    st = torch.cuda.current_stream().cuda_stream
    xb = torch.randn(8, 64, device="cuda"); yb = torch.empty_like(xb); rstd = torch.empty(8, device="cuda"); bias = torch.zeros(64, device="cuda")
    p = _native.ptr
    # RMSNorm (mean == NULL) takes no bias
    assert lib.thn_norm_act_fwd(p(xb), 64, p(yb), 64, 0, p(bias), 0, p(rstd), 8, 64, 1e-5, 0, _native.F32, _native.F32, st) == _native.E_SHAPE
    assert lib.thn_norm_act_fwd(p(xb), 64, p(yb), 64, 0, 0, 0, p(rstd), 8, 64, 1e-5, 7, _native.F32, _native.F32, st) == _native.E_SHAPE
    assert lib.thn_norm_act_fwd(p(xb), 64, p(yb), 64, 0, 0, 0, p(rstd), 8, 64, 1e-5, 3, _native.F32, _native.F32, st) == 0
    torch.cuda.synchronize()
    ref = torch.relu(xb * torch.rsqrt((xb * xb).mean(1, keepdim=True) + 1e-5))
    assert torch.allclose(yb, ref, atol=1e-6)


def fused_shapes():
    text = open(os.path.join(ROOT, "triton-hub_amd", "csrc", "thn_fused_dispatch.h")).read()
    out = []
    for macro in ("THN_FUSED_FWD_SHAPES", "THN_FUSED_BWD_SHAPES"):
        body = re.search(r"#define " + macro + r"\(X\)(.*?)\n\n", text, re.S).group(1)
        out.append([(int(k), int(t), int(b)) for k, t, b in re.findall(r"X\((\d+), (\d+), (\d+)\)", body)])
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_every_compiled_launch_shape(dtype):
    lib = _native.lib()
    fwd_shapes, bwd_shapes = fused_shapes()
    assert len(fwd_shapes) >= 12 and len(bwd_shapes) >= 10
    vec = 16 // torch.empty(0, dtype=dtype).element_size()
    try:
        for which, shapes in ((9, fwd_shapes), (10, bwd_shapes)):
            for k, tpr, block in shapes:
                for n_vecs in sorted({k * tpr, max((k - 1) * tpr + 1, k * tpr - tpr // 2 - 1)}):
                    n = n_vecs * vec
                    if n * (16 // vec) > 65536:
                        continue
                    rows_per_block = block // tpr
                    m = 2 * rows_per_block + max(1, rows_per_block // 2)
                    announce(f"fused shape family={which} K={k} TPR={tpr} block={block} N={n} M={m} {dtype}")
                    assert lib.thn_norm_set_launch_override(which, k, tpr, block, 0) == 0
                    assert query_launch(which, True, m, n, dtype)[:3] == (k, tpr, block)
                    x, dy, w, b = make((m, n), dtype, seed=k * 100 + tpr)
                    run_and_compare("ln", "gelu", x, dy, w, b, 1e-5, f"ln shape {k},{tpr},{block}")
                    run_and_compare("rms", "silu", x, dy, w, None, 1e-5, f"rms shape {k},{tpr},{block}")
                    assert lib.thn_norm_set_launch_override(which, 0, 0, 0, 0) == 0
    finally:
        lib.thn_norm_set_launch_override(9, 0, 0, 0, 0)
        lib.thn_norm_set_launch_override(10, 0, 0, 0, 0)


def test_frozen_bias_of_another_dtype_without_weight():
    """layernorm_act.apply(x, None, bias, ...) with 16-bit x and a float32 bias that does not require a gradient:
    the backward still reads the bias (it rebuilds the pre-activation from it) and must read it as float32.  dx equals
    the dx of the same call with a trainable bias, bit for bit."""
    from TritonHub.Normalization.fused import layernorm_act
    announce("fused LayerNorm, no weight, frozen float32 bias, bf16 rows")
    g = torch.Generator().manual_seed(11)
    x = torch.randn(300, 1024, generator=g).to(torch.bfloat16).cuda()
    dy = torch.randn(300, 1024, generator=g).to(torch.bfloat16).cuda()
    bias = (0.5 * torch.randn(1024, generator=g)).cuda()                     # float32
    outs = []
    for trainable in (True, False):
        a = x.clone().requires_grad_(True)
        b = bias.clone().requires_grad_(trainable)
        y = layernorm_act.apply(a, None, b, 1e-5, _native.ACT_GELU)
        y.backward(dy)
        torch.cuda.synchronize()
        outs.append((y.detach().clone(), a.grad.clone()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    # and against float64: z = xhat + b, y = gelu(z), dx = layernorm backward of dy * gelu'(z)
    x64 = f64(x); z, mean, rstd = no.layernorm_fwd(x64, None, f64(bias), 1e-5)
    dx_ref, _, _ = no.layernorm_bwd(x64, ao.bwd("gelu", z, f64(dy)), None, mean, rstd, has_bias=False)
    assert np.abs(f64(outs[1][1]) - dx_ref).max() < 0.02                    # bf16 dx of O(1) values: 2-3 ulp at most
