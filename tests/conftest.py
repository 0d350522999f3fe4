"""Shared fixtures: import paths, the `gpu` marker, the benchmark input generators and the tolerance checks."""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "triton-hub_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box with -m gpu)")


# ---------------------------------------------------------------------------------------------------------
# The five benchmark configurations.  `rows` lets a test shrink M while keeping N and the data recipe.
# Inputs are generated on the CPU in float32 with a seeded generator, then cast (so the GPU path and the
# oracle see bit-identical storage values).
# ---------------------------------------------------------------------------------------------------------
CONFIGS = {
    # name: (kind, shape, dtype, has_bias)
    "c1_ln_f32_quickstart": ("ln", (2, 100, 128), torch.float32, True),
    "c2_rms_bf16_llm": ("rms", (8, 2048, 4096), torch.bfloat16, False),
    "c3_ln_bf16_wide": ("ln", (32768, 8192), torch.bfloat16, True),
    "c4_ln_f32_small_hidden": ("ln", (1048576, 256), torch.float32, True),
    "c5a_ln_f16_hostile": ("ln", (8192, 6000), torch.float16, True),
    "c5a_ln_f32_hostile": ("ln", (8192, 6000), torch.float32, True),
    "c5b_rms_f16_outliers": ("rms", (4096, 16384), torch.float16, False),
    "c5b_rms_f32_outliers": ("rms", (4096, 16384), torch.float32, False),
}
EPS = 1e-6


def make_case(name, rows=None, seed=0):
    """Returns dict(kind, x, dy, w, b, eps) of CPU tensors in the configuration's storage dtype."""
    kind, shape, dtype, has_bias = CONFIGS[name]
    if rows is not None:
        shape = (rows, shape[-1])
    n = shape[-1]
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g, dtype=torch.float32)
    if name.startswith("c5a"):
        x = x + 1000.0
    if name.startswith("c5b"):
        mask = torch.rand(shape, generator=g) < 0.001
        x = torch.where(mask, x * 100.0, x)
    dy = torch.randn(shape, generator=g, dtype=torch.float32)
    w = 1.0 + 0.1 * torch.randn(n, generator=g, dtype=torch.float32)
    b = 0.1 * torch.randn(n, generator=g, dtype=torch.float32) if has_bias else None
    cast = lambda t: None if t is None else t.to(dtype)
    return dict(kind=kind, x=cast(x), dy=cast(dy), w=cast(w), b=cast(b), eps=EPS, dtype=dtype)


FMT = {torch.float32: "fp32", torch.float16: "fp16", torch.bfloat16: "bf16", torch.float64: "fp64"}
EPS32 = 2.0 ** -24


def f64(t):
    return t.detach().to("cpu", torch.float64).numpy()


def check_elementwise(got, ref, scale, dtype, what, abs_tol=1e-5, noise=4.0):
    """The north-star tolerance for y and dx.

    float32 (and float64 storage, whose arithmetic is float32): max |got - ref| <= 1e-5; where |ref| > 21 a
    float32 cannot hold the value to 1e-5 any more (4 ulp exceed it) and the bound is 4 float32 ulp of ref (the
    outlier configuration has |y| up to ~130).
    float16 / bfloat16: |got - ref| <= 1 ulp of the output dtype at ref, plus the rounding noise of the
    float32 arithmetic that produced the value before it was narrowed: `noise` * 2^-24 * scale, where `scale`
    is the magnitude of the operands that were added or subtracted to form the result (parity_util spells it
    out).  It only matters where those operands cancel (|result| << scale): there a float32-accumulated
    result is not accurate to an ulp of a 16-bit type, whoever computes it.  For |y| ~ 1 the allowance is
    about 5e-7, against a bfloat16 ulp of 4e-3 to 8e-3.
    """
    from oracle import norm_oracle as no
    got = np.asarray(got, dtype=np.float64)
    err = np.abs(got - ref)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    if dtype in (torch.float32, torch.float64):
        bound = np.maximum(abs_tol, 4.0 * no.ulp(ref, "fp32"))
        ratio = err / bound
        worst = float(ratio.max()) if ratio.size else 0.0
        if worst > 1.0:
            i = np.unravel_index(int(ratio.argmax()), ratio.shape)
            raise AssertionError(f"{what}: abs error {err[i]:.3e} at {i} (got {got[i]!r}, ref {ref[i]!r}) exceeds "
                                 f"max(1e-5, 4 float32 ulp) = {bound[i]:.3e}")
        return worst
    bound = no.ulp(ref, FMT[dtype]) + noise * EPS32 * scale
    ratio = err / bound
    worst = float(ratio.max()) if ratio.size else 0.0
    if worst > 1.0:
        i = np.unravel_index(int(ratio.argmax()), ratio.shape)
        sc = np.broadcast_to(scale, ratio.shape)[i]
        raise AssertionError(f"{what}: error is {worst:.3f} x the (1 ulp + float32 noise) bound at {i}: got {got[i]!r}, "
                             f"ref {ref[i]!r}, ulp {no.ulp(ref[i], FMT[dtype])!r}, scale {sc!r}; "
                             f"{int((ratio > 1).sum())} of {ratio.size} elements over")
    return worst


def check_param_grad(got, ref, terms_sq_sum, dtype, what, abs_tol=1e-5):
    """Tolerance for dW / dB, sums of `n_rows` terms per column.

    The literal bound (max abs error 1e-5 in float32) cannot hold once |dW| ~ sqrt(M) has an ulp above 2e-5
    (M >~ 3e4), whatever the algorithm, so the bound is: 1e-5, or 1 ulp of the OUTPUT dtype at ref, whichever
    is larger, plus the float32 rounding of the M terms themselves.  Each dy*xhat carries the relative error of
    a float32 xhat (three roundings and the rounding of the saved rstd: about 1.1 * 2^-24 rms), independent
    from row to row, so a column sum has a standard error of about 1.1 * 2^-24 * sqrt(sum of term^2) and the
    worst of N columns sits 4 to 5 standard errors out: the allowance is 6 * 2^-24 * sqrt(sum of term^2)
    (`terms_sq_sum` is that sum per column; for unit-variance terms it is M).
    """
    from oracle import norm_oracle as no
    got = np.asarray(got, dtype=np.float64)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - ref)
    fmt = FMT[dtype] if dtype != torch.float64 else "fp32"
    bound = np.maximum(abs_tol if dtype in (torch.float32, torch.float64) else 0.0, no.ulp(ref, fmt)) \
        + 6.0 * EPS32 * np.sqrt(terms_sq_sum)
    ratio = err / bound
    worst = float(ratio.max())
    if worst > 1.0:
        i = int(ratio.argmax())
        raise AssertionError(f"{what}: error is {worst:.3f} x the bound at column {i}: got {got[i]!r}, ref {ref[i]!r}, "
                             f"max abs err {err.max():.3e}, ulp {no.ulp(ref[i], fmt)!r}")
    return worst


def check_stats(got, ref, what, rel_tol=1e-6, floor=0.0):
    """Saved mean / rstd: within 1e-6 relative.  `floor` is the absolute scale below which a mean counts as
    zero (a mean of N(0,1) data is ~1/sqrt(N): its error is measured against the row's spread, not itself)."""
    got = np.asarray(got, dtype=np.float64)
    err = np.abs(got - ref) / np.maximum(np.abs(ref), floor)
    worst = float(err.max()) if err.size else 0.0
    assert worst <= rel_tol, f"{what}: relative error {worst:.3e} > {rel_tol:.1e}"
    return worst


@pytest.fixture(scope="session")
def golden():
    path = os.path.join(ROOT, "tests", "golden", "norm_golden.npz")
    data = np.load(path, allow_pickle=False)
    cases = {}
    for key in data.files:
        name, field = key.split("/")
        cases.setdefault(name, {})[field] = data[key]
    return cases
