"""Helpers of the GPU parity tests: run the HIP path through the Python operator interface (which calls the
C ABI), run the CPU oracle on the same storage values, and compare to the north-star tolerances."""
import numpy as np
import torch

from conftest import check_elementwise, check_param_grad, check_stats, f64
from oracle import c_oracle as co
from TritonHub.Normalization.layernorm import layernorm
from TritonHub.Normalization.rmsnorm import rmsnorm


def gpu_forward_backward(kind, x, dy, w, b, eps, device="cuda"):
    """x, dy, w, b: CPU tensors (w / b may be None).  Returns dict of GPU results (tensors on the device)."""
    xg = x.to(device).requires_grad_(True)
    wg = None if w is None else w.to(device).requires_grad_(True)
    bg = None if b is None else b.to(device).requires_grad_(True)
    if kind == "ln":
        y = layernorm.apply(xg, wg, bg, eps)
        saved = y.grad_fn.saved_tensors
        mean, rstd = saved[3], saved[4]
    else:
        assert b is None
        y = rmsnorm.apply(xg, wg, eps)
        mean, rstd = None, y.grad_fn.saved_tensors[2]
    y.backward(dy.to(device))
    torch.cuda.synchronize()
    return dict(y=y.detach(), dx=xg.grad, dw=None if wg is None else wg.grad, db=None if bg is None else bg.grad,
                mean=mean, rstd=rstd)


def compare_with_oracle(kind, x, dy, w, b, eps, out, what, chunk_rows=2048, sample_chunks=None):
    """Compares every output of the HIP path with the float64 C oracle, in row chunks.

    The oracle's backward is evaluated at the oracle's OWN float64 statistics: the expected dx / dW / dB are the
    exact functions of (x, dy, w), not functions of the float32-rounded statistics the GPU saved.
    `sample_chunks`: compare y / dx on that many evenly spread chunks only (dW / dB always use every row).
    Returns the worst ratios seen, for reporting.
    """
    dtype = x.dtype
    n = x.shape[-1]
    x2 = x.reshape(-1, n)
    dy2 = dy.reshape(-1, n)
    m = x2.shape[0]
    y2 = out["y"].reshape(-1, n)
    dx2 = out["dx"].reshape(-1, n)
    w64 = None if w is None else w.double().numpy()
    b64 = None if b is None else b.double().numpy()
    starts = list(range(0, m, chunk_rows))
    sampled = set(starts)
    if sample_chunks is not None and len(starts) > sample_chunks:
        idx = np.unique(np.linspace(0, len(starts) - 1, sample_chunks).round().astype(int))
        sampled = {starts[i] for i in idx}
    worst = dict(y=0.0, dx=0.0, mean=0.0, rstd=0.0, dw=0.0, db=0.0)
    dw_ref = np.zeros(n)
    db_ref = np.zeros(n)
    dw_sq = np.zeros(n)
    db_sq = np.zeros(n)
    rows_in_sq = 0
    for s in starts:
        e = min(s + chunk_rows, m)
        xc, dyc = x2[s:e], dy2[s:e]
        full = s in sampled
        if kind == "ln":
            yo, mean, rstd = co.layernorm_fwd(xc, w, b, eps, want_y=full)
            dxo, dwo, dbo = co.layernorm_bwd(xc, dyc, w, mean, rstd, has_bias=True, want_dx=full)
            db_ref += dbo
        else:
            yo, rstd = co.rmsnorm_fwd(xc, w, eps, want_y=full)
            mean = None
            dxo, dwo = co.rmsnorm_bwd(xc, dyc, w, rstd, want_dx=full)
        if dwo is not None:
            dw_ref += dwo
        # saved statistics: every row
        worst["rstd"] = max(worst["rstd"], check_stats(f64(out["rstd"][s:e]), rstd, f"{what} rstd rows {s}:{e}"))
        if kind == "ln":
            # a mean is compared against the spread of its row (1/rstd): means of N(0,1) rows are ~0
            worst["mean"] = max(worst["mean"], check_stats(f64(out["mean"][s:e]), mean, f"{what} mean rows {s}:{e}",
                                                           floor=1.0))
        if not full:
            continue
        xd, gd = xc.double().numpy(), dyc.double().numpy()
        mu = mean[:, None] if mean is not None else 0.0
        xhat = (xd - mu) * rstd[:, None]
        # Error model of a float32-accumulating implementation, used only for the 16-bit tolerance:
        #  - x - mean rounds relative to its operands: (|x| + |mean|)*rstd in units of the row's spread;
        #  - a row mean of N terms summed in float32 carries an error of about 2^-24 times the rms of the
        #    terms, so mean(x) is uncertain by ~2^-24/rstd, i.e. xhat by ~2^-24 (the "+ 1.0" below), and c1, c2
        #    by ~2^-24 times the rms of xhat*wdy and of wdy.
        xs = (np.abs(xd) + np.abs(mu)) * rstd[:, None] + 1.0
        y_scale = xs * (np.abs(w64) if w64 is not None else 1.0) + (np.abs(b64) if b64 is not None else 0.0)
        worst["y"] = max(worst["y"], check_elementwise(f64(y2[s:e]), yo.reshape(-1, n), y_scale, dtype,
                                                       f"{what} y rows {s}:{e}"))
        wdy = gd * (w64 if w64 is not None else 1.0)
        c1 = (xhat * wdy).mean(1, keepdims=True)
        c2 = wdy.mean(1, keepdims=True) if kind == "ln" else 0.0
        rms = lambda a: np.sqrt((a * a).mean(1, keepdims=True))
        dx_scale = (np.abs(wdy) + xs * np.abs(c1) + np.abs(c2) + np.abs(xhat) * rms(xhat * wdy)
                    + (rms(wdy) if kind == "ln" else 0.0)) * rstd[:, None]
        worst["dx"] = max(worst["dx"], check_elementwise(f64(dx2[s:e]), dxo.reshape(-1, n), dx_scale, dtype,
                                                         f"{what} dx rows {s}:{e}"))
        dw_sq += ((gd * xhat) ** 2).sum(0)
        db_sq += (gd ** 2).sum(0)
        rows_in_sq += e - s
    scale_up = m / max(rows_in_sq, 1)        # sampled chunks stand for all rows
    if out["dw"] is not None:
        worst["dw"] = check_param_grad(f64(out["dw"]), dw_ref, dw_sq * scale_up, out["dw"].dtype, f"{what} dW")
    if out["db"] is not None:
        worst["db"] = check_param_grad(f64(out["db"]), db_ref, db_sq * scale_up, out["db"].dtype, f"{what} dB")
    return worst


def run_and_compare(kind, x, dy, w, b, eps, what, **kw):
    out = gpu_forward_backward(kind, x, dy, w, b, eps)
    return compare_with_oracle(kind, x, dy, w, b, eps, out, what, **kw), out
