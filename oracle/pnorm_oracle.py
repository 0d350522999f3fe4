"""CPU oracle for the row p-norm / normalize operators, forward + backward (TEST INFRASTRUCTURE ONLY).

Float64 numpy restatement of the reference's ``TritonHub/Ops/norm.py`` and ``normalize.py``; imported by
``tests/`` only.  x: (..., K); norms, dnorms: (...).

* ``norm_fwd``       follows ``Ops/norm.py:24-40``:  sum |x|^p over the row (p=1: sum |x|, p=2: sum x*x), the
  p-th root (sqrt for p=2), then ``maximum(out, eps)``.  Rounding to the storage type (``:41``) is the caller's.
* ``norm_bwd``       follows ``Ops/norm.py:83-100``: p=1: g*sign(x); p=2: g*x/n; else g*sign(x)*|x|^(p-1)/n^(p-1),
  with n the SAVED (storage-rounded) norms.
* ``normalize_fwd``  follows ``Ops/normalize.py:27-31``: x / n, with n the storage-rounded norms the first kernel
  wrote (``normalize.py:48-50``); the caller passes that rounded n.
* ``normalize_bwd``  follows ``Ops/normalize.py:81-115``: proj = sum(y*g) (p=1: sum(x*g));
  p=1: g/n - sign(x)*(proj/(n*n)); p=2: (g - y*proj)/n; else g/n - sign(x)*|x|^(p-1)*(proj/(n^(p-1)*n)),
  with y and n the SAVED outputs of the forward.

Pinned in tests/test_pnorm_oracle_pins.py against torch's float64 CPU ``torch.norm`` / ``F.normalize`` and
autograd (live and frozen in tests/golden/pnorm_golden.npz), finite differences, closed forms, invariants.
"""
import numpy as np


def norm_fwd(x, p=2, eps=1e-6):
    x = np.asarray(x, dtype=np.float64)
    if p == 1:
        out = np.abs(x).sum(-1)
    elif p == 2:
        out = np.sqrt((x * x).sum(-1))
    else:
        out = (np.abs(x) ** p).sum(-1) ** (1.0 / p)
    # tl.maximum with its default NaN handling returns the other operand for a NaN (norm.py:40): a row that
    # holds a NaN comes out as eps
    return np.fmax(out, eps)


def norm_bwd(x, norms, dnorms, p=2):
    x = np.asarray(x, dtype=np.float64)
    g = np.asarray(dnorms, dtype=np.float64)[..., None]
    n = np.asarray(norms, dtype=np.float64)[..., None]
    if p == 1:
        return g * np.sign(x)
    if p == 2:
        return (g * x) / n
    return (g * np.sign(x) * np.abs(x) ** (p - 1)) / n ** (p - 1)


def normalize_fwd(x, norms):
    return np.asarray(x, dtype=np.float64) / np.asarray(norms, dtype=np.float64)[..., None]


def normalize_bwd(x, y, norms, dy, p=2):
    x = np.asarray(x, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    g = np.asarray(dy, dtype=np.float64)
    n = np.asarray(norms, dtype=np.float64)[..., None]
    if p == 1:
        proj = (x * g).sum(-1, keepdims=True)
        return g / n - np.sign(x) * (proj / (n * n))
    proj = (y * g).sum(-1, keepdims=True)
    if p == 2:
        return (g - y * proj) / n
    return g / n - np.sign(x) * np.abs(x) ** (p - 1) * (proj / (n ** (p - 1) * n))
