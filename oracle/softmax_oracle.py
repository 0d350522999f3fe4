"""CPU oracle for Softmax / Softmin / LogSoftmax forward + backward (TEST INFRASTRUCTURE ONLY).

Float64 numpy restatement of the reference's row-reduction activation kernels; imported by ``tests/`` only.

* ``softmax_fwd``     follows ``TritonHub/Activations/softmax.py:17-23``   (z = x - max; exp(z)/sum(exp(z)))
* ``softmax_bwd``     follows ``TritonHub/Activations/softmax.py:57-61``   (from the SAVED OUTPUT y: y*dy - y*sum(y*dy))
* ``softmin_fwd/bwd`` follow  ``TritonHub/Activations/softmin.py:103`` + ``:17-23`` / ``:57-61``: the callable
  negates its input and applies the softmax kernels; the gradient w.r.t. the callable's input carries the sign.
* ``logsoftmax_fwd``  follows ``TritonHub/Activations/logsoftmax.py:19-24`` (z - log(sum(exp(z))))
* ``logsoftmax_bwd``  follows ``TritonHub/Activations/logsoftmax.py:61-67`` (from the saved output y: dy - exp(y)*sum(dy))

For rows within the reference's 64 KiB block the kernels see the whole row; wider rows are split by the
reference into independently normalised 64 KiB chunks (softmax.py:34-36), which is not a softmax of the row.
This oracle and the product do not imitate that: both compute ONE softmax over the whole row, whatever its
width, so for rows wider than 64 KiB they deliberately differ from what the reference would return.

Pinned in tests/test_softmax_oracle_pins.py against torch's float64 CPU softmax / log_softmax and autograd,
the frozen vectors in tests/golden/softmax_golden.npz, finite differences, closed forms and invariants.
"""
import numpy as np


def _rows(a):
    a = np.asarray(a, dtype=np.float64)
    return a, a.reshape(-1, a.shape[-1])


def softmax_fwd(x):
    x, x2 = _rows(x)
    z = x2 - x2.max(axis=1, keepdims=True)
    num = np.exp(z)
    return (num / num.sum(axis=1, keepdims=True)).reshape(x.shape)


def softmax_bwd(y, dy):
    y, y2 = _rows(y)
    _, g = _rows(dy)
    n_grad = g * y2
    return (-y2 * n_grad.sum(axis=1, keepdims=True) + n_grad).reshape(y.shape)


def softmin_fwd(x):
    return softmax_fwd(-np.asarray(x, dtype=np.float64))


def softmin_bwd(y, dy):
    """Gradient w.r.t. x of softmax(-x), from the saved output y."""
    return -softmax_bwd(y, dy)


def logsoftmax_fwd(x):
    x, x2 = _rows(x)
    z = x2 - x2.max(axis=1, keepdims=True)
    return (z - np.log(np.exp(z).sum(axis=1, keepdims=True))).reshape(x.shape)


def logsoftmax_bwd(y, dy):
    y, y2 = _rows(y)
    _, g = _rows(dy)
    return (g - np.exp(y2) * g.sum(axis=1, keepdims=True)).reshape(y.shape)


FWD = {"softmax": softmax_fwd, "softmin": softmin_fwd, "logsoftmax": logsoftmax_fwd}
BWD = {"softmax": softmax_bwd, "softmin": softmin_bwd, "logsoftmax": logsoftmax_bwd}
