"""CPU oracle for the element-wise activations, forward + backward (TEST INFRASTRUCTURE ONLY).

Float64 numpy restatement of the reference's ``TritonHub/Activations`` element-wise kernels; imported by
``tests/`` only.  ``fwd(name, x, p0, p1)`` / ``bwd(name, saved, dy, p0, p1)``; ``saved`` is what the reference's
autograd Function saves -- the input, or the OUTPUT for sigmoid and tanh.

* gelu        gelu.py:28 / :77-80      0.5*x*(1 + erf(x/sqrt 2));  dy*(cdf + x*pdf)
* gelu_tanh   gelu.py:23-26 / :71-75   0.5*x*(1 + tanh(sqrt(2/pi)*(x + 0.044715 x^3)));  dy*0.5*(1 + t + x*(1 - t^2)*g'(x))
* silu        silu.py:19 / :56-57      x*sigmoid(x);  dy*(s*(1 + x*(1 - s)))
* relu        relu.py:19 / :56         x > 0 ? x : 0;  x > 0 ? dy : 0
* leaky_relu  leaky_relu.py:20 / :59   x > 0 ? x : p0*x;  x > 0 ? dy : p0*dy
* relu6       relu6.py:19-20 / :57-58  min(relu(x), 6);  (x > 0 and x < 6) ? dy : 0
* sigmoid     sigmoid.py:19 / :56      1/(1 + exp(-x));  dy*y*(1 - y)            (from the saved OUTPUT y)
* tanh        tanh.py:19-21 / :58      (e^x - e^-x)/(e^x + e^-x);  dy*(1 - y*y)  (from the saved OUTPUT y)
* mish        mish.py:19-23 / :60-66   x*tanh(sp), sp = x > 20 ? x : log(1 + exp(x));  dy*(t + x*(1 - t^2)*sigmoid(x))
* softplus    softplus.py:21 / :62     x*p0 > p1 ? x : log(1 + exp(p0*x))/p0;  x*p0 > p1 ? dy : dy/(1 + exp(-p0*x))
* threshold   threshold.py:20 / :59    x > p0 ? x : p1;  x > p0 ? dy : 0

tanh is evaluated with numpy's tanh: the reference's quotient of exponentials is the same function and differs only
where it overflows to NaN (|x| > 88 in float32).

Pinned in tests/test_act_oracle_pins.py against torch's float64 CPU functional ops and autograd (live and frozen in
tests/golden/act_golden.npz), finite differences and closed forms.
"""
import numpy as np
from scipy.special import erf

NAMES = ["gelu", "gelu_tanh", "silu", "relu", "leaky_relu", "relu6", "sigmoid", "tanh", "mish", "softplus", "threshold"]
SAVES_OUTPUT = {"sigmoid", "tanh"}
K = np.sqrt(2.0 / np.pi)


def _sigmoid(x):
    with np.errstate(over="ignore"):
        return 1.0 / (1.0 + np.exp(-x))


def _mish_sp(x):
    with np.errstate(over="ignore"):
        return np.where(x > 20.0, x, np.log(1.0 + np.exp(np.minimum(x, 50.0))))


def fwd(name, x, p0=0.0, p1=0.0):
    x = np.asarray(x, dtype=np.float64)
    if name == "gelu":
        return 0.5 * x * (1.0 + erf(x / np.sqrt(2.0)))
    if name == "gelu_tanh":
        return 0.5 * x * (1.0 + np.tanh(K * (x + 0.044715 * x * x * x)))
    if name == "silu":
        return x * _sigmoid(x)
    if name == "relu":
        return np.where(x > 0, x, 0.0)
    if name == "leaky_relu":
        return np.where(x > 0, x, p0 * x)
    if name == "relu6":
        r = np.where(x > 0, x, 0.0)
        return np.where(r < 6, r, 6.0)
    if name == "sigmoid":
        return _sigmoid(x)
    if name == "tanh":
        return np.tanh(x)
    if name == "mish":
        return x * np.tanh(_mish_sp(x))
    if name == "softplus":
        with np.errstate(over="ignore"):
            return np.where(x * p0 > p1, x, np.log(1.0 + np.exp(np.minimum(p0 * x, 700.0))) / p0)
    if name == "threshold":
        return np.where(x > p0, x, p1)
    raise KeyError(name)


def bwd(name, saved, dy, p0=0.0, p1=0.0):
    s = np.asarray(saved, dtype=np.float64)
    g = np.asarray(dy, dtype=np.float64)
    if name == "gelu":
        cdf = 0.5 * (1.0 + erf(s / np.sqrt(2.0)))
        pdf = np.exp(-0.5 * s * s) / np.sqrt(2.0 * np.pi)
        return g * (cdf + s * pdf)
    if name == "gelu_tanh":
        t = np.tanh(K * (s + 0.044715 * s * s * s))
        gp = K * (1.0 + 3.0 * 0.044715 * s * s)
        return g * (0.5 * (1.0 + t + s * (1.0 - t * t) * gp))
    if name == "silu":
        sg = _sigmoid(s)
        return g * (sg * (1.0 + s * (1.0 - sg)))
    if name == "relu":
        return np.where(s > 0, g, 0.0)
    if name == "leaky_relu":
        return np.where(s > 0, g, p0 * g)
    if name == "relu6":
        return np.where(s < 6, np.where(s > 0, g, 0.0), 0.0)
    if name == "sigmoid":
        return g * (s * (1.0 - s))
    if name == "tanh":
        return g * (1.0 - s * s)
    if name == "mish":
        t = np.tanh(_mish_sp(s))
        return g * (t + s * (1.0 - t * t) * _sigmoid(s))
    if name == "softplus":
        with np.errstate(over="ignore"):
            return np.where(s * p0 > p1, g, g / (1.0 + np.exp(-p0 * s)))
    if name == "threshold":
        return np.where(s > p0, g, 0.0)
    raise KeyError(name)
