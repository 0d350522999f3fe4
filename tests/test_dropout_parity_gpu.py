"""GPU parity tests of Dropout: the HIP path, called through the module and the C ABI, against the CPU oracle on the
same inputs and seeds.  The bar is bit-exactness in every storage type: the mask is an integer computation (Philox),
and the kept values are one correctly rounded division (float32, or float64 for float64 storage) and one rounding to
the storage type, which numpy reproduces exactly."""
import ctypes
import random

import numpy as np
import pytest
import torch

from oracle import dropout_oracle as do
from TritonHub import _native
from TritonHub.Layers import Dropout
from TritonHub.Layers.dropout import dropout

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16, torch.float16, torch.float64]


def announce(msg):
    print(f"\n[case] {msg}", flush=True)


def expected(x_cpu, p, seed, first_offset=0):
    """The oracle's result in the storage type of x (torch CPU tensor)."""
    dtype = x_cpu.dtype
    if dtype == torch.float64:
        return torch.from_numpy(do.dropout(x_cpu.numpy(), p, seed, first_offset))
    y32 = do.dropout(x_cpu.float().numpy(), p, seed, first_offset)
    return torch.from_numpy(y32).to(dtype)              # round to nearest even, as the store does


def same_bits(a, b):
    if a.dtype in (torch.bfloat16, torch.float16):
        return torch.equal(a.view(torch.int16), b.view(torch.int16))
    return torch.equal(a.view(torch.int32 if a.dtype == torch.float32 else torch.int64),
                       b.view(torch.int32 if b.dtype == torch.float32 else torch.int64))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("p", [0.1, 0.5, 0.73])
def test_module_forward_and_backward_are_bit_exact(p, dtype):
    announce(f"dropout module p={p} {dtype}")
    g = torch.Generator().manual_seed(11)
    x = (torch.randn(3, 37, 129, generator=g) * 3).to(dtype)
    dy = torch.randn(3, 37, 129, generator=g).to(dtype)
    mod = Dropout(p)
    random.seed(1234)
    seed = random.randint(0, 2 ** 16)                   # what the forward below will draw (dropout.py:98)
    random.seed(1234)
    xg = x.cuda().requires_grad_(True)
    y = mod(xg)
    y.backward(dy.cuda())
    assert y.shape == x.shape and y.dtype == dtype and xg.grad.shape == x.shape and xg.grad.dtype == dtype
    assert same_bits(y.detach().cpu(), expected(x, p, seed)), "forward"
    assert same_bits(xg.grad.cpu(), expected(dy, p, seed)), "backward"
    dropped = (y.detach().cpu() == 0) & (x != 0)
    assert abs(float(dropped.float().mean()) - p) < 5 * (p * (1 - p) / x.numel()) ** 0.5


def test_seeding_python_random_reproduces_the_masks():
    announce("dropout seeding")
    x = torch.ones(64, 512, device="cuda")
    mod = Dropout(0.3)
    random.seed(99)
    a, b = mod(x), mod(x)
    random.seed(99)
    a2, b2 = mod(x), mod(x)
    assert torch.equal(a, a2) and torch.equal(b, b2) and not torch.equal(a, b)      # one draw per call


def test_shortcuts_eval_p0_p1_and_empty():
    # dropout.py:29-32: p == 0 or eval mode hand the input back, p == 1 gives zeros
    announce("dropout shortcuts")
    x = torch.randn(5, 40, device="cuda", requires_grad=True)
    mod = Dropout(0.5).eval()
    y = mod(x)
    assert torch.equal(y, x)
    y.sum().backward()
    assert torch.equal(x.grad, torch.ones_like(x))
    assert torch.equal(Dropout(0.0)(x), x)
    z = Dropout(1.0)(x)
    assert torch.equal(z, torch.zeros_like(x))
    e = torch.empty(0, 7, device="cuda", requires_grad=True)
    out = Dropout(0.5)(e)
    out.sum().backward()
    assert out.shape == (0, 7) and e.grad.shape == (0, 7)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_views_strides_and_misaligned_pointers(dtype):
    announce(f"dropout views {dtype}")
    g = torch.Generator().manual_seed(5)
    base = torch.randn(40, 300, generator=g).to(dtype)
    bg = base.cuda()
    for i, view in enumerate((lambda t: t[:, 1:], lambda t: t[3:], lambda t: t.t(), lambda t: t[::2, 5:77],
                              lambda t: t.reshape(-1)[3:4003], lambda t: t[7, 1:2])):
        random.seed(i)
        seed = random.randint(0, 2 ** 16)
        random.seed(i)
        xv = view(base)
        y = Dropout(0.4)(view(bg))
        # the reference flattens after making the last dimension contiguous: element order of the contiguous copy
        assert y.shape == xv.shape and y.is_contiguous()
        assert same_bits(y.cpu(), expected(xv.contiguous(), 0.4, seed)), f"view {i}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_c_abi_direct_in_place_offsets_and_tails(dtype):
    announce(f"dropout C ABI {dtype}")
    lib = _native.lib()
    st = torch.cuda.current_stream().cuda_stream
    code = _native.dtype_code(dtype)
    g = torch.Generator().manual_seed(21)
    for n in (1, 3, 17, 1000, 4099, 65536 + 5):
        x = (torch.randn(n, generator=g) * 2).to(dtype)
        xg = x.cuda()
        out = torch.empty_like(xg)
        for seed, first in ((0, 0), (65536, 0), (12345, 10 ** 6 + 1), (7, 2 ** 32 - 3), (2 ** 40 + 3, 2 ** 33 + 17)):
            assert lib.thn_dropout(xg.data_ptr(), out.data_ptr(), n, first, 0.25, seed, code, st) == 0
            torch.cuda.synchronize()
            assert same_bits(out.cpu(), expected(x, 0.25, seed, first)), f"n={n} seed={seed} first={first}"
        # in place, and split into two calls that carry their positions
        inplace = xg.clone()
        assert lib.thn_dropout(inplace.data_ptr(), inplace.data_ptr(), n, 0, 0.25, 12345, code, st) == 0
        half = n // 2
        parts = torch.empty_like(xg)
        size = x.element_size()
        assert lib.thn_dropout(xg.data_ptr(), parts.data_ptr(), half, 0, 0.25, 12345, code, st) == 0
        assert lib.thn_dropout(xg.data_ptr() + half * size, parts.data_ptr() + half * size, n - half, half, 0.25, 12345,
                               code, st) == 0
        torch.cuda.synchronize()
        whole = expected(x, 0.25, 12345)
        assert same_bits(inplace.cpu(), whole) and same_bits(parts.cpu(), whole), f"n={n}"


def test_non_finite_inputs_and_extreme_p():
    announce("dropout non-finite")
    lib = _native.lib()
    st = torch.cuda.current_stream().cuda_stream
    x = torch.tensor([float("nan"), float("inf"), -float("inf"), 0.0, -0.0, 1e38, 1e-45] * 64)
    xg = x.cuda()
    out = torch.empty_like(xg)
    for p in (0.0, 1e-9, 0.5, 1.0 - 2.0 ** -24, 1.0):
        assert lib.thn_dropout(xg.data_ptr(), out.data_ptr(), x.numel(), 0, p, 77, _native.F32, st) == 0
        torch.cuda.synchronize()
        with np.errstate(all="ignore"):
            ref = expected(x, p, 77)
        got = out.cpu()
        assert torch.equal(torch.isnan(got), torch.isnan(ref))
        assert same_bits(torch.nan_to_num(got, nan=0.0), torch.nan_to_num(ref, nan=0.0)), f"p={p}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_properties_at_large_size(dtype):
    """16384 x 4096: the keep rate, the scale of the kept values, determinism, and agreement of forward and backward
    masks; a sample of rows against the oracle."""
    announce(f"dropout large {dtype}")
    m, n, p = 16384, 4096, 0.1
    x = torch.randn(m, n, device="cuda").to(dtype)
    x = torch.where(x == 0, torch.ones_like(x), x)
    mod = Dropout(p)
    random.seed(8)
    seed = random.randint(0, 2 ** 16)
    random.seed(8)
    xg = x.clone().requires_grad_(True)
    y = mod(xg)
    y.backward(torch.ones_like(y))
    kept = y != 0
    rate = 1.0 - float(kept.float().mean())
    assert abs(rate - p) < 5 * (p * (1 - p) / (m * n)) ** 0.5, rate
    assert torch.equal(xg.grad != 0, kept)                           # the backward regenerates the same mask
    scale = float(torch.tensor(1.0) / (torch.tensor(1.0) - torch.tensor(p)))
    assert torch.equal(xg.grad[kept], torch.full_like(xg.grad[kept], scale))
    random.seed(8)
    assert torch.equal(mod(x), y)
    rows = [0, 1, 4097, m - 1]
    for r in rows:
        ref = expected(x[r].cpu(), p, seed, first_offset=r * n)
        assert same_bits(y[r].detach().cpu(), ref), f"row {r}"


def test_random_sizes_offsets_seeds_and_alignments():
    """150 seeded random calls through the C ABI: sizes from 1 to 70000 elements, input and output views that start
    0-7 elements into their buffers, offsets up to 2^40, seeds up to 2^63, p over (0, 1)."""
    announce("dropout random C ABI calls")
    lib = _native.lib()
    st = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(2024)
    for case in range(150):
        dtype = DTYPES[int(rng.integers(len(DTYPES)))]
        n = int(np.exp(rng.uniform(0, np.log(70000))))
        skew_in, skew_out = int(rng.integers(0, 8)), int(rng.integers(0, 8))
        first = int(rng.integers(0, 2 ** 40)) if rng.random() < 0.5 else int(rng.integers(0, 2 ** 20))
        seed = int(rng.integers(0, 2 ** 63)) if rng.random() < 0.3 else int(rng.integers(0, 2 ** 16 + 1))
        p = float(rng.uniform(0.01, 0.99))
        x = torch.from_numpy(rng.standard_normal(n + skew_in).astype(np.float32)).to(dtype)
        xg = x.cuda()
        buf = torch.full((n + skew_out + 8,), 7.0, device="cuda", dtype=dtype)
        size = x.element_size()
        rc = lib.thn_dropout(xg.data_ptr() + skew_in * size, buf.data_ptr() + skew_out * size, n, first, p, seed,
                             _native.dtype_code(dtype), st)
        assert rc == 0, (case, rc)
        torch.cuda.synchronize()
        got = buf.cpu()
        what = f"case {case}: {dtype} n={n} skew=({skew_in},{skew_out}) first={first} seed={seed} p={p:.3f}"
        assert same_bits(got[skew_out:skew_out + n].contiguous(), expected(x[skew_in:].contiguous(), p, seed, first)), what
        assert bool((got[:skew_out] == 7).all()) and bool((got[skew_out + n:] == 7).all()), what + " (wrote outside)"
