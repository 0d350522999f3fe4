"""Property tests (CPU) of the host-side flattening the launch wrappers do before they hand pointers and strides
to the C ABI: whatever view comes in, (tensor, M, N, row stride) must describe exactly the rows of the view."""
import torch
from hypothesis import given, settings
from hypothesis import strategies as st

from TritonHub.Activations._launch import _flatten as act_flatten
from TritonHub.Normalization._launch import _flatten as norm_flatten
from TritonHub.Ops._launch import _rows3d


@st.composite
def views(draw):
    ndim = draw(st.integers(1, 4))
    shape = [draw(st.integers(1, 5)) for _ in range(ndim)]
    base = torch.arange(1, 1 + int(torch.tensor(shape).prod()) * 4, dtype=torch.float32)
    t = base[: int(torch.tensor(shape).prod())].reshape(shape).clone()
    ops = draw(st.lists(st.sampled_from(["slice_last", "slice_first", "step_first", "transpose", "expand", "unsqueeze"]), max_size=3))
    for op in ops:
        if op == "slice_last" and t.shape[-1] > 1:
            lo = draw(st.integers(0, t.shape[-1] - 1))
            t = t[..., lo:]
        elif op == "slice_first" and t.shape[0] > 1:
            t = t[1:]
        elif op == "step_first" and t.shape[0] > 2:
            t = t[::2]
        elif op == "transpose" and t.dim() >= 2:
            t = t.transpose(-1, -2)
        elif op == "expand" and t.dim() >= 2 and t.shape[0] == 1:
            t = t.expand(3, *t.shape[1:])
        elif op == "unsqueeze":
            t = t.unsqueeze(0)
    return t


def rows_described(t2, m, n, stride):
    """The (m, n) matrix that a kernel would read from t2's storage with that row stride."""
    return torch.as_strided(t2, (m, n), (stride, 1), t2.storage_offset())


@settings(max_examples=200, deadline=None)
@given(views())
def test_flatten_describes_the_rows_of_the_view(t):
    expect = t.reshape(-1, t.shape[-1])
    for flatten in (lambda v: norm_flatten(v, "input"), act_flatten):
        t2, m, n, stride, reshaped = flatten(t)
        assert (m, n) == tuple(expect.shape) and (t2.stride(-1) == 1 or n == 1)     # a size-1 dimension has no stride
        assert stride >= n or m <= 1                      # rows never overlap
        assert torch.equal(rows_described(t2, m, n, stride), expect)
        if not reshaped:
            assert t2 is t and t.is_contiguous()           # passed through untouched: outputs can take its shape


@settings(max_examples=100, deadline=None)
@given(views())
def test_rows3d_keeps_values_and_gives_addressable_rows(t):
    if t.dim() != 3:
        t = t.reshape(1, -1, t.shape[-1]) if t.dim() != 3 else t
    r = _rows3d(t)
    assert torch.equal(r, t) and (r.stride(-1) == 1 or r.shape[2] == 1)
    assert r.shape[1] == 1 or r.stride(1) >= r.shape[2]
