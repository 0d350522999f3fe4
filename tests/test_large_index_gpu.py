"""Tensors of more than 2^31 elements: every row offset is 64-bit.  The first and the last rows of one big call must
be bit-identical to the same rows run on their own (the row arithmetic does not depend on M), and the column sums
dW / dB must agree with the sums of the same call made chunk by chunk."""
import pytest
import torch

from TritonHub.Activations import GeLU, LogSoftmax, Softmax
from TritonHub.Normalization import LayerNorm, RMSNorm
from TritonHub.Ops import norm, normalize

pytestmark = pytest.mark.gpu
ROWS, N = (1 << 20) + 3, 2056            # 2 155 878 648 elements, 4.3 GB per bfloat16 tensor
EDGE = 96


def announce(msg):
    print(f"\n[case] {msg}", flush=True)


def big(seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    t = torch.empty(ROWS, N, device="cuda", dtype=torch.bfloat16)
    for s in range(0, ROWS, 1 << 17):                     # in pieces: no float32 temporary of the whole size
        t[s:s + (1 << 17)] = torch.randn(min(1 << 17, ROWS - s), N, device="cuda", generator=g).bfloat16()
    return t


def edges(t):
    return torch.cat([t[:EDGE], t[-EDGE:]])


@pytest.mark.parametrize("kind", ["ln", "rms"])
def test_norm_rows_beyond_2_31_elements(kind):
    announce(f"large index {kind}")
    assert ROWS * N > 2 ** 31
    make = (lambda: LayerNorm(N, device="cuda", dtype=torch.bfloat16)) if kind == "ln" else \
        (lambda: RMSNorm(N, device="cuda", dtype=torch.bfloat16))
    mod = make()
    with torch.no_grad():
        mod.weight.copy_(1 + 0.1 * torch.randn(N, device="cuda"))
    x = big(1).requires_grad_(True)
    dy = big(2)
    y = mod(x)
    y.backward(dy)
    small = make()
    small.load_state_dict(mod.state_dict())
    xe = edges(x.detach()).requires_grad_(True)
    ye = small(xe)
    ye.backward(edges(dy))
    assert torch.equal(edges(y.detach()), ye.detach()) and torch.equal(edges(x.grad), xe.grad)
    dw = torch.zeros(N, device="cuda")
    db = torch.zeros(N, device="cuda")
    step = 1 << 16
    for s in range(0, ROWS, step):
        part = make()
        part.load_state_dict(mod.state_dict())
        part = part.float()                               # float32 parameters: float32 partial sums
        xs = x.detach()[s:s + step].requires_grad_(True)
        part(xs).backward(dy[s:s + step])
        dw += part.weight.grad
        if kind == "ln":
            db += part.bias.grad
    got = mod.weight.grad.float()
    assert bool(((got - dw).abs() <= 2.0 ** -7 * dw.abs() + 0.05).all()), float((got - dw).abs().max())
    if kind == "ln":
        got = mod.bias.grad.float()
        assert bool(((got - db).abs() <= 2.0 ** -7 * db.abs() + 0.05).all()), float((got - db).abs().max())


@pytest.mark.parametrize("name", ["softmax", "logsoftmax", "gelu", "normalize", "norm"])
def test_row_operators_beyond_2_31_elements(name):
    announce(f"large index {name}")
    op = {"softmax": Softmax, "logsoftmax": LogSoftmax, "gelu": GeLU, "normalize": normalize, "norm": norm}[name]()
    x = big(3)
    three_d = name in ("normalize", "norm")
    xv = (x.view(1, ROWS, N) if three_d else x).requires_grad_(True)
    y = op(xv)
    dy = torch.ones_like(y) if name == "norm" else big(4).view_as(y)
    y.backward(dy)
    xe = edges(x.detach())
    xev = (xe.view(1, 2 * EDGE, N) if three_d else xe).requires_grad_(True)
    ye = op(xev)
    if name == "norm":
        dye = torch.ones_like(ye)
        ysel = torch.cat([y.detach()[0, :EDGE], y.detach()[0, -EDGE:]])
        assert torch.equal(ysel, ye.detach()[0])
    else:
        dye = edges(dy.view(ROWS, N)).view_as(ye)
        assert torch.equal(edges(y.detach().view(ROWS, N)), ye.detach().view(2 * EDGE, N))
    ye.backward(dye)
    assert torch.equal(edges(xv.grad.view(ROWS, N)), xev.grad.view(2 * EDGE, N))


def test_dropout_beyond_2_31_elements():
    """Element offsets of 2^31 and more: the Philox counter takes the offset as an unsigned 32-bit word (and a high
    word from 2^32 on); the last rows are compared with the oracle at their true offsets."""
    import random
    from oracle import dropout_oracle as do
    from TritonHub.Layers import Dropout
    announce("large index dropout")
    x = big(5)
    random.seed(3)
    seed = random.randint(0, 2 ** 16)
    random.seed(3)
    y = Dropout(0.25)(x)
    for r in (0, (1 << 31) // N, (1 << 31) // N + 1, ROWS - 1):
        ref = do.dropout(x[r].float().cpu().numpy(), 0.25, seed, first_offset=r * N)
        assert torch.equal(y[r].cpu(), torch.from_numpy(ref).bfloat16()), f"row {r}"
    rate = float((y == 0).float().mean())
    assert abs(rate - 0.25) < 1e-3
