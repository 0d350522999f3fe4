"""GPU tests of the stream contract of the C ABI: every kernel is enqueued on the stream it is given, nothing
synchronises, allocates or touches another stream -- so the calls can run on a side stream and can be captured
into a HIP graph and replayed."""
import ctypes

import pytest
import torch

from TritonHub import _native
from TritonHub.Activations import GeLU, Softmax
from TritonHub.Normalization import LayerNorm, RMSNorm
from TritonHub.Ops import normalize

pytestmark = pytest.mark.gpu


def announce(msg):
    print(f"\n[case] {msg}", flush=True)


def test_operators_on_a_side_stream():
    """The operator layer launches on torch's CURRENT stream: results computed on a side stream equal those of the
    default stream, and the side stream's work is ordered after the producer it waited on."""
    announce("side stream")
    torch.manual_seed(0)
    x = torch.randn(512, 1024, device="cuda")
    dy = torch.randn(512, 1024, device="cuda")
    mods = [LayerNorm(1024, device="cuda"), RMSNorm(1024, device="cuda"), Softmax(), GeLU("tanh")]
    expected = []
    for mod in mods:
        a = x.clone().requires_grad_(True)
        y = mod(a); y.backward(dy)
        expected.append((y.detach().clone(), a.grad.clone()))
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    got = []
    with torch.cuda.stream(side):
        big = torch.randn(4096, 8192, device="cuda")
        for _ in range(3):
            big = big * 1.0001                      # keeps the side stream busy: the launches below must queue behind it
        for mod in mods:
            a = x.clone().requires_grad_(True)
            y = mod(a); y.backward(dy)
            got.append((y.detach(), a.grad))
    side.synchronize()
    for (ye, ge), (yg, gg) in zip(expected, got):
        assert torch.equal(ye, yg) and torch.equal(ge, gg)
    x3 = x.reshape(4, 128, 1024).clone().requires_grad_(True)
    with torch.cuda.stream(side):
        side.wait_stream(torch.cuda.current_stream())
        y = normalize()(x3); y.backward(dy.reshape(4, 128, 1024))
    side.synchronize()
    ref = torch.nn.functional.normalize(x.reshape(4, 128, 1024), dim=-1, eps=1e-6)
    assert torch.allclose(y, ref, atol=1e-6)


def test_c_abi_calls_replay_from_a_hip_graph():
    """Forward + backward of RMSNorm, softmax and an activation captured into one graph through the C ABI (no
    allocation, no synchronisation inside the library), replayed three times on changing inputs with eager work
    and synchronisations in between; every replay must equal the eager result bit for bit."""
    announce("graph capture")
    lib = _native.lib()
    m, n = 2048, 1024
    code = _native.BF16
    dt = torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(m, n, device="cuda", generator=g).to(dt); dy = torch.randn(m, n, device="cuda", generator=g).to(dt)
    w = (1 + 0.1 * torch.randn(n, device="cuda", generator=g)).to(dt)
    y = torch.empty_like(x); dx = torch.empty_like(x); dw = torch.empty_like(w); rstd = torch.empty(m, device="cuda")
    sm = torch.empty_like(x); dsm = torch.empty_like(x); act = torch.empty_like(x); dact = torch.empty_like(x)
    nbytes = lib.thn_norm_bwd_workspace_bytes(m, n, 1, 0, code)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    p = _native.ptr

    def enqueue(st):
        assert lib.thn_norm_fwd(p(x), n, p(y), n, p(w), 0, 0, p(rstd), m, n, 1e-6, code, code, st) == 0
        assert lib.thn_norm_bwd(p(x), n, p(dy), n, p(dx), n, p(w), 0, p(rstd), p(dw), 0, p(ws), nbytes, m, n, code, code, st) == 0
        assert lib.thn_softmax_fwd(p(y), n, p(sm), n, m, n, _native.SOFTMAX, code, st) == 0
        assert lib.thn_softmax_bwd(p(sm), n, p(dy), n, p(dsm), n, m, n, _native.SOFTMAX, code, st) == 0
        assert lib.thn_act_fwd(p(y), n, p(act), n, m, n, _native.ACT_SILU, 0.0, 0.0, code, st) == 0
        assert lib.thn_act_bwd(p(y), n, p(dy), n, p(dact), n, m, n, _native.ACT_SILU, 0.0, 0.0, code, st) == 0

    outputs = (y, dx, dw, rstd, sm, dsm, act, dact)
    enqueue(torch.cuda.current_stream().cuda_stream)          # eager warm-up (fills the library's occupancy cache)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue(torch.cuda.current_stream().cuda_stream)       # the capture stream
    for trial in range(3):
        x.copy_(torch.randn(m, n, device="cuda", generator=g).to(dt))
        dy.copy_(torch.randn(m, n, device="cuda", generator=g).to(dt))
        enqueue(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        eager = [t.clone() for t in outputs]
        for t in outputs:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, e, t in zip("y dx dw rstd sm dsm act dact".split(), eager, outputs):
            assert torch.equal(e, t), f"replay {trial}: {name} differs from the eager result"


def test_operators_from_several_host_threads():
    """Four host threads, each on a stream of its own, run different row widths through the operator layer at the same
    time (the library's launch-plan and occupancy caches and the per-stream workspaces are shared state): every
    thread's results equal the ones computed alone beforehand."""
    import threading
    announce("host threads")
    torch.manual_seed(1)
    widths = [384, 1024, 4096, 6000]
    inputs, expected = [], []
    for n in widths:
        x = torch.randn(257, n, device="cuda", dtype=torch.bfloat16)
        dy = torch.randn(257, n, device="cuda", dtype=torch.bfloat16)
        mods = [LayerNorm(n, device="cuda", dtype=torch.bfloat16), RMSNorm(n, device="cuda", dtype=torch.bfloat16), Softmax()]
        outs = []
        for mod in mods:
            a = x.clone().requires_grad_(True)
            y = mod(a); y.backward(dy)
            outs.append((y.detach().clone(), a.grad.clone()))
        inputs.append((x, dy, mods))
        expected.append(outs)
    torch.cuda.synchronize()
    errors = []

    def work(i):
        try:
            x, dy, mods = inputs[i]
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for rep in range(20):
                    for mod, (ye, ge) in zip(mods, expected[i]):
                        a = x.clone().requires_grad_(True)
                        y = mod(a); y.backward(dy)
                        stream.synchronize()
                        if not (torch.equal(y.detach(), ye) and torch.equal(a.grad, ge)):
                            errors.append((i, rep, type(mod).__name__))
        except Exception as e:                      # surface the failure in the main thread
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(widths))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
    assert not any(t.is_alive() for t in threads), "a worker thread did not finish"
    assert not errors, errors[:5]


def test_two_host_threads_feed_one_stream():
    """Two host threads run backward passes of different layers on the SAME stream (the autograd engine's worker and
    a user thread can): the shared per-stream workspace of the two-stage dW / dB sum must never see one call's
    first stage, the other call's first stage, then a second stage.  Parameter gradients equal the ones computed
    alone beforehand, bit for bit, on every repetition."""
    import threading
    announce("two host threads, one stream")
    torch.manual_seed(3)
    stream = torch.cuda.Stream()
    cases = []
    for n, rows in ((1024, 4096), (1536, 3000)):
        x = torch.randn(rows, n, device="cuda", dtype=torch.bfloat16)
        dy = torch.randn(rows, n, device="cuda", dtype=torch.bfloat16)
        mod = LayerNorm(n, device="cuda", dtype=torch.bfloat16)
        a = x.clone().requires_grad_(True)
        mod(a).backward(dy)
        cases.append((x, dy, mod, mod.weight.grad.clone(), mod.bias.grad.clone(), a.grad.clone()))
    torch.cuda.synchronize()
    errors = []

    def work(i):
        try:
            x, dy, mod, dw, db, dx = cases[i]
            with torch.cuda.stream(stream):
                for rep in range(200):
                    a = x.clone().requires_grad_(True)
                    mod.weight.grad = None
                    mod.bias.grad = None
                    mod(a).backward(dy)
                    got = (mod.weight.grad, mod.bias.grad, a.grad)
                    if rep % 20 == 19:
                        stream.synchronize()
                        if not (torch.equal(got[0], dw) and torch.equal(got[1], db) and torch.equal(got[2], dx)):
                            errors.append((i, rep))
        except Exception as e:
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
    assert not any(t.is_alive() for t in threads), "a worker thread did not finish"
    assert not errors, errors[:5]


def test_operator_layer_backward_under_graph_capture():
    """The modules captured into a torch graph: the backward then takes a workspace of its own (the graph's) rather
    than the per-stream one it shares with eager calls, so replays interleaved with eager backward passes of another
    shape on the same stream still equal the eager result."""
    announce("operator layer under graph capture")
    torch.manual_seed(5)
    n = 2048
    mod = LayerNorm(n, device="cuda", dtype=torch.bfloat16)
    other = RMSNorm(768, device="cuda", dtype=torch.bfloat16)
    xs = torch.randn(1024, n, device="cuda", dtype=torch.bfloat16)
    dy = torch.randn(1024, n, device="cuda", dtype=torch.bfloat16)
    xo = torch.randn(5000, 768, device="cuda", dtype=torch.bfloat16)

    def eager(xin):
        a = xin.clone().requires_grad_(True)
        mod.weight.grad = None
        mod.bias.grad = None
        y = mod(a)
        y.backward(dy)
        return y.detach().clone(), a.grad.clone(), mod.weight.grad.clone(), mod.bias.grad.clone()

    eager(xs)                                            # warm-up outside the capture
    torch.cuda.synchronize()
    static_x = xs.clone().requires_grad_(True)
    mod.weight.grad = None
    mod.bias.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = mod(static_x)
        gx, gw, gb = torch.autograd.grad(y, (static_x, mod.weight, mod.bias), dy)
    for trial in range(3):
        new_x = torch.randn(1024, n, device="cuda", dtype=torch.bfloat16)
        expect = eager(new_x)
        with torch.no_grad():
            static_x.copy_(new_x)
        ao = xo.clone().requires_grad_(True)
        other(ao).backward(torch.ones_like(xo))          # eager work on the shared workspace, enqueued around the replay
        graph.replay()
        other(ao).backward(torch.ones_like(xo))
        torch.cuda.synchronize()
        for name, e, t in zip(("y", "dx", "dw", "db"), expect, (y, gx, gw, gb)):
            assert torch.equal(e, t), f"replay {trial}: {name} differs from the eager result"
