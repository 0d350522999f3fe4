#!/usr/bin/env python3
"""Benchmark of the LayerNorm / RMSNorm (and Softmax-family) forward + backward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

One step = one forward (`thn_norm_fwd`) plus one backward (`thn_norm_bwd`: the dx / partial-sum kernel and
the second-stage dW / dB reduction) over one batch of synthetic input that is already resident in HBM,
called through the C ABI exactly as the Python operator layer calls it.  The backward of a step works on the
batch its forward has just processed, as a training step does; the line also carries the step with the backward
on a batch whose forward ran two steps earlier (`no_reuse`), each kernel's duration inside the step and on its own,
and -- on the default workload -- the LayerNorm step of the same shape (`layernorm_same_shape`).  The default workload is the one the
headline metric is quoted on: RMSNorm, bfloat16, 16384 rows x 4096, weight = 1 + N(0, 0.1), eps = 1e-6.
Four independent buffer sets (x, dy, y, dx) are rotated so that no step re-reads what the previous one left
in the caches.  Prints ONE JSON line.

`value` is algorithmic bytes per step / time per step: 5*M*N*s + 8*M + 3*N*s_w bytes for RMSNorm,
5*M*N*s + 16*M + 5*N*s_w for LayerNorm (x read by forward and again by backward, dy read, y and dx written,
float32 row statistics written then read, parameters read, parameter gradients written; the partial-sum
workspace is overhead and is not counted).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "triton-hub_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X published peak
N_BUFFER_SETS = 4

WORKLOADS = {
    # name: (kind, rows, hidden, dtype name)
    "rmsnorm_bf16_16384x4096": ("rms", 16384, 4096, "bf16"),
    "layernorm_bf16_16384x4096": ("ln", 16384, 4096, "bf16"),
    "layernorm_bf16_32768x8192": ("ln", 32768, 8192, "bf16"),
    "layernorm_f32_1048576x256": ("ln", 1048576, 256, "f32"),
    "layernorm_f16_8192x6000_hostile": ("ln", 8192, 6000, "f16"),
    "layernorm_f32_8192x6000_hostile": ("ln", 8192, 6000, "f32"),
    "rmsnorm_f16_4096x16384_outliers": ("rms", 4096, 16384, "f16"),
    "rmsnorm_f32_4096x16384_outliers": ("rms", 4096, 16384, "f32"),
    "layernorm_f32_200x128_quickstart": ("ln", 200, 128, "f32"),
    # rows of 64 KiB (the 1024-thread workgroups) and rows that are not a whole number of 16-byte vectors
    "layernorm_bf16_4096x32768_wide": ("ln", 4096, 32768, "bf16"),
    "rmsnorm_bf16_4096x32768_wide": ("rms", 4096, 32768, "bf16"),
    "layernorm_f32_4096x16384_wide": ("ln", 4096, 16384, "f32"),
    "layernorm_f32_12279x4099_ragged": ("ln", 12279, 4099, "f32"),
    "rmsnorm_bf16_24564x4098_ragged": ("rms", 24564, 4098, "bf16"),
    # narrow rows, 2^26 elements: 9 vectors per 16-bit row (RMSNorm: the flat kernels) and 7 per float32 row (the staged kernels)
    "rmsnorm_bf16_932067x72_narrow": ("rms", 932067, 72, "bf16"),
    "layernorm_bf16_932067x72_narrow": ("ln", 932067, 72, "bf16"),
    "layernorm_f32_2396745x28_narrow": ("ln", 2396745, 28, "f32"),
    # off the 128-bit path (50 columns: 7 unaligned windows of bfloat16, 13 of float32: the flat kernels' other instances)
    # and shorter than one vector (3 float32 columns: a lane per row)
    "rmsnorm_bf16_1342177x50_ragged": ("rms", 1342177, 50, "bf16"),
    "layernorm_f32_1342177x50_ragged": ("ln", 1342177, 50, "f32"),
    "layernorm_f32_11184810x3_short": ("ln", 11184810, 3, "f32"),
    # norm with an activation epilogue (thn_norm_act_fwd + thn_norm_act_bwd): same bytes as the plain norm step
    "layernorm_gelu_bf16_16384x4096": ("ln+gelu", 16384, 4096, "bf16"),
    "layernorm_gelu_tanh_bf16_16384x4096": ("ln+gelu_tanh", 16384, 4096, "bf16"),
    "rmsnorm_silu_bf16_16384x4096": ("rms+silu", 16384, 4096, "bf16"),
    "layernorm_gelu_f32_16384x4096": ("ln+gelu", 16384, 4096, "f32"),
    # the row-reduction activations next to the norm path (thn_softmax_fwd + thn_softmax_bwd per step)
    "softmax_bf16_16384x4096": ("softmax", 16384, 4096, "bf16"),
    "softmax_f32_16384x4096": ("softmax", 16384, 4096, "f32"),
    "softmax_f16_65536x1024": ("softmax", 65536, 1024, "f16"),
    "softmin_bf16_16384x4096": ("softmin", 16384, 4096, "bf16"),
    "logsoftmax_bf16_8192x32768": ("logsoftmax", 8192, 32768, "bf16"),
    "logsoftmax_f32_16384x4096": ("logsoftmax", 16384, 4096, "f32"),
    # narrow rows, 2^26 elements: one and nine vectors per row (the flat softmax kernels)
    "softmax_bf16_8388608x8_narrow": ("softmax", 8388608, 8, "bf16"),
    "softmax_bf16_932067x72_narrow": ("softmax", 932067, 72, "bf16"),
    # off the 128-bit path: a ViT's attention row (197 columns, 25 unaligned windows: the flat kernels' other instances)
    "softmax_bf16_340654x197_ragged": ("softmax", 340654, 197, "bf16"),
    # vocabulary-sized rows, wider than 64 KiB: the looping kernels (two walks per row)
    "logsoftmax_f32_8192x32000_vocab": ("logsoftmax", 8192, 32000, "f32"),
    "logsoftmax_bf16_4096x128256_vocab": ("logsoftmax", 4096, 128256, "bf16"),
    # row p-norm / normalize of a (1, rows, K) tensor (thn_normalize_fwd + thn_normalize_bwd, or thn_pnorm_*)
    "normalize_p2_bf16_16384x4096": ("normalize_p2", 16384, 4096, "bf16"),
    "normalize_p2_f32_16384x4096": ("normalize_p2", 16384, 4096, "f32"),
    "normalize_p2_f16_65536x1024": ("normalize_p2", 65536, 1024, "f16"),
    "normalize_p1_bf16_16384x4096": ("normalize_p1", 16384, 4096, "bf16"),
    "normalize_p3_bf16_16384x4096": ("normalize_p3", 16384, 4096, "bf16"),
    "pnorm_p2_bf16_16384x4096": ("pnorm_p2", 16384, 4096, "bf16"),
    "pnorm_p3_f32_16384x4096": ("pnorm_p3", 16384, 4096, "f32"),
    # rows of one float32 vector (quaternions) and of nine bfloat16 vectors, 2^26 elements: the flat p-norm kernels
    "normalize_p2_f32_16777216x4_narrow": ("normalize_p2", 16777216, 4, "f32"),
    "normalize_p2_bf16_932067x72_narrow": ("normalize_p2", 932067, 72, "bf16"),
    # rows shorter than one vector: 3-component float32 vectors, a lane per row
    "normalize_p2_f32_11184810x3_short": ("normalize_p2", 11184810, 3, "f32"),
    # element-wise activations (thn_act_fwd + thn_act_bwd per step)
    "act_gelu_bf16_16384x4096": ("act_gelu", 16384, 4096, "bf16"),
    "act_gelu_tanh_bf16_16384x4096": ("act_gelu_tanh", 16384, 4096, "bf16"),
    "act_gelu_f32_16384x4096": ("act_gelu", 16384, 4096, "f32"),
    "act_silu_bf16_16384x4096": ("act_silu", 16384, 4096, "bf16"),
    "act_relu_bf16_16384x4096": ("act_relu", 16384, 4096, "bf16"),
    "act_mish_bf16_16384x4096": ("act_mish", 16384, 4096, "bf16"),
    "act_softplus_f16_16384x4096": ("act_softplus", 16384, 4096, "f16"),
    "act_sigmoid_f32_16384x4096": ("act_sigmoid", 16384, 4096, "f32"),
    # Layers.Dropout (thn_dropout on x, then on dy, with the same seed)
    "dropout_bf16_16384x4096": ("dropout", 16384, 4096, "bf16"),
    "dropout_f32_16384x4096": ("dropout", 16384, 4096, "f32"),
}
ACT_NAMES = ["gelu", "gelu_tanh", "silu", "relu", "leaky_relu", "relu6", "sigmoid", "tanh", "mish", "softplus", "threshold"]
ACT_PARAMS = {"leaky_relu": (0.01, 0.0), "softplus": (1.0, 20.0), "threshold": (0.1, 20.0)}
SOFTMAX_KINDS = ("softmax", "softmin", "logsoftmax")

# HBM bytes per launch of a workload's dominant kernel: not a figure of this run (counters need rocprofv3), but the
# one the named summary under profiles/ holds, read from that file when the line is printed.  A summary carries
# it as a line
#     bench.traffic <workload> <kernel> <bytes per launch> <cache policy of the run>
# (from two rocprofv3 --pmc runs of this script, FETCH_SIZE then WRITE_SIZE, each scaled by what the same counter
# reads for a plain copy of known size); a workload without such a line reports null.
PROFILES_DIR = os.path.join(ROOT, "profiles")


def traffic_from_profiles(workload):
    """{"bytes": ..., "kernel": ..., "cache_policy": ..., "source": "profiles/<file>"} or None."""
    try:
        names = sorted(os.listdir(PROFILES_DIR))
    except OSError:
        return None
    for name in names:
        if not name.endswith((".txt", ".md")):
            continue
        try:
            with open(os.path.join(PROFILES_DIR, name)) as fh:
                for line in fh:
                    parts = line.split()
                    if len(parts) >= 4 and parts[0] == "bench.traffic" and parts[1] == workload:
                        return {"bytes": int(parts[3]), "kernel": parts[2],
                                "cache_policy": parts[4] if len(parts) > 4 else None, "source": "profiles/" + name}
        except (OSError, ValueError):
            continue
    return None


# Untimed steps of the norm workloads before the W warm-up steps (see the timed region of the norm bench).
PREROLL_STEPS = 150


def traffic_fields(workload):
    """`traffic` of the roofline object and where it comes from."""
    t = traffic_from_profiles(workload)
    if t is None:
        return {"traffic": None}
    return {"traffic": t["bytes"], "traffic_source": f"{t['source']} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of {t['kernel']}, "
                                                     f"cache policy {t['cache_policy']}; not counted in this run)"}


def algorithmic_bytes(kind, m, n, s, sw):
    if kind.startswith("normalize"):          # forward: x read, y + norms written; backward: y (x for p=1; x and y for
        extra = 0 if kind[-1] in "12" else 1  # other p), dy and norms read, dx written
        return 2 * m * n * s + m * s, (3 + extra) * m * n * s + m * s
    if kind.startswith("pnorm"):              # forward: x read, norms written; backward: x, norms, dnorms read, dx written
        return m * n * s + m * s, 2 * m * n * s + 2 * m * s
    if kind in SOFTMAX_KINDS or kind.startswith("act_"):   # forward: x read, y written; backward: saved and dy read, dx written
        return 2 * m * n * s, 3 * m * n * s
    if kind == "ln":
        return 2 * m * n * s + 2 * n * sw + 8 * m, 3 * m * n * s + 3 * n * sw + 8 * m
    return 2 * m * n * s + n * sw + 4 * m, 3 * m * n * s + 2 * n * sw + 4 * m


class NormBench:
    """Buffers and launchers of one LayerNorm / RMSNorm workload, called through the C ABI."""

    def __init__(self, lib, dev, workload):
        import torch
        from TritonHub import _native
        self.torch, self.lib, self.native = torch, lib, _native
        kind, m, n, dname = WORKLOADS[workload]
        self.workload, self.fused_act = workload, -1
        self.x_flag = _native.X_KEEP          # this bench's forward calls say how they read x: see set_policy()
        if "+" in kind:
            kind, act_name = kind.split("+")
            self.fused_act = FUSED_ACTS.index(act_name)
        self.kind, self.m, self.n, self.dname = kind, m, n, dname
        self.ln = kind == "ln"
        self.dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[dname]
        self.s = torch.empty(0, dtype=self.dtype).element_size()
        self.code = _native.dtype_code(self.dtype)
        gen = torch.Generator(device=dev).manual_seed(0)

        def rand(*shape):
            return torch.randn(*shape, device=dev, generator=gen, dtype=torch.float32)

        self.sets = []
        for _ in range(N_BUFFER_SETS):
            x = rand(m, n)
            if "hostile" in workload:
                x += 1000.0
            if "outliers" in workload:
                x = torch.where(torch.rand(m, n, device=dev, generator=gen) < 0.001, x * 100.0, x)
            x = x.to(self.dtype)
            dy = rand(m, n).to(self.dtype)
            self.sets.append(dict(x=x, dy=dy, y=torch.empty_like(x), dx=torch.empty_like(x),
                                  mean=torch.empty(m, device=dev) if self.ln else None,
                                  rstd=torch.empty(m, device=dev)))
        self.w = (1.0 + 0.1 * rand(n)).to(self.dtype)
        self.b = (0.1 * rand(n)).to(self.dtype) if self.ln else None
        self.dw = torch.empty_like(self.w)
        self.db = torch.empty_like(self.w) if self.ln else None
        if self.fused_act >= 0:
            self.ws_bytes = lib.thn_norm_act_bwd_workspace_bytes(m, n, 1, int(self.ln), self.fused_act, self.code)
        else:
            self.ws_bytes = lib.thn_norm_bwd_workspace_bytes(m, n, 1, int(self.ln), self.code)
        assert self.ws_bytes >= 0, self.ws_bytes
        self.ws = torch.empty(max(self.ws_bytes, 16) // 4, device=dev)
        self.stream = torch.cuda.current_stream(dev).cuda_stream
        self.parts = ctypes.c_int32(0)
        self.fwd_bytes, self.bwd_bytes = algorithmic_bytes(kind, m, n, self.s, self.s)
        self.step_bytes = self.fwd_bytes + self.bwd_bytes

    def set_policy(self, policy):
        """'keep': the forward leaves x in the caches for the backward (THN_X_KEEP); 'stream': it does not."""
        self.x_flag = {"keep": self.native.X_KEEP, "stream": self.native.X_STREAM}[policy]

    # ---- the launches ----
    def forward(self, b_):
        p, lib, m, n, code = self.native.ptr, self.lib, self.m, self.n, self.code
        if self.fused_act >= 0:
            rc = lib.thn_norm_act_fwd(p(b_["x"]), n, p(b_["y"]), n, p(self.w), p(self.b), p(b_["mean"]), p(b_["rstd"]),
                                      m, n, 1e-6, self.fused_act, code | self.x_flag, code, self.stream)
        else:
            rc = lib.thn_norm_fwd(p(b_["x"]), n, p(b_["y"]), n, p(self.w), p(self.b), p(b_["mean"]), p(b_["rstd"]),
                                  m, n, 1e-6, code | self.x_flag, code, self.stream)
        assert rc == 0, self.native.strerror(rc)

    def backward(self, b_):
        p, lib, m, n, code = self.native.ptr, self.lib, self.m, self.n, self.code
        if self.fused_act >= 0:
            rc = lib.thn_norm_act_bwd(p(b_["x"]), n, p(b_["dy"]), n, p(b_["dx"]), n, p(self.w), p(self.b), p(b_["mean"]),
                                      p(b_["rstd"]), p(self.dw), p(self.db), p(self.ws), self.ws_bytes, m, n,
                                      self.fused_act, code, code, self.stream)
        else:
            rc = lib.thn_norm_bwd(p(b_["x"]), n, p(b_["dy"]), n, p(b_["dx"]), n, p(self.w), p(b_["mean"]), p(b_["rstd"]),
                                  p(self.dw), p(self.db), p(self.ws), self.ws_bytes, m, n, code, code, self.stream)
        assert rc == 0, self.native.strerror(rc)

    def backward_stage1(self, b_):
        """The dx / partial-sum kernel on its own (thn_norm_bwd is this plus backward_stage2, bit for bit)."""
        p, lib, m, n, code = self.native.ptr, self.lib, self.m, self.n, self.code
        rc = lib.thn_norm_bwd_dx_partials(p(b_["x"]), n, p(b_["dy"]), n, p(b_["dx"]), n, p(self.w), p(b_["mean"]),
                                          p(b_["rstd"]), 1, int(self.ln), p(self.ws), self.ws_bytes,
                                          ctypes.byref(self.parts), m, n, code, code, self.stream)
        assert rc == 0, self.native.strerror(rc)

    def backward_stage2(self):
        p = self.native.ptr
        rc = self.lib.thn_norm_bwd_reduce_partials(p(self.ws), self.parts.value, p(self.dw), p(self.db), self.n,
                                                   self.code, self.stream)
        assert rc == 0, self.native.strerror(rc)

    def step(self, i, lag=0):
        """Forward on batch i, backward on batch i - lag (lag = 0: the backward of the batch just forwarded)."""
        self.forward(self.sets[i % N_BUFFER_SETS])
        self.backward(self.sets[(i - lag) % N_BUFFER_SETS])

    # ---- measurements ----
    def timed_steps(self, steps, warmup, lag=0, preroll=0):
        """(ms per step by the host clock between two device synchronisations, ms per step by HIP events recorded
        on the launch stream inside that bracket).  The host clock starts after a device synchronisation and stops
        when the event behind the last step has completed (polled, then the device is synchronised again): it still
        carries the launch latency of the first step, a fraction of a percent of a step at K = 20."""
        torch = self.torch
        for i in range(preroll + warmup):
            self.step(i, lag)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()                   # torch creates an event at its first record(): not inside the bracket
        stop.record()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        start.record()
        for i in range(steps):
            self.step(i, lag)
        stop.record()
        while not stop.query():          # busy-wait for the last step: a blocking wait wakes up tens of microseconds late
            pass
        host_ms = (time.perf_counter() - t0) * 1e3 / steps
        torch.cuda.synchronize()
        return host_ms, start.elapsed_time(stop) / steps

    def kernels_in_step(self, steps, lag=0):
        """Average duration of each of the three kernels as they run inside the step: the same K steps once more,
        with HIP events on the launch stream between the kernels (forward | dx + partial sums | second stage).  The
        events cost the step about a microsecond each, which is why the step itself is timed without them."""
        torch = self.torch
        if self.fused_act >= 0:
            return None                       # the fused backward has no separate stage entry points
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(steps)]
        for i in range(3):
            self.step(i, lag)
        torch.cuda.synchronize()
        for i in range(steps):
            e = ev[i]
            e[0].record()
            self.forward(self.sets[i % N_BUFFER_SETS])
            e[1].record()
            self.backward_stage1(self.sets[(i - lag) % N_BUFFER_SETS])
            e[2].record()
            self.backward_stage2()
            e[3].record()
        torch.cuda.synchronize()
        out = []
        for k in range(3):
            out.append(sum(e[k].elapsed_time(e[k + 1]) for e in ev) * 1e3 / steps)
        return out

    def isolated_launch_us(self, launch, steps, warmup):
        """K back-to-back launches of ONE kernel between one pair of events, rotating the batches: the kernel
        with nothing of its operands left in the caches by a neighbour."""
        torch = self.torch
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(min(warmup, 5)):
            launch(self.sets[i % N_BUFFER_SETS])
        torch.cuda.synchronize()
        start.record()
        for i in range(steps):
            launch(self.sets[i % N_BUFFER_SETS])
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) * 1e3 / steps

    def shapes(self):
        from TritonHub.Normalization import _launch
        flavour = int(self.ln) | (self.fused_act << 1) if self.fused_act >= 0 else int(self.ln)
        f = _launch.query_launch(9 if self.fused_act >= 0 else 0, flavour, self.m, self.n, self.dtype)
        b = _launch.query_launch(10 if self.fused_act >= 0 else 1, flavour, self.m, self.n, self.dtype)
        return ({"vecs_per_thread": f[0], "threads_per_row": f[1], "block": f[2], "grid": f[3]},
                {"vecs_per_thread": b[0], "threads_per_row": b[1], "block": b[2], "grid": b[3]})

    def free(self):
        self.sets = None
        self.torch.cuda.empty_cache()


FUSED_ACTS = ["gelu", "gelu_tanh", "silu", "relu"]
STEP_NOTE = ("one step = forward and backward of the SAME batch, back to back, the forward under the 'keep' cache policy "
             "(THN_X_KEEP: x is loaded with cache-allocating loads, everything else streams): the backward re-reads the x "
             "its forward has just read, and a part of it is still in the 256 MB Infinity Cache.")
NO_REUSE_NOTE = ("the same step with the backward working on the batch whose forward ran two steps earlier (four batches "
                 "in rotation: 1.3 GB of other traffic lie between the two reads of an x, nothing of a backward's operands is "
                 "left in any cache -- what a training step sees when the rest of the network runs between a layer's forward "
                 "and its backward), the forward under the 'stream' cache policy (THN_X_STREAM)")

# The other configurations of the benchmark contract, measured after the headline on the default run.
CONTRACT_CONFIGS = ["layernorm_bf16_32768x8192", "layernorm_f32_1048576x256", "layernorm_f16_8192x6000_hostile",
                    "layernorm_f32_8192x6000_hostile", "rmsnorm_f16_4096x16384_outliers", "rmsnorm_f32_4096x16384_outliers",
                    "layernorm_f32_200x128_quickstart"]


def measure_norm(bench, args, policy="keep", lag=0, preroll=PREROLL_STEPS, with_kernels=True):
    """The step of one norm workload under one cache policy; lag = 0: the backward of the batch just forwarded,
    lag = 2: of the batch forwarded two steps earlier."""
    bench.set_policy(policy)
    ms_per_step, ms_events = bench.timed_steps(args.steps, args.warmup, lag=lag, preroll=preroll)
    gbps = bench.step_bytes / (ms_per_step * 1e-3) / 1e9
    res = {"ms_per_step": round(ms_per_step, 5), "GBps": round(gbps, 1),
           "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
           "ms_per_step_by_hip_events": round(ms_events, 5),
           "pct_of_hbm_peak_by_hip_events": round(100.0 * bench.step_bytes / (ms_events * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
           "rows_per_s": round(bench.m / (ms_per_step * 1e-3))}
    if with_kernels:
        # An event between two kernels keeps the second from starting the moment the first ends: the three
        # intervals of an instrumented step add up to more than the plain step.  That surplus is the events' own
        # cost; it is taken off the three intervals in equal parts (rocprofv3's kernel durations of the same run
        # agree with the result to half a microsecond).
        k = bench.kernels_in_step(args.steps, lag)
        if k is not None:
            cost = (sum(k) - ms_per_step * 1e3) / 3.0
            res["kernels_us"] = {"forward": round(k[0] - cost, 2), "backward_dx_partials": round(k[1] - cost, 2),
                                 "backward_reduce_partials": round(k[2] - cost, 2),
                                 "event_cost_taken_off_each": round(cost, 2)}
    return res


def norm_roofline(bench, cold, warm):
    """The dominant kernel -- the backward dx / partial-sum kernel -- against the HBM roofline.  `achieved` is taken
    from the kernel on a batch that no cache holds (the no-reuse step): only then are the algorithmic bytes HBM
    bytes.  Inside the same-batch step a part of x comes from the Infinity Cache; that figure is reported beside it
    and is not an HBM fraction."""
    roofline = {"bound": "hbm", "kernel": "norm_bwd_kernel (backward dx + dW/dB partials)", "peak": HBM_PEAK_GBPS,
                "unit": "GB/s", "algorithmic_bytes_per_launch": bench.bwd_bytes, **traffic_fields(bench.workload)}
    if cold is not None and "kernels_us" in cold:
        us = cold["kernels_us"]["backward_dx_partials"]
        achieved = bench.bwd_bytes / (us * 1e-6) / 1e9
        roofline.update({"achieved": round(achieved, 1), "frac": round(achieved / HBM_PEAK_GBPS, 4), "avg_launch_us": us,
                         "measured": "HIP events on the launch stream around the kernel inside the no-reuse step (its "
                                     "operands in no cache), less the events' own cost"})
    if warm is not None and "kernels_us" in warm:
        us = warm["kernels_us"]["backward_dx_partials"]
        ach = bench.bwd_bytes / (us * 1e-6) / 1e9
        roofline["in_step_cache_assisted"] = {
            "avg_launch_us": us, "algorithmic_GBps": round(ach, 1), "frac_of_hbm_peak": round(ach / HBM_PEAK_GBPS, 4),
            "note": "inside the same-batch step part of x is served by the Infinity Cache: algorithmic bytes per second, "
                    "not HBM bytes per second"}
        if "achieved" not in roofline:
            roofline.update({"achieved": round(ach, 1), "frac": round(ach / HBM_PEAK_GBPS, 4), "avg_launch_us": us,
                             "measured": "HIP events around the kernel inside the same-batch step (cache-assisted)"})
    return roofline


def config_summary(lib, dev, workload, args):
    """One more configuration of the benchmark contract: the step as defined, the no-reuse step, the kernels."""
    bench = NormBench(lib, dev, workload)
    short = argparse.Namespace(steps=args.steps, warmup=min(args.warmup, 5))
    warm = measure_norm(bench, short, "keep", 0)
    cold = measure_norm(bench, short, "stream", 2, preroll=0)
    fwd_shape, bwd_shape = bench.shapes()
    out = {"op": "LayerNorm" if bench.ln else "RMSNorm", "rows": bench.m, "hidden": bench.n, "dtype": bench.dname,
           "algorithmic_bytes_per_step": bench.step_bytes,
           "ms_per_step": warm["ms_per_step"], "GBps": warm["GBps"], "pct_of_hbm_peak": warm["pct_of_hbm_peak"],
           "rows_per_s": warm["rows_per_s"], "kernels_us": warm.get("kernels_us"),
           "no_reuse_ms_per_step": cold["ms_per_step"], "no_reuse_pct": cold["pct_of_hbm_peak"],
           "no_reuse_kernels_us": cold.get("kernels_us"),
           "launch": {"forward": fwd_shape, "backward": bwd_shape},
           "bwd_kernel_frac_of_hbm_peak_no_reuse": norm_roofline(bench, cold, None).get("frac")}
    bench.free()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="rmsnorm_bf16_16384x4096", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the other configurations of the benchmark contract (default run only)")
    ap.add_argument("--steps-only", action="store_true",
                    help="only the step itself (timed, then once more with events): every launch a profiler sees is "
                         "one of the step's")
    ap.add_argument("--policy", choices=("keep", "stream"), default="keep",
                    help="cache policy of the forward's read of x for --steps-only runs")
    ap.add_argument("--lag", type=int, default=0,
                    help="--steps-only: the backward works on the batch forwarded this many steps earlier (2 = no reuse)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="append five plain tensor copies of known size (reference points for rocprofv3 counters)")
    ap.add_argument("--ceiling", action="store_true",
                    help="instead of a workload: what plain streams reach on this GPU (copy, 2 reads + 1 write, empty "
                         "launches) and the launch intercept / slope of the norm kernels over 8192 ... 32768 rows")
    ap.add_argument("--scan", action="store_true",
                    help="instead of a workload: forward + backward of RMSNorm and LayerNorm over a grid of row widths "
                         "and row counts per storage type, %% of HBM peak per cell (the table the launch heuristic is "
                         "fitted against)")
    ap.add_argument("--scan-log2-elements", type=int, default=26,
                    help="--scan: elements per tensor in the long class, as a power of two (26: 2^26)")
    ap.add_argument("--host", action="store_true",
                    help="instead of a workload: the host cost of the module path (per-call microseconds of the Python "
                         "layer) and where forward + backward through the modules turns host-bound")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this path runs on ONE GPU: rows are independent and nothing here uses a second device; "
                 "run with --gpus 1 (a data-parallel job would only add one all-reduce of dW / dB).")

    import torch
    from TritonHub import _native

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback.")
    lib = _native.lib()
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    if args.ceiling:
        return ceiling_main(args, lib, dev)
    if args.scan:
        return scan_main(args, lib, dev)
    if args.host:
        return host_main(args, lib, dev)
    kind, m, n, dname = WORKLOADS[args.workload]
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[dname]
    if kind == "dropout":
        return dropout_main(args, lib, dev, m, n, dname, dtype)
    if kind in SOFTMAX_KINDS or kind.startswith(("normalize", "pnorm", "act_")):
        return softmax_main(args, lib, dev, kind, m, n, dname, dtype)

    bench = NormBench(lib, dev, args.workload)
    headline = args.workload == "rmsnorm_bf16_16384x4096"
    if args.steps_only:
        res = measure_norm(bench, args, args.policy, args.lag)
        cold = res if args.lag > 0 else None
        warm = res if args.lag == 0 else None
    else:
        res = warm = measure_norm(bench, args, "keep", 0)
        cold = measure_norm(bench, args, "stream", 2, preroll=0) if bench.fused_act < 0 else None
    kern = res.get("kernels_us")
    fwd_shape, bwd_shape = bench.shapes()
    roofline = norm_roofline(bench, cold, warm)
    if "achieved" not in roofline:             # the fused backward has no separate stage entry points
        pair = bench.isolated_launch_us(bench.backward, args.steps, args.warmup)
        achieved = bench.bwd_bytes / (pair * 1e-6) / 1e9
        roofline.update({"achieved": round(achieved, 1), "frac": round(achieved / HBM_PEAK_GBPS, 4),
                         "avg_launch_us": round(pair, 2),
                         "measured": "HIP events around back-to-back launches of the fused backward (both stages)"})

    op = "RMSNorm" if kind.startswith("rms") else "LayerNorm"
    out = {
        "metric": "fwd+bwd HBM GB/s and % of peak, RMSNorm/LayerNorm bf16 16384x4096",
        "value": res["GBps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": res["ms_per_step"],
        "ms_per_step_by_hip_events": res["ms_per_step_by_hip_events"],
        "pct_of_hbm_peak_by_hip_events": res["pct_of_hbm_peak_by_hip_events"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dname,
        "data": "synthetic",
        "config": {"workload": args.workload, "op": op, "rows": m,
                   "hidden": n, "eps": 1e-6, "buffer_sets": N_BUFFER_SETS, "preroll_steps": PREROLL_STEPS,
                   "entry_points": "thn_norm_act_fwd + thn_norm_act_bwd" if bench.fused_act >= 0 else "thn_norm_fwd + thn_norm_bwd",
                   **({"activation": FUSED_ACTS[bench.fused_act]} if bench.fused_act >= 0 else {}),
                   "cache_policy": (args.policy if args.steps_only else "keep") + "_x",
                   "backward_lag_steps": args.lag if args.steps_only else 0,
                   "step": STEP_NOTE if not (args.steps_only and (args.lag or args.policy == "stream")) else NO_REUSE_NOTE},
        "pct_of_hbm_peak": res["pct_of_hbm_peak"],
        "rows_per_s": res["rows_per_s"],
        "algorithmic_bytes_per_step": bench.step_bytes,
        "kernels_us": kern,
        "launch": {"forward": fwd_shape, "backward": bwd_shape},
        "roofline": roofline,
    }
    strip = lambda r: {k_: v for k_, v in r.items() if k_ != "GBps"} | {"value": r["GBps"], "unit": "GB/s"}
    if cold is not None and not args.steps_only:
        # first-class beside `value`: the no-reuse step under the stream policy, for both operators on the headline
        out["no_reuse"] = {"cache_policy": "stream_x", "what": NO_REUSE_NOTE, op.lower(): strip(cold)}
    if not args.steps_only and bench.fused_act < 0:
        # each kernel on its own: K back-to-back launches of that kernel alone
        iso_steps = min(args.steps, 50)
        iso = {}
        for pol in ("keep", "stream"):
            bench.set_policy(pol)
            iso["forward_" + pol + "_x"] = round(bench.isolated_launch_us(bench.forward, iso_steps, args.warmup), 2)
        iso["backward_dx_partials"] = round(bench.isolated_launch_us(bench.backward_stage1, iso_steps, args.warmup), 2)
        iso["backward_reduce_partials"] = round(bench.isolated_launch_us(lambda b_: bench.backward_stage2(), iso_steps,
                                                                         args.warmup), 2)
        out["isolated_kernels_us"] = iso
    if args.calibration_copy:
        # a plain copy of known size (x -> y: m*n*s bytes read, as many written) for scaling the HBM counters
        for i in range(5):
            bench.sets[i % N_BUFFER_SETS]["y"].copy_(bench.sets[i % N_BUFFER_SETS]["x"])
        torch.cuda.synchronize()
    cpu_args = (kind, m, n, bench.dtype, {k_: v for k_, v in bench.sets[0].items() if k_ in ("x", "dy")}, bench.w,
                bench.b, bench.step_bytes)
    bench.free()

    # The metric names both operators: on the default workload the LayerNorm step of the same shape is measured
    # the same way and reported beside it (`value` stays the RMSNorm step), and the other configurations of the
    # benchmark contract follow.
    if headline and not args.steps_only:
        other = NormBench(lib, dev, "layernorm_bf16_16384x4096")
        r2 = measure_norm(other, args, "keep", 0)
        c2 = measure_norm(other, args, "stream", 2, preroll=0)
        out["layernorm_same_shape"] = {"workload": "layernorm_bf16_16384x4096",
                                       "algorithmic_bytes_per_step": other.step_bytes, **strip(r2),
                                       "roofline": norm_roofline(other, c2, r2)}
        out["no_reuse"]["layernorm"] = strip(c2)
        other.free()
        if not args.no_configs:
            short = argparse.Namespace(steps=min(args.steps, 50), warmup=args.warmup)
            out["configs"] = {w_: config_summary(lib, dev, w_, short) for w_ in CONTRACT_CONFIGS}
    if not args.no_cpu_baseline and not args.steps_only and bench.fused_act < 0:      # (the fused workloads carry no CPU leg)
        out["cpu_baseline"] = cpu_baseline(*cpu_args)
    if headline and not args.steps_only:
        # The figures of the whole line once more, short, as its last key (a reader who keeps only the end of the line
        # still has every workload), and as plain numbers inside `config`.
        def row(r, cold_):
            k = r.get("kernels_us") or {}
            return [r["pct_of_hbm_peak"], cold_["pct_of_hbm_peak"] if cold_ else None, round(r["ms_per_step"] * 1e3, 1),
                    [k.get("forward"), k.get("backward_dx_partials"), k.get("backward_reduce_partials")]]
        digest = {"columns": ["% of 8 TB/s, same-batch step, keep_x", "% of 8 TB/s, no-reuse step, stream_x", "us per step",
                              "us forward | backward dx+partials | second stage, inside the step"],
                  "rmsnorm_bf16_16384x4096": row(res, cold),
                  "layernorm_bf16_16384x4096": row(out["layernorm_same_shape"], out["no_reuse"]["layernorm"])}
        for w_, c in out.get("configs", {}).items():
            k = c.get("kernels_us") or {}
            digest[w_] = [c["pct_of_hbm_peak"], c["no_reuse_pct"], round(c["ms_per_step"] * 1e3, 1),
                          [k.get("forward"), k.get("backward_dx_partials"), k.get("backward_reduce_partials")]]
        out["config"].update({"layernorm_same_shape_pct_of_hbm_peak": out["layernorm_same_shape"]["pct_of_hbm_peak"],
                              "no_reuse_stream_x_rmsnorm_pct_of_hbm_peak": cold["pct_of_hbm_peak"],
                              "no_reuse_stream_x_layernorm_pct_of_hbm_peak": out["no_reuse"]["layernorm"]["pct_of_hbm_peak"]})
        out["digest"] = digest
    print(json.dumps(out), flush=True)


SCAN_WIDTHS = [20, 50, 64, 72, 96, 100, 120, 128, 192, 197, 200, 248, 256, 320, 384, 512, 640, 768, 896, 1000, 1024, 1152, 1280, 1408, 1536, 1600, 1792,
               2048, 2304, 2560, 2816, 3072, 3584, 4000, 4096, 4098, 4104, 4608, 5120, 5632, 6000, 6144, 6656, 7168, 8192,
               9216, 10240, 12288, 14336, 16384, 20480, 24576, 28672, 32768]


SCAN_TABLE = "norm_step_width_scan_bf16_f16_f32.txt"
SCAN_WARMUP_STEPS = 60


def scan_reference():
    """{(storage type name, N): (RMSNorm %, LayerNorm %)} of the long class of the committed width scan (the first table
    of profiles/norm_step_width_scan_bf16_f16_f32.txt, 2^26 elements per tensor): what `--scan` printed on the GPU and
    the build the launch heuristic was last fitted on."""
    table = {}
    path = os.path.join(ROOT, "profiles", SCAN_TABLE)
    if not os.path.exists(path):
        return table
    with open(path) as fh:
        for line in fh:
            if line.startswith("----"):
                break                                       # the tables of other sizes follow
            parts = line.split()
            if len(parts) > 6 and parts[0] in ("bf16", "f16", "f32") and parts[3] == "|":
                try:
                    table[(parts[0], int(parts[1]))] = (float(parts[4]), float(parts[5]))
                except ValueError:
                    pass
    return table


def scan_pool(dev, dtype, total, gen):
    import torch
    return [{k: (torch.randn(total, device=dev, generator=gen).to(dtype) if k in ("x", "dy")
                 else torch.empty(total, device=dev, dtype=dtype)) for k in ("x", "dy", "y", "dx")}
            for _ in range(N_BUFFER_SETS)]


def scan_cell(lib, dev, pool, m, n, dtype, ln, steps, gen):
    """Forward + backward of one batch of m rows of n columns through the C ABI (same batch, 'keep' policy), the
    buffers taken from `pool` in rotation: % of the HBM peak on the algorithmic bytes, best of two runs of `steps`."""
    import torch
    from TritonHub import _native
    p = _native.ptr
    stream = torch.cuda.current_stream(dev).cuda_stream
    code = _native.dtype_code(dtype)
    s = torch.empty(0, dtype=dtype).element_size()
    w = (1.0 + 0.1 * torch.randn(n, device=dev, generator=gen)).to(dtype)
    b = (0.1 * torch.randn(n, device=dev, generator=gen)).to(dtype)
    dw, db = torch.empty_like(w), torch.empty_like(w)
    mean = torch.empty(m, device=dev)
    rstd = torch.empty(m, device=dev)
    ws_bytes = lib.thn_norm_bwd_workspace_bytes(m, n, 1, 1, code)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)

    def step(i):
        b_ = pool[i % N_BUFFER_SETS]
        rc = lib.thn_norm_fwd(p(b_["x"]), n, p(b_["y"]), n, p(w), p(b) if ln else 0, p(mean) if ln else 0,
                              p(rstd), m, n, 1e-6, code | _native.X_KEEP, code, stream)
        assert rc == 0, _native.strerror(rc)
        rc = lib.thn_norm_bwd(p(b_["x"]), n, p(b_["dy"]), n, p(b_["dx"]), n, p(w), p(mean) if ln else 0,
                              p(rstd), p(dw), p(db) if ln else 0, p(ws), ws_bytes, m, n, code, code, stream)
        assert rc == 0, _native.strerror(rc)
    # untimed steps first: the engine clock follows the load, and a cell whose kernels issue more arithmetic than the
    # cell before it takes some 100 launches to reach its steady state (LayerNorm over 72 bfloat16 columns: the first
    # 100 backward launches 77-88 us, then 66)
    for i in range(SCAN_WARMUP_STEPS):
        step(i)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for _ in range(2):
        start.record()
        for i in range(steps):
            step(i)
        stop.record()
        torch.cuda.synchronize()
        best = min(best, start.elapsed_time(stop) / steps)
    f_, b__ = algorithmic_bytes("ln" if ln else "rms", m, n, s, s)
    return 100.0 * (f_ + b__) / (best * 1e-3) / 1e9 / HBM_PEAK_GBPS


def scan_main(args, lib, dev):
    """Forward + backward of one batch (same batch, 'keep' policy) for RMSNorm and LayerNorm over a grid of row widths
    and two row-count classes per storage type, in % of the HBM peak on the algorithmic bytes: the table the launch
    heuristic (plan_launch in thn_api.hip) was fitted against, regenerated for the build and the GPU at hand.
    Prints a text table, one line per (storage type, width); at the size of the committed table (2^26 elements) a last
    column gives the ratio to that table's figures, and the run ends with the cells that fell below 0.9 of them."""
    import torch
    from TritonHub.Normalization import _launch
    total = 1 << args.scan_log2_elements                   # elements per tensor in the long class
    steps = min(args.steps, 30)
    gen = torch.Generator(device=dev).manual_seed(0)
    props = torch.cuda.get_device_properties(dev)
    reference = scan_reference() if args.scan_log2_elements == 26 else {}
    behind = []
    print(f"# bench.py --scan: forward + backward of one batch, % of {HBM_PEAK_GBPS:.0f} GB/s on the algorithmic bytes; "
          f"{props.name}, {props.multi_processor_count} compute units; {SCAN_WARMUP_STEPS} untimed + 2 x {steps} timed steps per cell (the better half counts), four buffer sets")
    print(f"# classes: long = 2^{args.scan_log2_elements} elements per tensor; short = 16 rows per compute unit (omitted where that is the long class "
          "or more)")
    print("# launch = forward KxTPR/BLOCK@grid | backward KxTPR/BLOCK@grid of the long class (LayerNorm)")
    print(f"{'dtype':5} {'N':>6} {'rows':>8} | {'RMS long':>8} {'LN long':>8} | {'rows':>6} {'RMS short':>9} {'LN short':>9} | launch")
    for dname in ("bf16", "f32", "f16"):
        dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[dname]
        s = torch.empty(0, dtype=dtype).element_size()
        pool = scan_pool(dev, dtype, total, gen)
        for n in SCAN_WIDTHS:
            if n * s > 65536:
                continue
            cells = {}
            m_long = total // n
            m_short = 16 * props.multi_processor_count
            for cls, m in (("long", m_long), ("short", m_short)):
                if cls == "short" and m_short >= m_long:
                    continue
                for ln in (False, True):
                    cells[(cls, ln)] = scan_cell(lib, dev, pool, m, n, dtype, ln, steps, gen)
            f = _launch.query_launch(0, True, m_long, n, dtype)
            g = _launch.query_launch(1, True, m_long, n, dtype)
            launch = f"{f[0]}x{f[1]}/{f[2]}@{f[3]} | {g[0]}x{g[1]}/{g[2]}@{g[3]}" + ("" if f[4] else "  (off the 128-bit path)")
            short = (f"{m_short:6d} {cells[('short', False)]:9.1f} {cells[('short', True)]:9.1f}" if ("short", False) in cells
                     else f"{'':6} {'':9} {'':9}")
            against = ""
            if (dname, n) in reference:
                ratios = [cells[("long", ln)] / max(reference[(dname, n)][int(ln)], 1e-9) for ln in (False, True)]
                against = f" | x{ratios[0]:.2f} x{ratios[1]:.2f} of the committed table"
                for ln, r in zip((False, True), ratios):
                    if r < 0.9:
                        behind.append(f"{dname} N={n} {'LayerNorm' if ln else 'RMSNorm'}: {cells[('long', ln)]:.1f} % against "
                                      f"{reference[(dname, n)][int(ln)]:.1f} %")
            print(f"{dname:5} {n:6d} {m_long:8d} | {cells[('long', False)]:8.1f} {cells[('long', True)]:8.1f} | {short} | {launch}{against}",
                  flush=True)
        del pool
        torch.cuda.empty_cache()
    if reference:
        print(f"# cells below 0.9 of profiles/{SCAN_TABLE}: {len(behind)}")
        for line in behind:
            print("#   " + line)


def host_main(args, lib, dev):
    """What the Python layer costs on the host, and where the module path turns host-bound: bfloat16 rows of 4096."""
    import torch
    from TritonHub.Normalization import LayerNorm, RMSNorm, _launch
    n, dtype = 4096, torch.bfloat16
    out = {"what": "host cost of the operator layer (autograd Function + launch wrapper + C ABI) per call, and forward + "
                   "backward through the modules against the same step through the C ABI; bfloat16 rows of 4096",
           "host_us_per_call": {}, "module_path": {}}
    # host cost: so few rows that the GPU never holds the host up; the clock runs over enqueueing only
    x = torch.randn(8, n, device=dev).to(dtype)
    dy = torch.randn(8, n, device=dev).to(dtype)
    w = torch.ones(n, device=dev, dtype=dtype)
    b = torch.zeros(n, device=dev, dtype=dtype)
    reps = 2000

    def host_us(fn):
        for _ in range(200):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        t = (time.perf_counter() - t0) * 1e6 / reps
        torch.cuda.synchronize()
        return round(t, 2)

    for ln in (False, True):
        name = "layernorm" if ln else "rmsnorm"
        _, mean, rstd = _launch.norm_fwd(x, w, b if ln else None, 1e-6, ln)
        out["host_us_per_call"][name] = {
            "_launch.norm_fwd": host_us(lambda: _launch.norm_fwd(x, w, b if ln else None, 1e-6, ln)),
            "_launch.norm_bwd": host_us(lambda: _launch.norm_bwd(x, dy, w, b if ln else None, mean, rstd, ln))}
        mod = (LayerNorm if ln else RMSNorm)(n, eps=1e-6, device=dev, dtype=dtype)
        xg = x.clone().requires_grad_(True)

        def fb():
            mod(xg).backward(dy)
        out["host_us_per_call"][name]["module forward + backward (autograd included)"] = host_us(fb)
        with torch.no_grad():
            out["host_us_per_call"][name]["module forward under no_grad"] = host_us(lambda: mod(x))
    # module path against the C ABI over row counts
    for ln in (False, True):
        name = "layernorm" if ln else "rmsnorm"
        rows_out = {}
        for m in (256, 1024, 2048, 4096, 8192, 16384):
            bench = NormBench(lib, dev, "layernorm_bf16_16384x4096" if ln else "rmsnorm_bf16_16384x4096")
            bench.m = m
            short = argparse.Namespace(steps=min(args.steps, 100), warmup=10)
            abi = measure_norm(bench, short, "keep", 0, preroll=20, with_kernels=False)
            mod = (LayerNorm if ln else RMSNorm)(n, eps=1e-6, device=dev, dtype=dtype)
            xs = [bench.sets[i]["x"][:m].requires_grad_(True) for i in range(N_BUFFER_SETS)]
            dys = [bench.sets[i]["dy"][:m] for i in range(N_BUFFER_SETS)]

            def step(i):
                xi = xs[i % N_BUFFER_SETS]
                xi.grad = None
                mod(xi).backward(dys[i % N_BUFFER_SETS])
            for i in range(20):
                step(i)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(short.steps):
                step(i)
            torch.cuda.synchronize()
            mod_us = (time.perf_counter() - t0) * 1e6 / short.steps
            rows_out[str(m)] = {"c_abi_us_per_step": round(abi["ms_per_step"] * 1e3, 2), "module_us_per_step": round(mod_us, 2),
                                "host_bound": bool(mod_us > 1.15 * abi["ms_per_step"] * 1e3)}
            bench.free()
            del xs, dys
        out["module_path"][name] = rows_out
    print(json.dumps(out), flush=True)


def ceiling_main(args, lib, dev):
    """What a plain stream reaches on this GPU, next to the norm kernels: the evidence for how far from the memory
    system's own ceiling they run.  Every line is launches between one pair of HIP events on the launch stream,
    over four rotating buffer sets; rocprofv3 --kernel-trace --stats of this command gives the same kernels'
    durations."""
    import torch
    from TritonHub import _native
    p = _native.ptr
    stream = torch.cuda.current_stream(dev).cuda_stream
    n, dtype, code, s = 4096, torch.bfloat16, _native.dtype_code(torch.bfloat16), 2
    rows_list = [8192, 12288, 16384, 24576, 32768]     # from 128 MiB per batch up: four batches exceed every cache
    mmax = max(rows_list)
    gen = torch.Generator(device=dev).manual_seed(0)
    sets = []
    for _ in range(N_BUFFER_SETS):
        x = torch.randn(mmax, n, device=dev, generator=gen).to(dtype)
        dy = torch.randn(mmax, n, device=dev, generator=gen).to(dtype)
        sets.append(dict(x=x, dy=dy, y=torch.empty_like(x), dx=torch.empty_like(x), rstd=torch.empty(mmax, device=dev),
                         mean=torch.empty(mmax, device=dev)))
    w = (1.0 + 0.1 * torch.randn(n, device=dev, generator=gen)).to(dtype)
    b = (0.1 * torch.randn(n, device=dev, generator=gen)).to(dtype)
    dw, db = torch.empty_like(w), torch.empty_like(w)
    ws_bytes = lib.thn_norm_bwd_workspace_bytes(mmax, n, 1, 1, code)
    ws = torch.empty(max(ws_bytes, 16) // 4, device=dev)
    parts = ctypes.c_int32(0)

    def timed(launch, iters):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(10):
            launch(sets[i % N_BUFFER_SETS])
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(3):
            start.record()
            for i in range(iters):
                launch(sets[i % N_BUFFER_SETS])
            stop.record()
            torch.cuda.synchronize()
            best = min(best, start.elapsed_time(stop) * 1e3 / iters)
        return best

    def fit(points):          # least squares t = a + b*m
        k = len(points)
        sx = sum(m_ for m_, _ in points); sy = sum(t for _, t in points)
        sxx = sum(m_ * m_ for m_, _ in points); sxy = sum(m_ * t for m_, t in points)
        slope = (k * sxy - sx * sy) / (k * sxx - sx * sx)
        return (sy - slope * sx) / k, slope

    out = {"what": "stream ceilings and launch intercepts, bfloat16 rows of 4096, four rotating buffer sets",
           "hbm_peak_GBps": HBM_PEAK_GBPS, "streams": {}, "norm_kernels": {}}
    empty = torch.empty(0, device=dev, dtype=dtype)

    def act_fwd(b_, m_):
        rc = lib.thn_act_fwd(p(b_["x"]), n, p(b_["y"]), n, m_, n, 3, 0.0, 0.0, code, stream)
        assert rc == 0, rc

    def act_bwd(b_, m_):
        rc = lib.thn_act_bwd(p(b_["x"]), n, p(b_["dy"]), n, p(b_["dx"]), n, m_, n, 3, 0.0, 0.0, code, stream)
        assert rc == 0, rc

    def norm_fwd(b_, m_, ln):
        rc = lib.thn_norm_fwd(p(b_["x"]), n, p(b_["y"]), n, p(w), p(b) if ln else 0, p(b_["mean"]) if ln else 0,
                              p(b_["rstd"]), m_, n, 1e-6, code | _native.X_STREAM, code, stream)     # a forward on its own: x streams
        assert rc == 0, rc

    def norm_bwd1(b_, m_, ln):
        rc = lib.thn_norm_bwd_dx_partials(p(b_["x"]), n, p(b_["dy"]), n, p(b_["dx"]), n, p(w), p(b_["mean"]) if ln else 0,
                                          p(b_["rstd"]), 1, int(ln), p(ws), ws_bytes, ctypes.byref(parts), m_, n, code,
                                          code, stream)
        assert rc == 0, rc

    streams = {
        "torch copy_ (1 read + 1 write)": (lambda b_, m_: b_["y"][:m_].copy_(b_["x"][:m_]), 2),
        "torch add out= (2 reads + 1 write)": (lambda b_, m_: torch.add(b_["x"][:m_], b_["dy"][:m_], out=b_["dx"][:m_]), 3),
        "thn_act_fwd ReLU (1 read + 1 write)": (act_fwd, 2),
        "thn_act_bwd ReLU (2 reads + 1 write)": (act_bwd, 3),
    }
    for name, (fn, units) in streams.items():
        pts = [(m_, timed(lambda b_, m_=m_: fn(b_, m_), 40)) for m_ in rows_list]
        a0, slope = fit(pts)
        out["streams"][name] = {
            "us_per_launch": {str(m_): round(t, 2) for m_, t in pts},
            "GBps_at_16384_rows": round(units * 16384 * n * s / dict(pts)[16384] / 1e3, 1),
            "fit_intercept_us": round(a0, 2), "fit_slope_GBps": round(units * n * s / slope / 1e3, 1)}
    for name, fn, units in (("rmsnorm forward", lambda b_, m_: norm_fwd(b_, m_, False), 2),
                            ("layernorm forward", lambda b_, m_: norm_fwd(b_, m_, True), 2),
                            ("rmsnorm backward dx + partials", lambda b_, m_: norm_bwd1(b_, m_, False), 3),
                            ("layernorm backward dx + partials", lambda b_, m_: norm_bwd1(b_, m_, True), 3)):
        if "backward" in name:           # the statistics the backward reads must be those of the rows it is given
            for b_ in sets:
                norm_fwd(b_, mmax, "layernorm" in name)
        pts = [(m_, timed(lambda b_, m_=m_: fn(b_, m_), 40)) for m_ in rows_list]
        a0, slope = fit(pts)
        out["norm_kernels"][name] = {
            "us_per_launch": {str(m_): round(t, 2) for m_, t in pts},
            "GBps_at_16384_rows": round(units * 16384 * n * s / dict(pts)[16384] / 1e3, 1),
            "fit_intercept_us": round(a0, 2), "fit_slope_GBps": round(units * n * s / slope / 1e3, 1)}
    # forward + backward of the SAME batch, back to back (16384 rows): what the memory-side cache gives a 2-read-1-write
    # stream that follows a 1-read-1-write stream over one of its inputs -- the plain streams (the ReLU forward keeps x
    # with cache-allocating loads, like the norm forward under the keep policy) next to the norm kernels
    def norm_fwd_keep(b_, m_, ln):
        rc = lib.thn_norm_fwd(p(b_["x"]), n, p(b_["y"]), n, p(w), p(b) if ln else 0, p(b_["mean"]) if ln else 0,
                              p(b_["rstd"]), m_, n, 1e-6, code | _native.X_KEEP, code, stream)
        assert rc == 0, rc

    def pair(f, g_):
        def both(b_):
            f(b_, 16384)
            g_(b_, 16384)
        return both
    out["same_batch_pairs_us_at_16384_rows"] = {
        "thn_act_fwd + thn_act_bwd ReLU": round(timed(pair(act_fwd, act_bwd), 40), 2),
        "rmsnorm forward (keep_x) + backward dx + partials": round(timed(pair(lambda b_, m_: norm_fwd_keep(b_, m_, False),
                                                                              lambda b_, m_: norm_bwd1(b_, m_, False)), 40), 2),
        "layernorm forward (keep_x) + backward dx + partials": round(timed(pair(lambda b_, m_: norm_fwd_keep(b_, m_, True),
                                                                                lambda b_, m_: norm_bwd1(b_, m_, True)), 40), 2)}
    # the second stage alone, and launches that move nothing
    norm_bwd1(sets[0], 16384, False)
    out["second_stage_us"] = round(timed(lambda b_: lib.thn_norm_bwd_reduce_partials(p(ws), parts.value, p(dw), 0, n, code,
                                                                                     stream), 200), 2)
    out["empty_launch_us"] = {
        "thn_act_fwd on 0 rows (returns before launching)": round(timed(lambda b_: act_fwd(b_, 0), 200), 2),
        "thn_act_fwd on 1 row": round(timed(lambda b_: act_fwd(b_, 1), 400), 2),
        "torch copy_ of 8 elements": round(timed(lambda b_: b_["y"][0, :8].copy_(b_["x"][0, :8]), 400), 2)}

    print(json.dumps(out), flush=True)


def softmax_main(args, lib, dev, kind, m, n, dname, dtype):
    """One step = thn_softmax_fwd + thn_softmax_bwd (the backward reads the output the forward just wrote,
    as the autograd Function does) over one of four rotating buffer sets."""
    import torch
    from TritonHub import _native
    from TritonHub.Normalization import _launch
    s = torch.empty(0, dtype=dtype).element_size()
    code = _native.dtype_code(dtype)
    kcode = {"softmax": _native.SOFTMAX, "softmin": _native.SOFTMIN, "logsoftmax": _native.LOGSOFTMAX}.get(kind)
    row_op = None if kcode is not None else kind.split("_")[0]          # "normalize", "pnorm" or "act"
    pval = float(kind[-1]) if row_op in ("normalize", "pnorm") else 0.0
    act_name = kind[4:] if row_op == "act" else None
    act_code = ACT_NAMES.index(act_name) if act_name else -1
    ap0, ap1 = ACT_PARAMS.get(act_name, (0.0, 0.0))
    saves_output = act_name in ("sigmoid", "tanh")
    gen = torch.Generator(device=dev).manual_seed(0)
    sets = []
    for _ in range(N_BUFFER_SETS):
        x = (3.0 * torch.randn(m, n, device=dev, generator=gen)).to(dtype)
        dy = torch.randn(m, n, device=dev, generator=gen).to(dtype)
        sets.append(dict(x=x, dy=dy, y=torch.empty_like(x), dx=torch.empty_like(x),
                         norms=torch.empty(m, device=dev, dtype=dtype),
                         dnorms=torch.rand(m, device=dev, generator=gen).to(dtype)))
    stream = torch.cuda.current_stream(dev).cuda_stream
    p = _native.ptr
    mn = m * n

    def forward(b_):
        if row_op == "normalize":
            rc = lib.thn_normalize_fwd(p(b_["x"]), mn, n, p(b_["y"]), mn, n, p(b_["norms"]), 1, m, n, pval, 1e-12, code,
                                       stream)
        elif row_op == "pnorm":
            rc = lib.thn_pnorm_fwd(p(b_["x"]), mn, n, p(b_["norms"]), 1, m, n, pval, 1e-12, code, stream)
        elif row_op == "act":
            rc = lib.thn_act_fwd(p(b_["x"]), n, p(b_["y"]), n, m, n, act_code, ap0, ap1, code, stream)
        else:
            rc = lib.thn_softmax_fwd(p(b_["x"]), n, p(b_["y"]), n, m, n, kcode, code, stream)
        assert rc == 0, _native.strerror(rc)

    def backward(b_):
        if row_op == "normalize":
            rc = lib.thn_normalize_bwd(p(b_["x"]), mn, n, p(b_["y"]), mn, n, p(b_["norms"]), p(b_["dy"]), mn, n,
                                       p(b_["dx"]), mn, n, 1, m, n, pval, code, stream)
        elif row_op == "pnorm":
            rc = lib.thn_pnorm_bwd(p(b_["x"]), mn, n, p(b_["norms"]), p(b_["dnorms"]), p(b_["dx"]), mn, n, 1, m, n,
                                   pval, code, stream)
        elif row_op == "act":
            rc = lib.thn_act_bwd(p(b_["y"] if saves_output else b_["x"]), n, p(b_["dy"]), n, p(b_["dx"]), n, m, n,
                                 act_code, ap0, ap1, code, stream)
        else:
            rc = lib.thn_softmax_bwd(p(b_["y"]), n, p(b_["dy"]), n, p(b_["dx"]), n, m, n, kcode, code, stream)
        assert rc == 0, _native.strerror(rc)

    def step(i):
        forward(sets[i % N_BUFFER_SETS])
        backward(sets[i % N_BUFFER_SETS])

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    fwd_bytes, bwd_bytes = algorithmic_bytes(kind, m, n, s, s)
    step_bytes = fwd_bytes + bwd_bytes
    gbps = step_bytes / (ms_per_step * 1e-3) / 1e9

    def avg_launch_us(launch):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(min(args.warmup, 5)):
            launch(sets[i % N_BUFFER_SETS])
        torch.cuda.synchronize()
        start.record()
        for i in range(args.steps):
            launch(sets[i % N_BUFFER_SETS])
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) * 1e3 / args.steps

    fwd_us = avg_launch_us(forward)
    bwd_us = avg_launch_us(backward)
    if args.calibration_copy:
        for i in range(5):
            sets[i % N_BUFFER_SETS]["dx"].copy_(sets[i % N_BUFFER_SETS]["x"])
        torch.cuda.synchronize()
    achieved = bwd_bytes / (bwd_us * 1e-6) / 1e9
    fam = {None: (2, 3), "normalize": (4, 6), "pnorm": (4, 5), "act": None}[row_op]
    if fam is not None:
        # (for the p-norm forward the flag asks for the launch of the normalize entry point)
        fs = _launch.query_launch(fam[0], kind == "logsoftmax" or row_op == "normalize", m, n, dtype)
        bs = _launch.query_launch(fam[1], kind == "logsoftmax", m, n, dtype)
    else:                                   # flat element-wise kernels: vectors per thread and step, no rows
        fs, bs = (4, 0, 256, 0), (2 if act_name in ("gelu", "gelu_tanh", "mish") else 4, 0, 256, 0)
    bwd_kernel = {None: "softmax_bwd_kernel", "normalize": "normalize_bwd_kernel", "pnorm": "pnorm_bwd_kernel",
                  "act": "act_flat_kernel (backward)"}[row_op]
    entry = {None: "thn_softmax_fwd + thn_softmax_bwd", "normalize": "thn_normalize_fwd + thn_normalize_bwd",
             "pnorm": "thn_pnorm_fwd + thn_pnorm_bwd", "act": "thn_act_fwd + thn_act_bwd"}[row_op]
    out = {
        "metric": f"fwd+bwd HBM GB/s and % of peak, {kind} {dname} {m}x{n}",
        "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dname, "data": "synthetic",
        "config": {"workload": args.workload, "op": kind, "rows": m, "row_width": n, "buffer_sets": N_BUFFER_SETS,
                   "entry_points": entry},
        "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "rows_per_s": round(m / (ms_per_step * 1e-3)),
        "algorithmic_bytes_per_step": step_bytes,
        "kernels_us": {"forward": round(fwd_us, 2), "backward": round(bwd_us, 2),
                       "forward_GBps": round(fwd_bytes / (fwd_us * 1e-6) / 1e9, 1)},
        "launch": {"forward": dict(zip(("vecs_per_thread", "threads_per_row", "block", "grid"), fs[:4])),
                   "backward": dict(zip(("vecs_per_thread", "threads_per_row", "block", "grid"), bs[:4]))},
        "roofline": {"bound": "hbm", "kernel": bwd_kernel, "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "algorithmic_bytes_per_launch": bwd_bytes, "avg_launch_us": round(bwd_us, 2),
                     **traffic_fields(args.workload)},
    }
    if not args.no_cpu_baseline:
        baseline = {None: softmax_cpu_baseline, "act": act_cpu_baseline}.get(row_op, row_op_cpu_baseline)
        out["cpu_baseline"] = baseline(kind, m, n, dtype, sets[0], step_bytes)
    print(json.dumps(out), flush=True)


def dropout_main(args, lib, dev, m, n, dname, dtype):
    """One step = thn_dropout on x (forward) + thn_dropout on dy with the same seed (backward), p = 0.1, over one of
    four rotating buffer sets.  Every element costs a Philox-4x32-10 block of its own (the reference draws
    tl.rand(seed, i) per element): the kernel is bound by 32-bit integer multiplications, and the HBM fraction below
    says how far that is from the memory roofline, not how good the kernel is."""
    import torch
    from TritonHub import _native
    s = torch.empty(0, dtype=dtype).element_size()
    code = _native.dtype_code(dtype)
    gen = torch.Generator(device=dev).manual_seed(0)
    sets = []
    for _ in range(N_BUFFER_SETS):
        x = torch.randn(m, n, device=dev, generator=gen).to(dtype)
        dy = torch.randn(m, n, device=dev, generator=gen).to(dtype)
        sets.append(dict(x=x, dy=dy, y=torch.empty_like(x), dx=torch.empty_like(x)))
    stream = torch.cuda.current_stream(dev).cuda_stream
    p = _native.ptr
    mn, prob = m * n, 0.1

    def forward(b_, seed=12345):
        rc = lib.thn_dropout(p(b_["x"]), p(b_["y"]), mn, 0, prob, seed, code, stream)
        assert rc == 0, _native.strerror(rc)

    def backward(b_, seed=12345):
        rc = lib.thn_dropout(p(b_["dy"]), p(b_["dx"]), mn, 0, prob, seed, code, stream)
        assert rc == 0, _native.strerror(rc)

    def step(i):
        forward(sets[i % N_BUFFER_SETS], 1000 + i)
        backward(sets[i % N_BUFFER_SETS], 1000 + i)

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    launch_bytes = 2 * mn * s
    step_bytes = 2 * launch_bytes
    gbps = step_bytes / (ms_per_step * 1e-3) / 1e9
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(args.steps):
        forward(sets[i % N_BUFFER_SETS])
    stop.record()
    torch.cuda.synchronize()
    fwd_us = start.elapsed_time(stop) * 1e3 / args.steps
    achieved = launch_bytes / (fwd_us * 1e-6) / 1e9
    out = {
        "metric": f"fwd+bwd HBM GB/s and % of peak, dropout {dname} {m}x{n}",
        "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dname, "data": "synthetic",
        "config": {"workload": args.workload, "op": "dropout", "rows": m, "row_width": n, "p": prob,
                   "buffer_sets": N_BUFFER_SETS, "entry_points": "thn_dropout (x) + thn_dropout (dy)"},
        "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "elements_per_s": round(2 * mn / (ms_per_step * 1e-3)),
        "algorithmic_bytes_per_step": step_bytes,
        "kernels_us": {"forward": round(fwd_us, 2)},
        "roofline": {"bound": "hbm", "kernel": "dropout_flat_kernel", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "algorithmic_bytes_per_launch": launch_bytes, "avg_launch_us": round(fwd_us, 2), "traffic": None,
                     "note": "limited by the 37 32x32-bit multiplications of one Philox-4x32-10 block per element "
                             "(quarter-rate instructions), not by memory"},
    }
    if not args.no_cpu_baseline:
        from oracle import dropout_oracle as do
        rows = min(m, max(16, (1 << 21) // n))
        x = sets[0]["x"][:rows].float().cpu().numpy()
        dy = sets[0]["dy"][:rows].float().cpu().numpy()

        def oracle_step():
            do.dropout(x, prob, 12345)
            do.dropout(dy, prob, 12345)

        oracle_step()
        best = float("inf")
        for _ in range(3):
            t0 = time.perf_counter()
            oracle_step()
            best = min(best, time.perf_counter() - t0)
        out["cpu_baseline"] = {"value": round(step_bytes * rows / m / best / 1e9, 3), "unit": "GB/s", "cores": 1,
                               "kind": "port",
                               "sample": f"first {rows} of {m} rows of the same workload, forward + backward, best of 3 "
                                         f"passes of oracle/dropout_oracle.py (numpy, one thread; {best * 1e3:.1f} ms "
                                         "per pass)",
                               "host_cpu_count": os.cpu_count()}
    print(json.dumps(out), flush=True)


def act_cpu_baseline(kind, m, n, dtype, buffers, step_bytes):
    """oracle/act_oracle.py (numpy float64, one thread) on a bounded sample of the same rows, and torch on the host
    cores next to it."""
    import torch
    import torch.nn.functional as F
    from oracle import act_oracle as ao
    name = kind[4:]
    p0, p1 = ACT_PARAMS.get(name, (0.0, 0.0))
    rows = min(m, max(64, (1 << 23) // n))
    x = buffers["x"][:rows].cpu()
    dy = buffers["dy"][:rows].cpu()
    x64, dy64 = x.double().numpy(), dy.double().numpy()

    def oracle_step():
        y = ao.fwd(name, x64, p0, p1)
        ao.bwd(name, y if name in ao.SAVES_OUTPUT else x64, dy64, p0, p1)

    fn = {"gelu": F.gelu, "gelu_tanh": lambda t: F.gelu(t, approximate="tanh"), "silu": F.silu, "relu": F.relu,
          "leaky_relu": lambda t: F.leaky_relu(t, p0), "relu6": F.relu6, "sigmoid": torch.sigmoid, "tanh": torch.tanh,
          "mish": F.mish, "softplus": lambda t: F.softplus(t, p0, p1), "threshold": lambda t: F.threshold(t, p0, p1)}[name]

    def torch_step():
        xr = x.clone().requires_grad_(True)
        fn(xr).backward(dy)

    def timed(f, reps):
        f()
        best = float("inf")
        for _ in range(reps):
            t0 = time.perf_counter()
            f()
            best = min(best, time.perf_counter() - t0)
        return best

    sample_bytes = step_bytes * rows / m
    t_oracle, t_torch = timed(oracle_step, 3), timed(torch_step, 3)
    return {"value": round(sample_bytes / t_oracle / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"first {rows} of {m} rows of the same workload, forward + backward, best of 3 passes of "
                      f"oracle/act_oracle.py (numpy float64, one thread; {t_oracle * 1e3:.1f} ms per pass)",
            "host_cpu_count": os.cpu_count(),
            "torch_functional": {"value": round(sample_bytes / t_torch / 1e9, 2), "unit": "GB/s",
                                 "threads": torch.get_num_threads(),
                                 "what": f"torch {name} forward + autograd backward on the host cores, same sample "
                                         f"({t_torch * 1e3:.1f} ms per pass)"}}


def row_op_cpu_baseline(kind, m, n, dtype, buffers, step_bytes):
    """oracle/pnorm_oracle.py (numpy float64, one thread) on a bounded sample of the same rows, and torch on the
    host cores next to it."""
    import torch
    from oracle import pnorm_oracle as po
    op, pval = kind.split("_")[0], int(kind[-1])
    rows = min(m, max(64, (1 << 23) // n))
    x = buffers["x"][:rows].cpu()
    dy = buffers["dy"][:rows].cpu()
    gn = buffers["dnorms"][:rows].cpu()
    x64, dy64, gn64 = x.double().numpy(), dy.double().numpy(), gn.double().numpy()

    def oracle_step():
        nrm = po.norm_fwd(x64, pval, 1e-12)
        if op == "normalize":
            po.normalize_bwd(x64, po.normalize_fwd(x64, nrm), nrm, dy64, pval)
        else:
            po.norm_bwd(x64, nrm, gn64, pval)

    def torch_step():
        xr = x.clone().requires_grad_(True)
        if op == "normalize":
            torch.nn.functional.normalize(xr, p=pval, dim=-1, eps=1e-12).backward(dy)
        else:
            torch.norm(xr, p=pval, dim=-1).backward(gn)

    def timed(f, reps):
        f()
        best = float("inf")
        for _ in range(reps):
            t0 = time.perf_counter()
            f()
            best = min(best, time.perf_counter() - t0)
        return best

    sample_bytes = step_bytes * rows / m
    t_oracle, t_torch = timed(oracle_step, 3), timed(torch_step, 3)
    return {"value": round(sample_bytes / t_oracle / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"first {rows} of {m} rows of the same workload, forward + backward, best of 3 passes of "
                      f"oracle/pnorm_oracle.py (numpy float64, one thread; {t_oracle * 1e3:.1f} ms per pass)",
            "host_cpu_count": os.cpu_count(),
            "torch_functional": {"value": round(sample_bytes / t_torch / 1e9, 2), "unit": "GB/s",
                                 "threads": torch.get_num_threads(),
                                 "what": f"torch {op} forward + autograd backward on the host cores, same sample "
                                         f"({t_torch * 1e3:.1f} ms per pass)"}}


def softmax_cpu_baseline(kind, m, n, dtype, buffers, step_bytes):
    """The numpy restatement of the reference's kernels (oracle/softmax_oracle.py, one thread, float64) on a
    bounded sample of the same rows, and torch.nn.functional on the host cores next to it."""
    import torch
    from oracle import softmax_oracle as so
    rows = min(m, max(64, (1 << 23) // n))             # 8M elements per pass at most
    x = buffers["x"][:rows].cpu()
    dy = buffers["dy"][:rows].cpu()
    x64, dy64 = x.double().numpy(), dy.double().numpy()

    def oracle_step():
        so.BWD[kind](so.FWD[kind](x64), dy64)

    fn = {"softmax": torch.softmax, "softmin": lambda t, d: torch.softmax(-t, d), "logsoftmax": torch.log_softmax}[kind]

    def torch_step():
        xr = x.clone().requires_grad_(True)
        fn(xr, -1).backward(dy)

    def timed(f, reps):
        f()
        best = float("inf")
        for _ in range(reps):
            t0 = time.perf_counter()
            f()
            best = min(best, time.perf_counter() - t0)
        return best

    sample_bytes = step_bytes * rows / m
    t_oracle, t_torch = timed(oracle_step, 3), timed(torch_step, 3)
    return {"value": round(sample_bytes / t_oracle / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"first {rows} of {m} rows of the same workload, forward + backward, best of 3 passes of "
                      f"oracle/softmax_oracle.py (numpy float64, one thread; {t_oracle * 1e3:.1f} ms per pass)",
            "host_cpu_count": os.cpu_count(),
            "torch_functional": {"value": round(sample_bytes / t_torch / 1e9, 2), "unit": "GB/s",
                                 "threads": torch.get_num_threads(),
                                 "what": f"torch {kind} forward + autograd backward on the host cores, same sample "
                                         f"({t_torch * 1e3:.1f} ms per pass)"}}


def cpu_baseline(kind, m, n, dtype, buffers, w, b, step_bytes):
    """The same forward + backward on the GPU box's host cores.  `value`: torch.nn.functional.layer_norm /
    rms_norm forward + autograd backward on ALL rows of the workload (the baseline the metric names).  Nested
    `oracle_port`: the C restatement of the reference's arithmetic (oracle/norm_oracle.c, OpenMP over rows,
    storage-dtype outputs) on a bounded sample of the rows, scaled by row count."""
    import torch
    from oracle import c_oracle as co
    threads = co.num_threads()
    xa = buffers["x"].cpu()
    dya = buffers["dy"].cpu()
    wc = w.cpu()
    bc = None if b is None else b.cpu()
    rows = min(m, max(256, (1 << 25) // n))            # the oracle's sample: 32M elements per pass at most
    x, dy = xa[:rows], dya[:rows]

    def oracle_step():
        if kind == "ln":
            _, mean, rstd = co.layernorm_fwd(x, wc, bc, 1e-6, out_dtype=dtype)
            co.layernorm_bwd(x, dy, wc, mean, rstd, has_bias=True, out_dtype=dtype, param_dtype=dtype)
        else:
            _, rstd = co.rmsnorm_fwd(x, wc, 1e-6, out_dtype=dtype)
            co.rmsnorm_bwd(x, dy, wc, rstd, out_dtype=dtype, param_dtype=dtype)

    # torch on the whole workload unless that is more than 128M elements (then on the first 128M, scaled)
    t_rows = min(m, max(256, (1 << 27) // n))

    def torch_step():
        xr = xa[:t_rows].clone().requires_grad_(True)
        wr = wc.clone().requires_grad_(True)
        if kind == "ln":
            br = bc.clone().requires_grad_(True)
            y = torch.nn.functional.layer_norm(xr, (n,), wr, br, 1e-6)
        else:
            y = torch.nn.functional.rms_norm(xr, (n,), wr, 1e-6)
        y.backward(dya[:t_rows])

    def timed(fn, reps):
        fn()
        best = float("inf")
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            best = min(best, time.perf_counter() - t0)
        return best

    t_oracle = timed(oracle_step, 3)
    t_torch = timed(torch_step, 3)
    torch_threads = torch.get_num_threads()
    return {
        "value": round(step_bytes * t_rows / m / t_torch / 1e9, 2), "unit": "GB/s", "cores": torch_threads,
        "kind": "torch_functional",
        "sample": (f"all {m} rows" if t_rows == m else f"first {t_rows} of {m} rows") + " of the same workload: "
                  f"torch.nn.functional.{'layer_norm' if kind == 'ln' else 'rms_norm'} forward + autograd backward on the "
                  f"host, {torch_threads} threads, 1 warm-up + best of 3 passes ({t_torch * 1e3:.1f} ms per pass)",
        "host_cpu_count": os.cpu_count(),
        "oracle_port": {"value": round(step_bytes * rows / m / t_oracle / 1e9, 2), "unit": "GB/s", "cores": threads,
                        "kind": "port",
                        "sample": f"first {rows} of {m} rows, forward + backward, best of 3 passes of "
                                  f"oracle/norm_oracle.c with {threads} OpenMP threads ({t_oracle * 1e3:.1f} ms per pass)"},
    }


if __name__ == "__main__":
    main()
