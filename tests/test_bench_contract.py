"""CPU tests of bench.py's command-line contract: the workload table is consistent, more than one GPU is refused
with a message, and without a GPU the script says so instead of falling back to anything."""
import os
import subprocess
import sys

from conftest import ROOT

sys.path.insert(0, ROOT)
import bench  # noqa: E402


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          env={**os.environ, "WORLD_SIZE": "1"})


def test_more_than_one_gpu_is_refused_with_a_message():
    r = run("--gpus", "2")
    assert r.returncode != 0 and "ONE GPU" in (r.stderr + r.stdout)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")], capture_output=True, text=True,
                       env={**os.environ, "WORLD_SIZE": "4"})
    assert r.returncode != 0 and "ONE GPU" in (r.stderr + r.stdout)


def test_help_prints():
    r = run("--help")
    assert r.returncode == 0 and "--workload" in r.stdout and "--scan" in r.stdout, r.stderr[-400:]


def test_workload_table():
    assert "rmsnorm_bf16_16384x4096" in bench.WORKLOADS           # the configuration the headline metric is quoted on
    for name, (kind, m, n, dname) in bench.WORKLOADS.items():
        assert m > 0 and n > 0 and dname in ("bf16", "f16", "f32"), name
        s = {"bf16": 2, "f16": 2, "f32": 4}[dname]
        fwd, bwd = bench.algorithmic_bytes(kind.split("+")[0], m, n, s, s)
        assert fwd >= m * n * s and bwd >= 2 * m * n * s, name      # at least one read; a read and a write
    # algorithmic bytes of the default workload: 5*M*N*s + 8*M + 3*N*s
    f, b = bench.algorithmic_bytes("rms", 16384, 4096, 2, 2)
    assert f + b == 5 * 16384 * 4096 * 2 + 8 * 16384 + 3 * 4096 * 2
    f, b = bench.algorithmic_bytes("ln", 16384, 4096, 2, 2)
    assert f + b == 5 * 16384 * 4096 * 2 + 16 * 16384 + 5 * 4096 * 2


def test_traffic_comes_from_the_profile_summaries():
    """roofline.traffic is read from `bench.traffic` lines of the summaries under profiles/: every such line names a
    workload of the table, and the headline workload has one."""
    seen = set()
    for name in sorted(os.listdir(os.path.join(ROOT, "profiles"))):
        for line in open(os.path.join(ROOT, "profiles", name)):
            parts = line.split()
            if parts[:1] == ["bench.traffic"]:
                assert len(parts) >= 5 and parts[1] in bench.WORKLOADS and int(parts[3]) > 0, (name, line)
                seen.add(parts[1])
    assert "rmsnorm_bf16_16384x4096" in seen and "layernorm_bf16_16384x4096" in seen
    t = bench.traffic_from_profiles("rmsnorm_bf16_16384x4096")
    f, b = bench.algorithmic_bytes("rms", 16384, 4096, 2, 2)
    assert t is not None and t["source"].startswith("profiles/") and b <= t["bytes"] < 1.1 * b
    assert bench.traffic_from_profiles("layernorm_f32_200x128_quickstart") is None
    assert bench.traffic_fields("no_such_workload") == {"traffic": None}


def test_committed_width_scan_is_readable():
    """`bench.py --scan` compares itself with the committed table, and the GPU throughput guard reads it: every storage
    type and the guarded widths must parse."""
    import bench
    table = bench.scan_reference()
    assert len(table) >= 140
    for key in (("bf16", 72), ("bf16", 4096), ("bf16", 4098), ("f32", 256), ("f16", 6000)):
        assert key in table and all(20.0 < v < 100.0 for v in table[key]), key
