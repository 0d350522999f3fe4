"""Throughput guard between the points the launch rules were fitted on: forward + backward of one batch at a handful
of row widths must stay within reach of the committed width scan (profiles/norm_step_width_scan_bf16_f16_f32.txt,
the output of `bench.py --scan`).  The bound is loose on purpose -- 0.75 of the committed figure: boxes differ by a
few per cent, a launch rule that picks a wrong shape costs 20 to 50 -- and the widths are the ones a rule boundary sits
next to: narrow rows on and off powers of two, the flat and staged kernels, rows off the 128-bit path (narrow and wide), the widest one-row shapes.
Collected late (the file name sorts behind the parity tests): it says nothing about correctness."""
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

pytestmark = pytest.mark.gpu

GUARDED = {
    "bf16": [50, 72, 128, 197, 200, 640, 1024, 2048, 4096, 4098, 6000, 8192, 16384],
    "f32": [50, 72, 256, 1536, 4096],
}
FLOOR = 0.75


@pytest.mark.parametrize("dname", sorted(GUARDED))
def test_step_throughput_stays_within_reach_of_the_committed_scan(dname):
    import bench
    from TritonHub import _native
    reference = bench.scan_reference()
    assert reference, "the committed scan table is missing or unreadable"
    lib = _native.lib()
    dev = torch.device("cuda", 0)
    dtype = {"bf16": torch.bfloat16, "f32": torch.float32}[dname]
    total = 1 << 26
    gen = torch.Generator(device=dev).manual_seed(0)
    pool = bench.scan_pool(dev, dtype, total, gen)
    behind = []
    try:
        for n in GUARDED[dname]:
            assert (dname, n) in reference, f"{dname} N={n} is not in the committed table"
            for ln in (False, True):
                print(f"[scan guard] {dname} N={n} {'LayerNorm' if ln else 'RMSNorm'}", flush=True)
                got = bench.scan_cell(lib, dev, pool, total // n, n, dtype, ln, 20, gen)
                want = reference[(dname, n)][int(ln)]
                if got < FLOOR * want:
                    behind.append(f"{dname} N={n} {'LayerNorm' if ln else 'RMSNorm'}: {got:.1f} % of the HBM peak, "
                                  f"committed scan {want:.1f} %")
    finally:
        del pool
        torch.cuda.empty_cache()
    assert not behind, "; ".join(behind)
