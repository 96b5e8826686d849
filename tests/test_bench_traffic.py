"""bench.py reports `roofline.traffic` from the committed rocprofv3 summaries, not from constants:
the numbers it would print must be the ones in profiles/*.txt."""
import os
import re
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def _table():
    out = {}
    pdir = os.path.join(ROOT, "profiles")
    for name in sorted(os.listdir(pdir)):
        if not name.endswith(".txt"):
            continue
        text = open(os.path.join(pdir, name)).read()
        # every summary states the command that produced it, and that command runs bench.py
        assert re.search(r"rocprofv3 .* -- python3 bench\.py", text), name
        for w, k, v in re.findall(r"^traffic (\S+) (\S+) (\d+)$", text, flags=re.M):
            out.setdefault(w, {})[k] = float(v)
    return out


def test_bench_reads_the_traffic_the_profiles_hold():
    import bench
    table = _table()
    assert "headline" in table
    for w in bench.WORKLOADS:
        assert w in table, "no rocprofv3 summary under profiles/ covers workload %s" % w
        got = bench.measured_traffic(w)
        assert got == table[w]
        for key in ("k_gemm", "k_normmap_a", "k_normmap_b"):
            assert got[key] > 0


def test_traffic_is_at_least_the_bytes_the_kernels_must_move():
    # C is written once by the GEMM (4 N^2 bytes) and each conversion pass reads its fp32 matrix once
    import bench
    for w, (N, tile, *_rest) in bench.WORKLOADS.items():
        t = bench.measured_traffic(w)
        assert t["k_gemm"] >= 4.0 * N * N
        assert t["k_normmap_a"] >= 4.0 * N * N and t["k_normmap_b"] >= 4.0 * N * N
        assert t["k_normmap_b"] <= 6.1 * N * N                 # nothing re-read: at most read + full fp16 copy


def test_unknown_workload_has_no_traffic():
    import bench
    assert bench.measured_traffic("no_such_workload") == {}
