"""CPU-only checks of the pieces a driver calls: bench.py's argument contract and the two entry points."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu_before_touching_one():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "one GPU" in r.stderr and not r.stdout.strip()


def test_entry_points_exist():
    sys.path.insert(0, ROOT)
    import __graft_entry__ as g
    assert callable(g.build) and callable(g.smoke)


def test_bench_reads_the_committed_traffic_figure():
    sys.path.insert(0, ROOT)
    import bench
    t, fresh = bench.profiled_traffic("conv_wide<64, 64,", 3, "fp32")
    assert t is not None and 5e6 < t < 1e8                      # bytes per launch, from profiles/
    assert isinstance(fresh, bool)                              # whether profiles/ was collected on this kernel source
    assert bench.profiled_traffic("no_such_kernel", 3, "fp32")[0] is None
    assert len(bench.kernel_source_hash()) == 12
