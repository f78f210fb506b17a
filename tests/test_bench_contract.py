"""bench.py's command-line contract, checked without a GPU: more than one GPU is refused with a message, and the
per-kernel tables (traffic per launch, rocprofv3 kernel names) name the same launches."""

import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                          timeout=120)
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr
    assert proc.stdout.strip() == ""  # no JSON line for a run that measured nothing


def test_kernel_tables_agree():
    sys.path.insert(0, ROOT)
    import bench

    assert set(bench.TRAFFIC_BYTES_PER_LAUNCH) == set(bench.ROCPROF_KERNEL)
    assert all(v > 0 for v in bench.TRAFFIC_BYTES_PER_LAUNCH.values())
    # the headline workload is configs[2] of the baseline: T=16,384, H=4096, E=8, top-2, I=14,336
    assert (bench.T, bench.H, bench.E, bench.TOP_K, bench.I) == (16384, 4096, 8, 2, 14336)
    assert 18.0 * bench.T * bench.TOP_K * bench.H * bench.I == 34634616274944.0
