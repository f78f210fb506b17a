"""bench.py's command-line contract, checked without a GPU: more than one GPU is refused with a message, the workload
constants are the baseline's, and the HBM-traffic figure of the roofline record is taken from a counter summary by
kernel name (and is null for a kernel the summary does not hold)."""

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


def test_traffic_is_matched_by_kernel_name(tmp_path):
    sys.path.insert(0, ROOT)
    import bench

    summary = tmp_path / "traffic.txt"
    summary.write_text(
        "# comment\n"
        "void ck::(anonymous namespace)::grouped_gemm_line_kernel<__hip_bfloat16, 4, 256, true, 2, false>(ck::GemmParams)\t40\t1000.0\t24.0\n"
        "void ck::(anonymous namespace)::grouped_gemm_line_kernel<__hip_bfloat16, 2, 256, false, 2, true>(ck::GemmParams)\t20\t5.0\t5.0\n"
    )
    assert bench.traffic_for("grouped_gemm_dw_rows", str(summary)) == 1024.0 * 1024.0
    assert bench.traffic_for("grouped_gemm<swiglu>", str(summary)) is None  # the summary holds another instantiation
    assert bench.traffic_for("no such launch", str(summary)) is None
    assert bench.traffic_for("grouped_gemm_dw_rows", str(tmp_path / "missing.txt")) is None


def test_workload_is_the_baselines():
    sys.path.insert(0, ROOT)
    import bench

    # the headline workload is configs[2] of the baseline: T=16,384, H=4096, E=8, top-2, I=14,336
    assert (bench.T, bench.H, bench.E, bench.TOP_K, bench.I) == (16384, 4096, 8, 2, 14336)
    assert 18.0 * bench.T * bench.TOP_K * bench.H * bench.I == 34634616274944.0
