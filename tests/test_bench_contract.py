"""bench.py's command-line contract, as far as it can be checked without a GPU."""
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]


def test_more_than_one_gpu_is_refused_with_a_message():
    run = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert run.returncode != 0
    assert "one GPU" in run.stderr


def test_roofline_constants_match_the_published_peaks():
    sys.path.insert(0, str(ROOT))
    import bench

    assert bench.PEAK_FP32_MFMA_TFLOPS == 157.3 and bench.PEAK_HBM_GBS == 8000.0
    # 2 m n k of the eight products of one wide-MLP step: three forward, two input-gradient, three weight-gradient
    assert abs(bench.gemm_flops_per_step(bench.WIDE_DIMS, bench.WIDE_BATCH) - 790.274e9) < 1e6


def test_gemm_traffic_comes_from_the_committed_counter_summary(tmp_path):
    """roofline.traffic is whatever profiles/gemm_kernel_wide_mlp_step_hbm_traffic.txt states, never a literal."""
    sys.path.insert(0, str(ROOT))
    import re

    import bench

    text = bench.GEMM_TRAFFIC_PROFILE.read_text()
    got = bench.gemm_traffic_bytes_per_launch()
    stated_mb = float(re.search(r"([\d.]+) MB per launch on average", text).group(1))
    assert got is not None and abs(got / 1e6 - stated_mb) < 0.06
    # per-variant rows of the same file: launches-weighted mean of fetch + write, in MiB, gives the same figure
    rows = re.findall(r"n=\s*(\d+)\s+fetch\s+([\d.]+) MiB\s+write\s+([\d.]+) MiB", text)
    n = sum(int(r[0]) for r in rows)
    mean = sum(int(r[0]) * (float(r[1]) + float(r[2])) for r in rows) / n * 1024 * 1024
    assert abs(mean - got) / got < 2e-3
    alg = bench.gemm_bytes_per_step(bench.WIDE_DIMS, bench.WIDE_BATCH) / 8
    assert alg <= got <= 10 * alg
    assert bench.gemm_traffic_bytes_per_launch(tmp_path / "absent.txt") is None


def test_the_cpu_legs_of_the_small_configurations_run_on_the_oracle_device():
    """bench.py times the DQN update and the GCN step on the CPU oracle beside the GPU: the function that runs them must
    work with a device that launches nothing."""
    sys.path.insert(0, str(ROOT))
    import bench
    from oracle.oracle_device import OracleDevice

    for kind in ("dqn", "gcn"):
        out = bench.run_small(OracleDevice(), kind, 2, graph=False)
        assert out["ms_per_step"] > 0 and "launches_per_step" not in out
