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
