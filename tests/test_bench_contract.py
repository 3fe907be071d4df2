"""bench.py pieces that can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert out.returncode != 0
    assert "one GPU" in (out.stderr + out.stdout)


def test_workload_parsing_and_algorithmic_bytes():
    sys.path.insert(0, ROOT)
    import bench
    w = bench.parse_workload("square:8192")
    assert (w["m"], w["n"], w["k"]) == (8192, 8192, 8192)
    w = bench.parse_workload("decode:11008x4096x16")
    assert (w["m"], w["k"], w["n"]) == (11008, 4096, 16)
    # 1.5 bits per weight + fp16 B + fp16 D: the decode figure quoted with the metric
    assert bench.algorithmic_bytes(11008, 16, 4096, 0.0) == 8937472
    assert bench.algorithmic_bytes(11008, 4, 4096, 0.0) == 8574976
    assert bench.algorithmic_bytes(11008, 1, 4096, 0.0) == 8484352
    assert bench.parse_workload("prefill")["beta"] == 1.0
    assert abs(bench.SMFMAC_PEAK_TFLOPS - 5033.1648) < 1e-6
