"""The benchmark's command-line contract, as far as it can be checked without a GPU."""
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and not r.stdout.strip()


def test_help_lists_the_workloads():
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--help"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0
    for w in ("decode9b", "smallm", "moe", "qvb8r", "lmhead"):
        assert w in r.stdout


def test_metric_names_of_the_decode_step():
    sys.path.insert(0, str(ROOT))
    import bench
    assert bench.decode_metric_name("9b") == "dequant-GEMV HBM GB/s (% of peak) + decode tokens/s, 9B-shape pack, 1 MI355X"
    assert "27B-shape" in bench.decode_metric_name("27b")
