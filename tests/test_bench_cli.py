"""bench.py's command line: one GPU only, and helpers that need no GPU."""
import importlib.util
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert res.returncode != 0
    assert "one GPU" in res.stderr and "--gpus 1" in res.stderr


def test_visible_pairs_of_work_items():
    spec = importlib.util.spec_from_file_location("bench", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    assert bench.visible_pairs((0, 128, 0, 256, -1, 0)) == 128 * 256          # no mask
    assert bench.visible_pairs((0, 128, 0, 128, 0, 0)) == 128 * 129 // 2      # plain diagonal
    assert bench.visible_pairs((64, 64, 0, 128, 64, 0)) == 64 * 64 + 64 * 65 // 2   # diagonal shifted by 64 keys
    # published peaks the roofline is priced against
    assert bench.PEAK_TFLOPS == {"bf16": 2500.0, "fp16": 2500.0} and bench.PEAK_HBM_GBS == 8000.0
