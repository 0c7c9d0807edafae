"""What bench.py promises without a GPU: more than one GPU is refused with one line and exit code 2, and
the numbers its roofline fractions are made of (bytes a decode step must read, operations of a prompt)."""

import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]


def test_more_than_one_gpu_is_refused_with_one_line():
    done = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert done.returncode == 2
    lines = [l for l in done.stdout.splitlines() if l.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_step_sizes_of_the_headline_configuration():
    sys.path.insert(0, str(ROOT))
    import bench
    n = bench.model_numbers(bench.TINYLLAMA, 2)
    # 22 layers x 88.08 MB + 131 MB of head + float norm weights = 2.069 GB; 22,528 bytes of K/V per cached token
    assert abs(n["weight_bytes"] - 2.069e9) < 2e6
    assert n["kv_bytes_per_token"] == 22528
    # a 2048-token prompt: 3.969 TFLOP in the layers' products and the head row, 0.378 TFLOP of causal attention
    flops = bench.prefill_flops(bench.TINYLLAMA, 2048, 1)
    assert abs(flops - 4.347e12) < 0.01e12
    assert set(bench.MODELS) == {"tinyllama-1.1b", "llama-3.2-1b", "llama-3.2-3b", "llama-3.1-8b"}
