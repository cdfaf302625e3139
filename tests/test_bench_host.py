"""Host-side checks of bench.py that need no GPU: the byte model behind the reported GB/s and the
refusal of multi-GPU runs."""
import os
import subprocess
import sys

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_algorithmic_bytes_model():
    # 2 B of value + 4 bits of delta per stored entry, int32 row_ptr, the fp16 input and output vectors
    assert bench.algorithmic_bytes(0, 0, 0) == 4
    assert bench.algorithmic_bytes(8, 1, 32) == 16 + 4 + 8 + 64 + 2
    P, rows, cols = 8388720, 4096, 4096
    assert bench.algorithmic_bytes(P, rows, cols) == 2 * P + P // 2 + 4 * 4097 + 2 * 4096 + 2 * 4096
    assert bench.dense_bytes(4096, 11008) == 2 * 4096 * 11008 + 2 * 11008 + 2 * 4096


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       cwd=ROOT, timeout=300)
    assert r.returncode != 0
    assert "--gpus 1" in (r.stderr + r.stdout)
