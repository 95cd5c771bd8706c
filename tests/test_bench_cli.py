"""bench.py's command line, as far as it can be checked without a GPU."""
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and "--gpus 1" in r.stderr
    assert r.stdout.strip() == ""


def test_synthetic_stream_is_seeded_and_byte_valued():
    sys.path.insert(0, ROOT)
    import bench
    a = bench.markov3_dirichlet(5000)
    b = bench.markov3_dirichlet(5000)
    assert np.array_equal(a, b)
    assert a.min() >= 0 and a.max() <= 255 and len(a) == 5000
    # order-3 contexts with Dirichlet(0.05) rows: far from uniform, far from constant
    counts = np.bincount(a.astype(np.int64), minlength=256)
    assert (counts > 0).sum() > 32 and counts.max() < len(a) // 2
