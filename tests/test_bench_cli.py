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


def test_traffic_is_read_from_the_committed_counter_summary(tmp_path, monkeypatch):
    sys.path.insert(0, ROOT)
    import bench
    (tmp_path / "t.txt").write_text(
        "header line with words and 1 2 3\n"
        "kernel                                   n FETCH_SIZE KiB WRITE_SIZE KiB    read MB   write MB\n"
        "gemm_kernel<128, 128, 32, 4, 2, 0, 1, 0, 1, 2, 0>    3   1589431.1   147968.0   3254.78   151.52\n"
        "gemm_kernel<64, 64, 32, 2, 2, 1, 0, 0, 2, 4, 0>    147     13722.4     4096.0     28.10     4.19\n"
        "opt_update_multi_kernel                              3    223500.0   297914.0    457.68   305.06\n")
    monkeypatch.setattr(bench, "PROFILES", str(tmp_path))
    # the event records name an instantiation by its leading template arguments
    assert bench.measured_traffic("gemm_kernel<128,128,32,4,2,0,1,0>", "t.txt") == (3254.78 + 151.52) * 1e6
    assert bench.measured_traffic("gemm_kernel<64,64,32,2,2,1,0,0>", "t.txt") == (28.10 + 4.19) * 1e6
    assert bench.measured_traffic("opt_update_multi_kernel", "t.txt") == (457.68 + 305.06) * 1e6
    assert bench.measured_traffic("gemm_kernel<64,64,32,2,2,0,1,0>", "t.txt") is None
    assert bench.measured_traffic("gemm_kernel<128,128,32,4,2,0,1,0>", "absent.txt") is None
    # the summary the repository holds covers the kernel the bench line names
    monkeypatch.undo()
    assert bench.measured_traffic("gemm_kernel<128,128,32,4,2,0,1,0>") > 1e9
