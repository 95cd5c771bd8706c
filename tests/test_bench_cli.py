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
    (tmp_path / "two.txt").write_text(
        "gemm_kernel<128, 128, 64, 2, 2, 0, 1, 2, 1, 3, 1>    3   100.0   100.0   10.00   1.00\n"
        "gemm_kernel<128, 128, 64, 2, 2, 0, 1, 2, 1, 2, 1>    3   100.0   100.0   20.00   2.00\n")
    monkeypatch.setattr(bench, "PROFILES", str(tmp_path))
    monkeypatch.setattr(bench, "TRAFFIC_SUMMARY", {"fp32": "t.txt", "bf16": "absent.txt", "two": "two.txt"})
    # the event records name an instantiation by its leading template arguments
    traffic, source = bench.measured_traffic("gemm_kernel<128,128,32,4,2,0,1,0>", "fp32")
    assert traffic == (3254.78 + 151.52) * 1e6 and "t.txt" in source and "not re-measured" in source
    assert bench.measured_traffic("gemm_kernel<64,64,32,2,2,1,0,0>", "fp32")[0] == (28.10 + 4.19) * 1e6
    assert bench.measured_traffic("opt_update_multi_kernel", "fp32")[0] == (457.68 + 305.06) * 1e6
    assert bench.measured_traffic("gemm_kernel<64,64,32,2,2,0,1,0>", "fp32") == (None, None)
    # a leading argument list is not a prefix of a longer number (32 vs 320)
    assert bench.measured_traffic("gemm_kernel<128,128,3", "fp32") == (None, None)
    assert bench.measured_traffic("gemm_kernel<128,128,32,4,2,0,1,0>", "bf16") == (None, None)
    # two instantiations the record cannot tell apart: no figure rather than the first one
    assert bench.measured_traffic("gemm_kernel<128,128,64,2,2,0,1,2>", "two") == (None, None)
    # the grouped launch runs the same template: its record's mark is not part of the name
    assert bench.measured_traffic("gemm_kernel<128,128,32,4,2,0,1,0,grouped>", "fp32")[0] == traffic
    # the summary the repository holds covers the kernel the bench line names
    monkeypatch.undo()
    assert bench.measured_traffic("gemm_kernel<128,128,32,4,2,0,1,0>", "fp32")[0] > 1e9