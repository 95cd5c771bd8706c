"""Parameter files of the host mirror (nc_save_coefs / nc_load_coefs, libnc.h:530, 536) on
the CPU checker; the GPU side of the same round trip is in tests/test_gpu_zz_new_paths.py."""
import os

import numpy as np

import modelutil as M


def test_parameter_file_round_trip_on_the_checker(tmp_path):
    """nc_save_coefs / nc_load_coefs (libnc.h:530, 536): a trained model's parameters
    written to a file and read into a freshly initialised model of the same configuration
    are the same bits, and the two models then evaluate identically; a file that is not a
    parameter file, or that names a parameter the model lacks, ends the process with a
    message (libnc's error model), which a child process shows."""
    import subprocess, sys, textwrap
    pkg = M.load_pkg()
    cfg = dict(M.TINY)
    a = pkg.host.Model(M.ref_host(), pkg.host.make_config(**dict(cfg, use_device=0, nb_threads=2, sgd_opt=M.rmsprop(3e-3))))
    syms = M.markov1(cfg["batch_size"] * cfg["seg_len"] * 3, cfg["n_symbols"], seed=5)
    for tok, tgt in M.segment_batches(syms, cfg["batch_size"], cfg["seg_len"], 3):
        a.train_step(tok, tgt, 3e-3)
    path = tmp_path / "coefs.bin"
    a.save_coefs(str(path))
    b = pkg.host.Model(M.ref_host(), pkg.host.make_config(**dict(cfg, seed=99, use_device=0, nb_threads=2, sgd_opt=M.rmsprop(3e-3))))
    assert any(not np.array_equal(a.get_param(n), b.get_param(n)) for n in a.param_names())
    b.load_coefs(str(path))
    for n in a.param_names():
        assert np.array_equal(a.get_param(n), b.get_param(n)), n
    # file layout as documented: magic, version, empty configuration, first record's name
    raw = path.read_bytes()
    assert raw[:4] == b"NCPF" and int.from_bytes(raw[4:8], "little") == 1 and int.from_bytes(raw[8:12], "little") == 0
    nl = int.from_bytes(raw[12:16], "little")
    assert raw[16:16 + nl].decode() == a.param_names()[0]
    a.close(); b.close()
    bad = tmp_path / "bad.bin"
    bad.write_bytes(b"not a parameter file")
    code = textwrap.dedent('''
        import sys; sys.path.insert(0, %r)
        import modelutil as M
        pkg = M.load_pkg()
        m = pkg.host.Model(M.ref_host(), pkg.host.make_config(**dict(M.TINY, use_device=0, nb_threads=1)))
        m.load_coefs(%r)
    ''') % (os.path.dirname(os.path.abspath(__file__)), str(bad))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "not a parameter file" in r.stderr
