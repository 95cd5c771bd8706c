"""The product's kernels without a GPU.  tests/hipcpu builds csrc/ for the host
against a stand-in HIP runtime: work-items are fibers, wavefront shuffles and
the three MFMA instructions follow their documented lane layouts, and device
memory and dynamic LDS end at guard pages, so an out-of-range access is a
SIGSEGV at the faulting statement.  The GPU parity tests are then re-run
against that build: same kernel sources, same checks, on the CPU.  (The
float results of libm's tanhf / expf differ in the last bit from the GPU's,
which is why one tolerance-marginal model case is left to the GPU run.)"""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EMU_DIR = os.path.join(ROOT, "tests", "hipcpu")
EMU_LIB = os.path.join(EMU_DIR, "libnc_hipcpu.so")
EMU_HOST = os.path.join(EMU_DIR, "libnncp_host_hipcpu.so")


@pytest.fixture(scope="module")
def emulated():
    sys.path.insert(0, EMU_DIR)
    try:
        import build as hipcpu_build
        hipcpu_build.build()
    finally:
        sys.path.remove(EMU_DIR)
    # (rebuilt only when a source is newer; a stale library cannot pass for a fresh one)
    r = subprocess.run(["make", "LIBNC_DIR=../../tests/hipcpu", "LIBNC=nc_hipcpu", "OUT=" + EMU_HOST,
                        "RPATH=$$ORIGIN"], cwd=os.path.join(ROOT, "nncp-metal_amd", "host"),
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    return dict(os.environ, NNCP_TEST_HIP_LIB=EMU_LIB, NNCP_TEST_HOST_HIP_LIB=EMU_HOST)


# Largest shapes of three op tests: a minute or minutes each as fibers, and the same kernels and code paths as
# the smaller shapes of the same tests that do run here (the GPU run has all of them)
OPS_LEFT_TO_THE_GPU = ("not (k_major_weight_copies and (512-2048-32 or 1024-1024-33 or 2048-512-32)) and "
                       "not (few_column_products and (512-2048-32 or 2048-512-32)) and "
                       "not (embedding_gradient and 16384-64-4096)")


def _pytest(env, args):
    return subprocess.Popen([sys.executable, "-m", "pytest", "-q", "-m", "gpu", "-p", "no:cacheprovider"] + args,
                            cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)


def test_gpu_parity_tests_pass_on_the_cpu_build(emulated):
    """The op-level GPU tests (all op cases forward and backward, GEMM shapes in
    fp32 / bf16 / bf16 from rounded copies, fused and batched-GEMM attention up to
    256 keys, integer CDF and lookup bit-exactness, optimiser, ...) and a
    model-level subset (training steps against the checker op by op and fused,
    whole-model gradient, cached per-timestep logits bit-identical, a profile
    variant, the retrain pass, the LSTM model class and a file through the container), with
    guard pages behind every device buffer."""
    ops = _pytest(emulated, ["-n", "4", "tests/test_gpu_ops.py", "-k", OPS_LEFT_TO_THE_GPU])
    model = _pytest(emulated, ["-n", "2", "tests/test_gpu_model.py", "-k",
                               "(test_training_steps_match_checker and TINY) or "
                               "(test_cached_timestep_logits_are_bit_identical and SMALL32) or "
                               "test_gradients_match_checker_c1 or "
                               "(test_profile_variants_match_checker and 1-relu_coef)"])
    # (of the three file-container cases one runs here: fibers make the others minutes long)
    # (and the full-size round trip is hours of fibers: it waits for the GPU)
    new = _pytest(emulated, ["-n", "6", "tests/test_gpu_zz_new_paths.py", "-k",
                             "not (file_container and (reference or bf16)) and not full_size and "
                             "not (properties_small and bf16) and not 100_steps and not enwik8_profile and "
                             "not (memory_window and 0)"])
    out_ops, out_model = ops.communicate(timeout=1500)[0], model.communicate(timeout=1500)[0]
    out_new = new.communicate(timeout=1500)[0]
    assert ops.returncode == 0, out_ops[-3000:]
    assert model.returncode == 0, out_model[-3000:]
    assert new.returncode == 0, out_new[-3000:]
    assert " passed" in out_ops and " passed" in out_model and " passed" in out_new and "skipped" not in out_new


def test_results_do_not_depend_on_work_item_order(emulated):
    """The op-level tests again with the work-items of every workgroup, and the workgroups of
    every launch, run from the last to the first (HIPCPU_ORDER=reverse).  Between two
    barriers any order is one the hardware may pick, so a kernel that is missing a barrier
    (or whose workgroups rely on one another) gives different results here."""
    p = _pytest(dict(emulated, HIPCPU_ORDER="reverse"), ["-n", "7", "tests/test_gpu_ops.py", "-k", OPS_LEFT_TO_THE_GPU])
    out = p.communicate(timeout=1500)[0]
    assert p.returncode == 0 and " passed" in out, out[-3000:]


def test_bf16_operand_paths_pass_on_the_cpu_build(emulated):
    """The products that read bf16 operand copies (every tile class and transposition, the
    grouped launch, the copies the epilogues and norms write), the tensor-level shadow route
    with its consistency checker on, and attention on the bf16 matrix cores forward and
    backward - the unguarded 16-byte loads and the transposed LDS tiles of these kernels are
    exactly what guard pages behind every buffer are for."""
    p = _pytest(emulated, ["-n", "7", "tests/test_gpu_bf16_operands.py"])
    out = p.communicate(timeout=1500)[0]
    assert p.returncode == 0 and " passed" in out, out[-3000:]


def test_host_tensor_compute_is_refused(emulated):
    """No CPU fallback in the product library: compute on a host tensor aborts with a
    message.  (Host-side logic, so it is exercised on the CPU build and not by aborting
    a process that holds the GPU.)"""
    code = ("import sys, os; sys.path.insert(0, %r); from conftest import load_pkg; import numpy as np;"
            "B = load_pkg().binding; nc = B.NC(os.environ['NNCP_TEST_HIP_LIB'], use_device=True);"
            "a = nc.tensor(np.ones((2, 2), np.float32), device=nc.cpu);"
            "nc.nc_add(a, nc.dup(a))") % (os.path.join(ROOT, "tests"),)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=emulated)
    assert r.returncode != 0 and "GPU only" in r.stderr


def test_malformed_parameter_files_end_with_a_message(emulated, tmp_path):
    """The product's own reader of parameter files (csrc/nc_params_io.cpp) against the malformed
    records of tests/test_host_model.py: each ends in nc_fatal's message, none in a fault."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import test_host_model as T
    T.check_malformed_files_end_cleanly(
        tmp_path, "pkg.host.Host(%r, %r)" % (EMU_HOST, EMU_LIB), 1, env=emulated)


def test_token_outside_the_table_reads_nothing_and_ends_the_process_at_the_next_wait(emulated):
    """nc_get_col with an index >= the number of columns (and a negative one): the kernel reads
    nothing out of range (the guard pages of this build would end the process with SIGSEGV), the
    column comes out as zeros and the next wait ends the process with a message.  Through the
    raw entry point the flag is returned by nchip_index_error()."""
    code = ("import sys, os, ctypes as C; sys.path.insert(0, %r); from conftest import load_pkg; import numpy as np;"
            "B = load_pkg().binding; path = os.environ['NNCP_TEST_HIP_LIB']; nc = B.NC(path, use_device=True);"
            "lib = C.CDLL(path);"
            "w = nc.tensor(np.ones((5, 8), np.float32)); idx = nc.tensor(np.array([1, %s, 4], np.int32));"
            "y = nc.tensor(np.full((3, 8), 7.0, np.float32)); nc.nc_synchronize(nc.dev);"
            "p = lambda t: C.c_void_p(nc.lib.nc_tensor_get_ptr(t, None));"
            "assert lib.nchip_get_col(None, p(w), p(idx), p(y), 8, 5, C.c_int64(3)) == 0;"
            "lib.hipcpu_flush_copies();"
            "print('flag', lib.nchip_index_error(), lib.nchip_index_error());"
            "out = np.ctypeslib.as_array(C.cast(p(y), C.POINTER(C.c_float)), (3, 8));"
            "print('rows', out[0, 0], out[1].any(), out[2, 0]); sys.stdout.flush();"
            "z = nc.nc_get_col(w, idx); nc.numpy(z)")
    for bad in ("5", "-1"):
        r = subprocess.run([sys.executable, "-c", code % (os.path.join(ROOT, "tests"), bad)],
                           capture_output=True, text=True, env=emulated)
        assert "flag 1 0" in r.stdout and "rows 1.0 False 1.0" in r.stdout, (r.stdout, r.stderr[-2000:])
        assert r.returncode != 0 and "outside its table" in r.stderr, r.stderr[-2000:]


def test_random_shapes_stay_in_bounds_and_match(emulated):
    """Seeded random campaigns through the raw kernel entry points of the CPU build, each
    operand in an exact-size buffer ending at a guard page: GEMM (layouts, paddings, batches,
    split-K, fp32 / bf16 / bf16 from copies, forced tile configurations, epilogue options),
    attention (both generations, backward, single-query step), integer CDF and lookup; and
    through the tensor ABI, every op family forward and backward (broadcast forms, reductions,
    norms, softmax and log-likelihood, slicing / concatenation / permutation, padding, relative
    shift, embedding gather, linear layers with activations, the optimiser, views and copies)."""
    jobs = [("fuzz_gemm.py", "101", "150"), ("fuzz_gemm.py", "102", "150"), ("fuzz_attn.py", "103", "12"),
            ("fuzz_attn.py", "104", "12"), ("fuzz_cdf.py", "105", "25"),
            ("fuzz_ops.py", "106", "800")]
    procs = [subprocess.Popen([sys.executable, os.path.join(EMU_DIR, name), seed, count], env=emulated,
                              stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
             for name, seed, count in jobs]
    for job, p in zip(jobs, procs):
        out = p.communicate(timeout=1500)[0]
        assert p.returncode == 0 and out.strip().startswith("ok:"), (job, out[-3000:])
