"""The C-ABI library loads and exports every symbol the headers declare (no
compute: runs without a GPU)."""
import ctypes
import os
import re

from conftest import ROOT, load_pkg


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = set(re.findall(r"\b((?:nc_|nchip_)\w+|sgd_opt_update_var|vec_sum_f32)\s*\(", text))
    return names


def test_hip_library_exports_declared_symbols():
    pkg = load_pkg()
    lib = ctypes.CDLL(pkg.binding.HIP_LIB)
    missing = []
    for header in ("nc_api.h", "nc_ext.h", "nchip_kernels.h"):
        for name in sorted(_declared(header)):
            if not hasattr(lib, name):
                missing.append(name)
    assert not missing, missing


def test_checker_exports_the_same_abi():
    lib = ctypes.CDLL(os.path.join(ROOT, "oracle", "libnc_ref.so"))
    missing = [n for h in ("nc_api.h", "nc_ext.h") for n in sorted(_declared(h)) if not hasattr(lib, n)]
    assert not missing, missing


def test_binding_covers_the_link_set_of_the_reference_host():
    """The 90 symbols nncp.c + cp_utils.c leave undefined (nm -u on the objects
    compiled from the reference sources) must all be exported."""
    link_set = """nc_add nc_backward nc_cmul nc_combine_nodes nc_concat nc_concat_node
    nc_concat_optimization nc_context_end nc_context_init nc_convert nc_dup_node nc_dup_tensor
    nc_free nc_free_node nc_free_tensor nc_gated_swish nc_gelu nc_get_col nc_get_node
    nc_get_param_count nc_get_scalar_f32 nc_get_tensor_device nc_hconcat nc_indexed_log
    nc_layer_norm nc_lerp nc_lstm_clamped nc_malloc nc_mallocz nc_masked_fill nc_matmul
    nc_matmul_add nc_mul nc_new_cpu_device nc_new_cuda_device nc_new_f32 nc_new_param
    nc_new_scalar nc_new_tensor_1d nc_new_tensor_2d nc_new_tensor_3d nc_new_tensor_4d
    nc_new_tensor_from_tensor_nz nc_node_set_arg nc_node_set_parent nc_pad nc_param_list_end
    nc_param_list_init nc_permute nc_permute_4d nc_prof_dump nc_reduce_sum nc_rel_shift nc_relu
    nc_repeat_1d nc_repeat_2d nc_reshape_1d nc_reshape_2d nc_reshape_3d nc_reshape_4d
    nc_rms_norm nc_rnd_end nc_rnd_init nc_set1_i32_2d nc_sgd_opt_end nc_sgd_opt_init
    nc_sgd_opt_set_all nc_sgd_opt_set_lr nc_sgd_opt_update nc_sigmoid nc_slice nc_slice_alias
    nc_soft_max nc_split nc_sum nc_tanh nc_tensor_copy nc_tensor_copy_slice nc_tensor_get_dims
    nc_tensor_get_ptr nc_tensor_set_dropout nc_tensor_set_f32 nc_tensor_set_name
    nc_tensor_set_rnd_unif nc_tensor_set_zero nc_tensor_to_cpu_device nc_tensor_to_device
    nc_vconcat sgd_opt_update_var vec_sum_f32""".split()
    assert len(link_set) == 90
    pkg = load_pkg()
    for path in (pkg.binding.HIP_LIB, os.path.join(ROOT, "oracle", "libnc_ref.so")):
        lib = ctypes.CDLL(path)
        missing = [n for n in link_set if not hasattr(lib, n)]
        assert not missing, (path, missing)


def test_host_library_exports_declared_symbols():
    """include/nncp_host.h against the host library of the product and of the checker."""
    text = open(os.path.join(ROOT, "include", "nncp_host.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(nncp_\w+)\s*\(", text)))
    assert len(names) > 30
    pkg = load_pkg()
    for path in (pkg.host.HOST_HIP_LIB, os.path.join(ROOT, "oracle", "libnncp_host_ref.so")):
        lib = ctypes.CDLL(path)
        missing = [n for n in names if not hasattr(lib, n)]
        assert not missing, (path, missing)


def test_host_loader_refuses_a_host_library_bound_to_another_libnc():
    """With the checker in the process-wide namespace the dynamic linker would hand its nc_*
    functions to the product's host library (a GPU run would then silently compute on the
    CPU): Host() must notice and refuse.  Run in a child process, whose namespace it spoils."""
    import subprocess
    import sys
    code = ("import sys, ctypes; sys.path.insert(0, %r); from conftest import load_pkg, REF_LIB;"
            "pkg = load_pkg(); ctypes.CDLL(REF_LIB, mode=ctypes.RTLD_GLOBAL)\n"
            "try:\n    pkg.host.Host()\nexcept RuntimeError as e:\n    print('refused:', e); sys.exit(0)\n"
            "sys.exit(1)") % (os.path.join(ROOT, "tests"),)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True)
    assert r.returncode == 0 and "bound to another libnc" in r.stdout, r.stdout + r.stderr
    # and the plain pairing loads
    pkg = load_pkg()
    pkg.host.Host()
    pkg.host.Host(os.path.join(ROOT, "oracle", "libnncp_host_ref.so"), os.path.join(ROOT, "oracle", "libnc_ref.so"))
