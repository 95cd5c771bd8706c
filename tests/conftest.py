"""Shared fixtures.  `ref` is the CPU checker (oracle/libnc_ref.so); `hip` is
the product library on the GPU.  Only tests may load the checker."""
import importlib.util
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
REF_LIB = os.path.join(ROOT, "oracle", "libnc_ref.so")


def load_pkg():
    """The package directory name holds a hyphen, so it is loaded by path."""
    name = "nncp_metal_amd"
    if name in sys.modules:
        return sys.modules[name]
    spec = importlib.util.spec_from_file_location(
        name, os.path.join(ROOT, "nncp-metal_amd", "__init__.py"),
        submodule_search_locations=[os.path.join(ROOT, "nncp-metal_amd")])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_runtest_setup(item):
    """Names every GPU test on the real stderr, flushed, before it touches the card: if a run
    ends without a report, the last such line says which case was on the GPU."""
    if item.get_closest_marker("gpu") is not None:
        capture = item.config.pluginmanager.getplugin("capturemanager")
        with capture.global_and_fixture_disabled():   # past pytest's capture of file descriptor 2
            sys.stderr.write("[gpu] %s\n" % item.nodeid)
            sys.stderr.flush()


@pytest.fixture(scope="session")
def pkg():
    return load_pkg()


@pytest.fixture(scope="session", autouse=True)
def library_runtime_first(request):
    """Whenever a GPU test is selected, the product library's HIP runtime is brought up before
    the first test runs.  torch bundles a HIP runtime of its own (its autograd engine counts the
    devices at its first backward pass); of two runtimes in one process the one that
    initialises second finds no device, and the library then ends the process
    ("no HIP device 0 (found 0)").  Done here, no test can let torch's copy come up first,
    whatever it does before it asks for the library."""
    if any(item.get_closest_marker("gpu") is not None for item in request.session.items):
        lib = hip_lib_path(load_pkg())
        if not os.path.exists(lib):
            pytest.fail("%s is missing: build it first (there is no fallback path)" % lib)
        import ctypes
        nc = ctypes.CDLL(lib, mode=ctypes.RTLD_LOCAL)
        nc.nc_context_init.restype = ctypes.c_void_p
        nc.nc_new_cuda_device.restype = ctypes.c_void_p
        nc.nc_new_cuda_device.argtypes = [ctypes.c_void_p, ctypes.c_int]
        nc.nc_context_end.argtypes = [ctypes.c_void_p]
        ctx = nc.nc_context_init(1)
        nc.nc_new_cuda_device(ctx, 0)
        nc.nc_context_end(ctx)
    yield


@pytest.fixture()
def ref(pkg):
    if not os.path.exists(REF_LIB):
        pytest.fail("oracle/libnc_ref.so missing: run `make -C oracle`")
    nc = pkg.binding.NC(REF_LIB, use_device=False, nb_threads=4)
    yield nc
    nc.close()


def hip_lib_path(pkg):
    """The product library, or - for tests/test_kernels_on_cpu.py, which re-runs the GPU
    op tests without a GPU - the same sources built for the host (tests/hipcpu)."""
    return os.environ.get("NNCP_TEST_HIP_LIB") or pkg.binding.HIP_LIB


@pytest.fixture()
def hip(pkg):
    nc = pkg.binding.NC(hip_lib_path(pkg), use_device=True)
    yield nc
    nc.close()


@pytest.fixture()
def rng():
    return np.random.default_rng(1234)
