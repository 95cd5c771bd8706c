"""Test infrastructure: builds tests/hipcpu/libnc_hipcpu.so, the product's own
csrc/ sources compiled for the HOST against the stand-in HIP runtime in this
directory (kernels run as fibers, device memory sits against guard pages).
Nothing in the product loads it; tests/test_kernels_on_cpu.py does."""
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "nncp-metal_amd", "csrc")
BUILD = os.path.join(HERE, "_build")
OUT = os.path.join(HERE, "libnc_hipcpu.so")
CXX = os.environ.get("HIPCPU_CXX", "/opt/rocm/llvm/bin/clang++")
SOURCES = ["k_gemm.hip", "k_elementwise.hip", "k_norm.hip", "k_attention.hip", "k_attn_fused.hip", "k_attn_bf16.hip", "k_cdf.hip",
           "nc_core.cpp", "nc_autodiff.cpp", "nc_ops.cpp", "nc_params_io.cpp"]
NO_CONTRACT = {"k_cdf.hip", "nc_ops.cpp"}
FLAGS = ["-x", "c++", "-std=c++17", "-O1", "-g", "-fPIC", "-fno-strict-aliasing", "-Wno-unknown-attributes",
         "-Wno-unused-function", "-Wno-unused-value", "-Wno-array-bounds", "-I", HERE, "-iquote", CSRC]
# the dynamic LDS array of a kernel becomes a pointer to the launch's guarded buffer
DYN_LDS = re.compile(r"extern\s+__shared__\s+__attribute__\(\(aligned\(16\)\)\)\s+(\w+)\s+(\w+)\[\];")
# occupancy hints mean nothing to the host compiler (and it rejects them on plain functions)
GPU_ATTR = re.compile(r"__attribute__\(\(amdgpu_waves_per_eu\([^)]*\)\)\)")


def _compile(name):
    text = open(os.path.join(CSRC, name)).read()
    text = DYN_LDS.sub(r"\1 *\2 = (\1 *)hipcpu_dynamic_lds();", text)
    text = GPU_ATTR.sub("", text)
    src = os.path.join(BUILD, name + ".cpp")
    open(src, "w").write('#line 1 "%s"\n' % os.path.join(CSRC, name) + text)
    obj = os.path.join(BUILD, name + ".o")
    extra = ["-ffp-contract=off"] if name in NO_CONTRACT else []
    r = subprocess.run([CXX] + FLAGS + extra + ["-c", src, "-o", obj], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("host compile of %s failed:\n%s" % (name, "\n".join(l for l in r.stderr.splitlines() if "error" in l or "note" in l)[-4000:]))
    return obj


def up_to_date():
    """The library is newer than everything it is built from."""
    if not os.path.exists(OUT):
        return False
    inc = os.path.join(ROOT, "include")
    deps = [os.path.join(d, f) for d in (CSRC, inc, HERE, os.path.join(HERE, "hip")) for f in os.listdir(d)
            if f.endswith((".hip", ".cpp", ".h", ".py"))]
    return os.path.getmtime(OUT) > max(os.path.getmtime(f) for f in deps)


def build(jobs=8, force=False):
    if not force and up_to_date():
        return OUT
    os.makedirs(BUILD, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, SOURCES))
    rt = os.path.join(BUILD, "hipcpu_runtime.o")
    r = subprocess.run([CXX] + FLAGS + ["-c", os.path.join(HERE, "hipcpu_runtime.cpp"), "-o", rt],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("host compile of the runtime failed:\n" + "\n".join(l for l in r.stderr.splitlines() if "error" in l or "note" in l)[-4000:])
    r = subprocess.run([CXX, "-shared", "-fPIC", "-Wl,-Bsymbolic", "-o", OUT] + objs + [rt, "-lm"],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + "\n".join(l for l in r.stderr.splitlines() if "error" in l or "note" in l)[-4000:])
    return OUT


if __name__ == "__main__":
    print(build(force=True))
