"""Builds csrc/libnc_hip.so for gfx950 with hipcc (cross-compiles without a
GPU).  Usage: python nncp-metal_amd/build.py [-j N]"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
SOURCES = {
    "k_gemm.hip": [], "k_elementwise.hip": [], "k_norm.hip": [], "k_attention.hip": [], "k_attn_fused.hip": [], "k_attn_bf16.hip": [],
    # bit-exact integer-CDF path: no contraction, no reassociation
    "k_cdf.hip": ["-ffp-contract=off"],
    "nc_core.cpp": ["-x", "hip"], "nc_autodiff.cpp": ["-x", "hip"], "nc_params_io.cpp": ["-x", "hip"],
    "nc_ops.cpp": ["-x", "hip", "-ffp-contract=off"],
}


def _compile(item):
    src, extra = item
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + COMMON + extra + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    msgs = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, msgs))
    return obj, msgs


def build_hip(jobs=8, verbose=False):
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, SOURCES.items()))
    objs = [o for o, _ in results]
    if verbose:
        for _, msgs in results:
            if msgs.strip():
                print(msgs)
    out = os.path.join(CSRC, "libnc_hip.so")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,-Bsymbolic", "-o", out] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return out


if __name__ == "__main__":
    print(build_hip(verbose=True))
