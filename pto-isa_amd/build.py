"""Builds libpto_amd.so (HIP kernels + C ABI) in-tree for gfx950.

    python pto-isa_amd/build.py

hipcc cross-compiles without a GPU.  The library has no dependency on PyTorch.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libpto_amd.so")
SOURCES = ["pto_core.hip", "pto_gemm.hip", "pto_gemm_w8.hip", "pto_gemm_m16.hip", "pto_gemm_m16w4.hip", "pto_gemm_mx.hip", "pto_elementwise.hip", "pto_topk.hip", "pto_mla.hip", "pto_fa.hip", "pto_fa_w8.hip", "pto_fa_w8m16.hip", "pto_optest.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
         # packed-fp32 VALU forms are kept off for every device function
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unknown-warning-option"]


def _compile(src):
    obj = os.path.join(HERE, "build", src.replace(".hip", ".o"))
    os.makedirs(os.path.dirname(obj), exist_ok=True)
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj


def build(verbose=True):
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT] + objs, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", OUT)
    build_host(verbose)
    return OUT


def build_host(verbose=True):
    """The `call_kernel` libraries of the two demos and the GEMM and flash-attention host programs; plain host C++ on top of libpto_amd.so."""
    inc = ["-I" + os.path.join(ROOT, "include"), "-I/opt/rocm/include", "-D__HIP_PLATFORM_AMD__"]
    link = ["-L" + HERE, "-lpto_amd", "-Wl,-rpath,$ORIGIN"]
    jobs = [
        (["-shared", "-fPIC", os.path.join(CSRC, "call_kernel_gemm.cpp")], os.path.join(HERE, "libpto_call_gemm.so"), link),
        (["-shared", "-fPIC", os.path.join(CSRC, "call_kernel_fa.cpp")], os.path.join(HERE, "libpto_call_fa.so"), link),
        ([os.path.join(HERE, "host", "gemm_main.cpp")], os.path.join(HERE, "host", "gemm_main"),
         ["-L" + HERE, "-lpto_amd", "-Wl,-rpath,$ORIGIN/..", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"]),
        ([os.path.join(HERE, "host", "fa_main.cpp")], os.path.join(HERE, "host", "fa_main"),
         ["-L" + HERE, "-lpto_amd", "-Wl,-rpath,$ORIGIN/..", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"]),
    ]
    for srcs, out, libs in jobs:
        cmd = ["g++", "-O2", "-std=c++17"] + inc + srcs + ["-o", out] + libs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("host build failed for %s:\n%s" % (out, r.stderr))
        if verbose:
            print("built", out)


if __name__ == "__main__":
    build()
    sys.exit(0)
