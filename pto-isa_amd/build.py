"""Builds libpto_amd.so (HIP kernels + C ABI) in-tree for gfx950.

    python pto-isa_amd/build.py

hipcc cross-compiles without a GPU.  The library has no dependency on PyTorch.
"""
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libpto_amd.so")
# libpto_st.so: the same sources with the tuning hooks compiled in (PTO_ST_HOOKS) plus the single-tile test programs; what
# the parity tests load to drive single instructions and kernel variants.  Not part of the product.
OUT_ST = os.path.join(HERE, "libpto_st.so")
SOURCES = ["pto_core.hip", "pto_gemm.hip", "pto_gemm_w4.hip", "pto_gemm_mx.hip", "pto_gemm_mxw4.hip", "pto_elementwise.hip", "pto_quant.hip", "pto_topk.hip", "pto_mla.hip", "pto_fa.hip", "pto_fa_w8.hip", "pto_fa_w8m16.hip"]
ST_ONLY_SOURCES = ["pto_optest.hip", "pto_optest_matmul.hip"]
# sources of libpto_st.so that differ from the product's objects (they hold a hook); the others are linked as they are
HOOK_SOURCES = ["pto_gemm.hip", "pto_gemm_w4.hip", "pto_gemm_mx.hip", "pto_fa.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
         # packed-fp32 VALU forms are kept off for every device function
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unknown-warning-option"]


def _compile(job):
    src, st = job
    obj = os.path.join(HERE, "build", ("st_" if st else "") + src.replace(".hip", ".o"))
    os.makedirs(os.path.dirname(obj), exist_ok=True)
    cmd = [HIPCC] + FLAGS + (["-DPTO_ST_HOOKS=1"] if st else []) + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj


def build(verbose=True):
    jobs = [(s, False) for s in SOURCES] + [(s, True) for s in HOOK_SOURCES + ST_ONLY_SOURCES]
    with ThreadPoolExecutor(max_workers=8) as ex:
        objs = dict(zip(jobs, ex.map(_compile, jobs)))
    product = [objs[(s, False)] for s in SOURCES]
    st = [objs[(s, s in HOOK_SOURCES)] for s in SOURCES] + [objs[(s, True)] for s in ST_ONLY_SOURCES]
    for out, group in ((OUT, product), (OUT_ST, st)):
        r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + group, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stderr)
        if verbose:
            print("built", out)
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


REFERENCE = os.environ.get("PTO_REFERENCE", "/root/reference")
# the reference's kernel sources compiled against this library's headers are the thing under test, not the checker: they are
# kept apart from oracle/_ref (the compiled reference that the oracle is pinned against)
PORTED_DIR = os.path.join(ROOT, "build", "ported")
# (library, reference source, constants rewritten for 160 KiB of LDS, dynamic LDS bytes of the launch, further options)
PORTED = [
    ("libpto_ported_gemm.so", "kernels/manual/a2a3/gemm_performance/gemm_performance_kernel.cpp",
     [("stepKa", "1"), ("stepKb", "1")], 160 * 1024, {}),
    # the flash-attention kernel: Cube and Vec roles in one workgroup (both __DAV_* families defined), one Vec core per
    # Cube core, single-buffered Q / K / P / V panels (128 KiB of LDS), Vec tiles in the unified buffer in memory
    ("libpto_ported_fa.so", "kernels/manual/common/flash_atten/fa_performance_kernel.cpp",
     [("VEC_CORES", "1"), ("MAX_VEC_UB_BYTES", "512U * 1024U"), ("kMatTNBuffers", "1"), ("pMatTNBuffers", "1"), ("vMatTNBuffers", "1")],
     128 * 1024,
     dict(defines=("__DAV_CUBE__", "__DAV_VEC__", "__DAV_C220_CUBE__", "__DAV_C220_VEC__"), vec_in_memory=True,
          extra_includes=(os.path.join(HERE, "host", "port_cases"),), extra_flags=("-Wno-unknown-attributes",))),
    # the top-k kernel: every tile a Vec tile at an address of the unified buffer, re-viewed through tiles of other shapes
    ("libpto_ported_topk.so", "kernels/manual/a2a3/topk/topk_kernel.cpp", [], 0,
     dict(vec_in_memory=True, extra_flags=("-Wno-unknown-attributes",))),
    # the MXFP8 matmul kernel (e5m2 operands, e8m0 block scales, bf16 output): one K-128 step per L1 panel instead of four
    ("libpto_ported_mxfp8.so", "kernels/manual/a5/matmul_mxfp8_performance/mxmatmul_performance_kernel.cpp",
     [("stepKa", "1"), ("stepKb", "1")], 160 * 1024, dict(extra_flags=("-Wno-unknown-attributes",))),
    # the MXFP4 matmul kernel (e2m1 operands, m = 2040 and n = 8100 through run-time valid extents of its Mat, operand, scale
    # and accumulator tiles): one K-256 step per L1 panel instead of two
    ("libpto_ported_mxfp4.so", "kernels/manual/a5/matmul_mxfp4_performance/mxmatmul_performance_kernel.cpp",
     [("stepKa", "1"), ("stepKb", "1")], 160 * 1024, dict(extra_flags=("-Wno-unknown-attributes",))),
]


def port_and_compile(rel_src, sets, lds_bytes, out, extra_flags=(), extra_includes=(), defines=(), vec_in_memory=False, l1_map=None):
    """Runs a kernel source of the reference through port_ascend_source.py into a temporary directory and compiles the
    result against include/pto with hipcc; `out` ends in .o (compile only) or .so.  The ported text never enters the
    repository tree."""
    import importlib.util
    import tempfile
    spec = importlib.util.spec_from_file_location("port_ascend_source", os.path.join(HERE, "port_ascend_source.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    src = os.path.join(REFERENCE, rel_src)
    with open(src) as f:
        text, _ = mod.port(f.read(), sets, lds_bytes, defines, os.path.dirname(src), vec_in_memory, l1_map)
    with tempfile.TemporaryDirectory() as tmp:
        hip = os.path.join(tmp, os.path.basename(rel_src).replace(".cpp", ".hip"))
        with open(hip, "w") as f:
            f.write(text)
        mode = ["-c"] if out.endswith(".o") else ["-shared"]
        cmd = [HIPCC] + FLAGS + ["-I" + os.path.dirname(src)] + ["-I" + i for i in extra_includes] + list(extra_flags) + mode + [hip, "-o", out]
        r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    return r.returncode, err


def build_ported(verbose=True):
    """The reference's own kernel sources compiled against this library's headers (only where the reference tree is
    mounted; the libraries go to build/ported/, which is kept out of the history)."""
    if not os.path.isdir(REFERENCE):
        return
    os.makedirs(PORTED_DIR, exist_ok=True)
    for lib, rel_src, sets, lds, opts in PORTED:
        out = os.path.join(PORTED_DIR, lib)
        rc, err = port_and_compile(rel_src, sets, lds, out, **opts)
        if rc != 0:
            raise RuntimeError("ported build failed for %s:\n%s" % (rel_src, err))
        if verbose:
            print("built", out)


# The reference's host programs (main.cpp beside each manual kernel: Ascend runtime calls, the file protocol, ResultCmp),
# compiled where they lie against this library's runtime shim (include/acl/acl.h, include/pto/host/test_common.h) and linked
# with the ported kernel library that holds their launcher: build/ported/host/<name>.
PORTED_HOSTS = [
    ("gemm_performance_main", "kernels/manual/a2a3/gemm_performance/main.cpp", "pto_ported_gemm"),
    ("matmul_mxfp8_performance_main", "kernels/manual/a5/matmul_mxfp8_performance/main.cpp", "pto_ported_mxfp8"),
    ("matmul_mxfp4_performance_main", "kernels/manual/a5/matmul_mxfp4_performance/main.cpp", "pto_ported_mxfp4"),
    ("topk_main", "kernels/manual/a2a3/topk/main.cpp", "pto_ported_topk"),
    # the flash-attention program takes its case list from generated_cases.h (written by the reference's build from a
    # case string; here the list the ported kernel library is built with) and runs the cases named with --case=
    ("flash_atten_main", "kernels/manual/common/flash_atten/main.cpp", "pto_ported_fa"),
]


def build_ported_hosts(verbose=True):
    if not os.path.isdir(REFERENCE):
        return
    out_dir = os.path.join(PORTED_DIR, "host")
    os.makedirs(out_dir, exist_ok=True)
    for name, rel_src, lib in PORTED_HOSTS:
        out = os.path.join(out_dir, name)
        cmd = ["g++", "-O2", "-std=c++17", "-w", "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "include", "pto", "host"),
               "-I/opt/rocm/include", "-I" + os.path.dirname(os.path.join(REFERENCE, rel_src)), "-I" + os.path.join(HERE, "host", "port_cases"),
               "-D__HIP_PLATFORM_AMD__", os.path.join(REFERENCE, rel_src), "-o", out,
               "-L" + PORTED_DIR, "-l" + lib, "-Wl,-rpath,$ORIGIN/..", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("host program build failed for %s:\n%s" % (rel_src, r.stderr))
        if verbose:
            print("built", out)


# Per-instruction test kernels of the reference (tests/npu/a2a3/src/st/testcase/<op>/<op>_kernel.cpp) that tests/st_ref_cases.py
# runs on the GPU: each compiled unchanged (register tiles; no constant rewritten) into build/ported/st/<op>.so.
# build/ported/st/manifest.json holds, per test, the launcher symbols (mangled -> demangled, so that the tests need no
# binutils) and, for sources whose launchers are numbered cases (`launch<OP>Case<N>` kernels that fix the template arguments
# of one run function each), the table case number -> [run function, template arguments] read from the source.
ST_KERNELS = ["tabs", "tneg", "tnot", "texp", "tlog", "tsqrt", "trsqrt", "trecip", "trelu", "tmov_vect", "tsub", "tmul", "tdiv", "tadd",
              "tand", "tor", "tshl", "tshr", "tprelu", "taddplus", "tfmod", "trem", "txor", "tands", "tors", "txors", "tshls", "tshrs",
              "tadds", "tsubs", "tmuls", "tdivs", "tmaxs", "tfmods", "trems", "tlrelu",
              "tcolsum", "tcolmax", "tcolmin", "tcolprod", "trowexpand",
              "trowexpandadd", "trowexpandsub", "trowexpandmul", "trowexpanddiv", "trowexpandmax", "trowexpandmin", "trowexpandexpdif",
              "tcolexpandadd", "tcolexpandsub", "tcolexpandmul", "tcolexpanddiv", "tcolexpandmax", "tcolexpandmin", "tcolexpandexpdif",
              "tcmp", "tcmps", "tsel", "ttri", "trowsum", "trowmax", "trowmin", "tcvt", "tmatmul", "textract",
              "tmax", "tmin", "tmins", "texpands", "tsels", "tsort32", "tgather", "tmrgsort", "tstore",
              "tcolexpand", "ttrans", "trowprod", "tpartadd", "tpartmul", "tpartmax", "tpartmin", "tmov_acc2mat", "tstore_acc2gm", "tfillpad", "tquant", "tdequant", "tscatter", "tgatherb", "tstore_mat2gm", "tci", "tload",
              "a5_tadd_tdiv", "a5_tmul_tadds", "a5_tmuls_trowsum", "a5_trowsum_trowexpand", "a5_trowexpand_tdiv", "a5_trowexpand_tsqrt",
              "a5_trowexpand_trowsum", "a5_tsub_texp", "a5_mgather", "a5_mscatter", "a5_tpack", "a5_trowexpandbrcb", "a5_tpartmul", "a5_tfmods", "a5_tmov_vect"]
_ST_CASE = re.compile(r"void\s+launch\w+?Case(\d+)\s*\(([^)]*)\)\s*\{\s*(\w+)\s*<([^;{}]*?)>\s*\(")
_ST_KEYED = re.compile(r"(?:tilingKey|testKey)\s*==\s*(\d+)\s*\)\s*\{\s*(\w+)\s*<([^;{}]*?)>\s*<<<[^;]*?>>>\s*\(([^;]*)\)\s*;")
_ST_LAUNCHER = re.compile(r"^void\s+(\w+)\s*\(", re.M)
_ST_KEYED_KERNEL = re.compile(r"(?:tilingKey|testKey)\s*==\s*(\d+)\s*\)\s*\{\s*(\w+)\s*<<<")
_ST_KERNEL_BODY = re.compile(r'extern "C" __global__ AICORE void (\w+)\([^)]*\)\s*\{(.*?)\n\}', re.S)
# options of the port script per test kernel: L1 addresses written for Ascend's 512 KiB moved inside the LDS
ST_PORT_OPTIONS = {
    "tmatmul": dict(l1_map={0x20000: 0x10000, 0x40000: 0x1C000}),
    # four of its 46 kernels keep 64 + 128 KiB of fp32 tiles in L1: they end at their TASSIGN and are not run
    "textract": dict(defines=["PTO_TASSIGN_BEYOND_LDS_ENDS_KERNEL"]),
}
# its top-k kernel works through Vec tiles that are views of one another (TASSIGN to the same address)
ST_PORT_OPTIONS["tmrgsort"] = dict(vec_in_memory=True)
# the NPU form of TSCATTER (indices are element numbers of the destination; the CPU simulation's are row numbers)
ST_PORT_OPTIONS["tscatter"] = dict(defines=["PTO_TSCATTER_FLAT_INDEX"])
# the NPU form of TREM / TREMS (the sign of the divisor; the CPU simulation's % / fmod take the dividend's)
ST_PORT_OPTIONS["trem"] = dict(defines=["PTO_TREM_FLOOR_FORM"])
ST_PORT_OPTIONS["trems"] = dict(defines=["PTO_TREM_FLOOR_FORM"])
# three of its kernels keep more than 160 KiB of L1 tiles: they end at their TASSIGN and are not run
ST_PORT_OPTIONS["tstore_mat2gm"] = dict(defines=["PTO_TASSIGN_BEYOND_LDS_ENDS_KERNEL"])
# stores through a second tile object at the address of the one it loaded: tiles as addresses
ST_PORT_OPTIONS["tload"] = dict(vec_in_memory=True)
# multiplies in one function and declares the accumulator tile again, at the same address, in the next: tiles as addresses
ST_PORT_OPTIONS["tmov_acc2mat"] = dict(vec_in_memory=True, defines=["PTO_ACC_TILES_IN_MEMORY"])
# sources that keep their device code under the Ascend device compiler's own macro
for _name in ("tmax", "tmin", "tmins", "texpands"):
    ST_PORT_OPTIONS[_name] = dict(defines=["__CCE_AICORE__=220"])


def st_case_table(source_text):
    """{case: {"run": run function, "targs": [template arguments], "params": kernel parameter list, "args": the launch's
    arguments where the source writes them}} for the ways the
    test sources number their cases: `launch<OP>Case<N>` kernels (case = "N"), and launchers that switch on their template
    argument, `if constexpr (tilingKey == N) { run<...><<<` (case = "<launcher>:N")."""
    table = {}
    for m in _ST_CASE.finditer(source_text):
        table[m.group(1)] = {"run": m.group(3), "targs": [a.strip() for a in m.group(4).split(",")],
                             "params": " ".join(m.group(2).replace("__gm__", "").split())}
    launchers = [(m.start(), m.group(1)) for m in _ST_LAUNCHER.finditer(source_text)]
    for m in _ST_KEYED.finditer(source_text):
        owner = [name for pos, name in launchers if pos < m.start()]
        if owner:
            table["%s:%s" % (owner[-1], m.group(1))] = {"run": m.group(2), "targs": [a.strip() for a in m.group(3).split(",")], "params": "",
                                                        "args": " ".join(m.group(4).split())}
    # ... or `if constexpr (tilingKey == N) { kernel<<<`, the kernel fixing its case through local constants
    # (`constexpr uint32_t M = 64;`) that it hands to one run function: the constants and the run function's leading type
    # arguments are the case
    bodies = {m.group(1): m.group(2) for m in _ST_KERNEL_BODY.finditer(source_text)}
    for m in _ST_KEYED_KERNEL.finditer(source_text):
        owner = [name for pos, name in launchers if pos < m.start()]
        body = bodies.get(m.group(2))
        if not owner or body is None:
            continue
        run = re.search(r"(run\w+)\s*<([^;]*?)>\s*\(", body, re.S)
        if run is None:
            continue
        table["%s:%s" % (owner[-1], m.group(1))] = {
            "run": run.group(1), "targs": [a.strip() for a in run.group(2).split(",")], "params": "",
            "consts": {k: " ".join(v.split()) for k, v in re.findall(r"constexpr\s+\w+\s+(\w+)\s*=\s*([^;]+);", body)}}
    return table


def build_ported_st(verbose=True, jobs=8):
    import concurrent.futures
    import json
    if not os.path.isdir(REFERENCE):
        if verbose:
            print("reference tree not mounted: per-instruction test kernels not built")
        return
    out_dir = os.path.join(PORTED_DIR, "st")
    os.makedirs(out_dir, exist_ok=True)

    def one(name):
        # "a5_<op>": the test source of that name in the a5 tree (instruction sequences that the a2a3 tree does not have)
        arch, op = ("a5", name[3:]) if name.startswith("a5_") else ("a2a3", name)
        rel = "tests/npu/%s/src/st/testcase/%s/%s_kernel.cpp" % (arch, op, op)
        lib = os.path.join(out_dir, name + ".so")
        rc, err = port_and_compile(rel, [], 160 * 1024, lib, extra_flags=("-Wno-unknown-attributes",), **ST_PORT_OPTIONS.get(name, {}))
        if rc != 0:
            raise RuntimeError("ported build failed for %s:\n%s" % (rel, err))
        syms = subprocess.run(["nm", "-D", "--defined-only", lib], capture_output=True, text=True, check=True).stdout.split("\n")
        mangled = [l.split()[2] for l in syms if len(l.split()) == 3 and l.split()[1] in "TW"]
        demangled = subprocess.run(["c++filt"], input="\n".join(mangled), capture_output=True, text=True, check=True).stdout.split("\n")
        with open(os.path.join(REFERENCE, rel)) as f:
            table = st_case_table(f.read())
        return name, {"launchers": {m: d for m, d in zip(mangled, demangled) if d.startswith("void ") and "pto::" not in d.split("(")[0]},
                      "cases": table}
    manifest = {}
    with concurrent.futures.ThreadPoolExecutor(jobs) as ex:
        for name, entry in ex.map(one, ST_KERNELS):
            manifest[name] = entry
            if verbose:
                print("built", os.path.join(out_dir, name + ".so"), "(%d launchers)" % len(entry["launchers"]))
    with open(os.path.join(out_dir, "manifest.json"), "w") as f:
        json.dump(manifest, f, indent=1, sort_keys=True)


if __name__ == "__main__":
    build()
    build_ported()
    build_ported_hosts()
    build_ported_st()
    sys.exit(0)
