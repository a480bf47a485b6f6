"""The C++ boundary as a drop-in: kernel sources of the reference compile against include/pto with hipcc for gfx950
after the mechanical edits of pto-isa_amd/port_ascend_source.py (device-code brackets, the launch statement, tile-size
constants that fit 160 KiB of LDS), and the mistakes a port can make are compile errors, not wrong results.

The reference sources are read where they lie; the tests are skipped where the reference tree is not mounted.  Nothing
here needs a GPU: hipcc cross-compiles."""
import importlib.util
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "pto-isa_amd")


def _build_mod():
    spec = importlib.util.spec_from_file_location("pto_amd_build", os.path.join(PKG, "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


B = _build_mod()
needs_reference = pytest.mark.skipif(not os.path.isdir(B.REFERENCE), reason="reference tree not mounted")
GEMM_SRC = "kernels/manual/a2a3/gemm_performance/gemm_performance_kernel.cpp"


def _hipcc_snippet(tmp_path, body, defines=()):
    src = tmp_path / "snippet.hip"
    src.write_text(body)
    cmd = [B.HIPCC] + B.FLAGS + ["-D" + d for d in defines] + ["-c", str(src), "-o", str(tmp_path / "snippet.o")]
    r = subprocess.run(cmd, capture_output=True, text=True)
    return r.returncode, r.stderr


@needs_reference
def test_reference_gemm_kernel_compiles(tmp_path):
    """gemm_performance_kernel.cpp with stepKa = stepKb = 1 (two 16 KiB A panels and two 32 KiB B panels in LDS)."""
    rc, err = B.port_and_compile(GEMM_SRC, [("stepKa", "1"), ("stepKb", "1")], 160 * 1024, str(tmp_path / "gemm.o"))
    assert rc == 0, err


@needs_reference
def test_reference_gemm_kernel_with_its_own_l1_sizes_is_a_compile_error(tmp_path):
    """Unchanged, the kernel TASSIGNs 384 KiB of L1: the build stops with a [PTO][SA] message instead of overrunning LDS."""
    rc, err = B.port_and_compile(GEMM_SRC, [], 160 * 1024, str(tmp_path / "gemm.o"))
    assert rc != 0 and "[PTO][SA] TASSIGN" in err and "160 KiB" in err, err


@needs_reference
def test_reference_flash_attention_kernel_compiles(tmp_path):
    """fa_performance_kernel.cpp with its stage macros (pto_macro_matmul / _fa_softmax / _fa_gu.hpp, inlined by the port
    script), runTFA and LaunchTFA for the committed case list: the options of build_ported()."""
    lib, rel_src, sets, lds, opts = [p for p in B.PORTED if p[0] == "libpto_ported_fa.so"][0]
    rc, err = B.port_and_compile(rel_src, sets, lds, str(tmp_path / "fa.o"), **opts)
    assert rc == 0, err


@needs_reference
def test_reference_topk_kernel_compiles(tmp_path):
    """topk_kernel.cpp as it is (no constant rewritten): TSORT32 / TMRGSORT / TGATHER on Vec tiles that are views of the
    unified buffer, launchTopk<float>."""
    lib, rel_src, sets, lds, opts = [p for p in B.PORTED if p[0] == "libpto_ported_topk.so"][0]
    assert sets == []
    rc, err = B.port_and_compile(rel_src, sets, lds, str(tmp_path / "topk.o"), **opts)
    assert rc == 0, err


@needs_reference
def test_reference_mxfp8_matmul_kernel_compiles(tmp_path):
    """mxmatmul_performance_kernel.cpp of a5/matmul_mxfp8_performance with stepKa = stepKb = 1 (its own four K-steps per L1
    panel need 384 KiB): scale panels as boxed Mat tiles, TileLeftScale / TileRightScale, GetScaleAddr, TMATMUL_MX, tiles by
    value."""
    lib, rel_src, sets, lds, opts = [p for p in B.PORTED if p[0] == "libpto_ported_mxfp8.so"][0]
    rc, err = B.port_and_compile(rel_src, sets, lds, str(tmp_path / "mx.o"), **opts)
    assert rc == 0, err


@needs_reference
def test_reference_mxfp4_matmul_kernel_compiles(tmp_path):
    """mxmatmul_performance_kernel.cpp of a5/matmul_mxfp4_performance with stepKa = stepKb = 1: e2m1 Mat / Left / Right
    tiles, TileLeftScaleCompact / TileRightScaleCompact, every tile with run-time valid extents set by assigning a
    temporary `TileT(validRows, validCols)` to a TASSIGNed tile."""
    lib, rel_src, sets, lds, opts = [p for p in B.PORTED if p[0] == "libpto_ported_mxfp4.so"][0]
    rc, err = B.port_and_compile(rel_src, sets, lds, str(tmp_path / "mx4.o"), **opts)
    assert rc == 0, err


def test_assigning_a_temporary_tile_keeps_the_address(tmp_path):
    """`tile = TileT(vr, vc)` on a TASSIGNed Mat tile takes the valid extents and keeps the address (host-side check of the
    tile object; the reference's MXFP4 kernel re-shapes its tiles this way per block)."""
    src = tmp_path / "assign.hip"
    src.write_text("""
#include <pto/pto-inst.hpp>
#include <cstdio>
using namespace pto;
int main()
{
    using T = Tile<TileType::Mat, half, 64, 64, BLayout::ColMajor, -1, -1, SLayout::RowMajor>;
    T a(64, 64), b(64, 64);
    a.S().lds = 4096; a.S().bound = true;
    a = T(17, 33);
    if (a.GetValidRow() != 17 || a.GetValidCol() != 33 || a.S().lds != 4096u) { std::printf("moved: %u\\n", a.S().lds); return 1; }
    b.S().lds = 8192; b.S().bound = true;
    a = b;                      // a named, TASSIGNed tile: the address comes along
    if (a.S().lds != 8192u) return 2;
    std::printf("ok\\n");
    return 0;
}
""")
    exe = tmp_path / "assign"
    r = subprocess.run([B.HIPCC, "--offload-arch=gfx950", "-std=c++17", "-I" + os.path.join(ROOT, "include"), str(src), "-o", str(exe)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0 and "ok" in r.stdout, (r.returncode, r.stdout, r.stderr)


def test_port_script_rewrites():
    """The mechanical edits on a synthetic source: launch statement, function-local static, kernel prologue, brackets."""
    spec = importlib.util.spec_from_file_location("port_ascend_source", os.path.join(PKG, "port_ascend_source.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    src = """#include <pto/pto-inst.hpp>
using namespace pto;
constexpr int kSize = 512;
AICORE inline int counter()
{
    static int calls = 0;
    static uint64_t ticks = 7;
    return ++calls + (int)ticks;
}
__global__ AICORE void kern(__gm__ float *out)
{
    out[0] = counter();
}
void Launch(float *out, void *stream)
{
    kern<<<4, nullptr, stream>>>(out);
}
"""
    text, notes = mod.port(src, [("kSize", "128")], 4096, ("__DAV_VEC__",), None, True)
    assert "constexpr int kSize = 128;" in text
    # statics are numbered in the order of the source, one LDS slot each
    assert "PTO_CORE_STATIC(int, calls, 0, 0);" in text and "PTO_CORE_STATIC(uint64_t, ticks, 7, 1);" in text
    assert "PTO_KERNEL_PROLOGUE();" in text
    many = src.replace("    static int calls = 0;\n", "".join("    static int c%d = 0;\n" % i for i in range(32)) + "    int calls = 0;\n")
    with pytest.raises(SystemExit, match="33 function-local statics"):
        mod.port(many, [("kSize", "128")], 4096, ("__DAV_VEC__",), None, True)
    # an innermost loop over Cube / Vec role blocks becomes one loop per block; loops with anything else in the body, or whose
    # blocks hold loops themselves, stay
    roles = """#include <pto/pto-inst.hpp>
__global__ AICORE void k(__gm__ float *o)
{
    for (int t = 0; t < 4; ++t) {
        int next = t + 1;
        for (int s = 0; s < 2; ++s) {
            if constexpr (DAV_CUBE) {
                o[0] += s;
            }
            if constexpr (DAV_VEC) {
                o[1] += next;
            }
            if constexpr (DAV_CUBE) {
                o[2] += t;
            }
        }
        if constexpr (DAV_VEC) {
            o[3] += 1;
        }
    }
    for (int p = 0; p < 4; ++p) {
        if constexpr (DAV_CUBE) {
            for (int s = 0; s < 2; ++s)
                o[4] += s;
        }
        if constexpr (DAV_VEC) {
            o[5] += p;
        }
    }
}
"""
    text2, notes2 = mod.port(roles, [], 4096, ("DAV_CUBE=1", "DAV_VEC=1"), None, True)
    assert any("1 loop over Cube / Vec role blocks split" in n for n in notes2), notes2
    assert text2.count("for (int s = 0; s < 2; ++s) {") == 3 and text2.count("for (int p = 0; p < 4; ++p) {") == 1
    cube0, vec1, cube2 = text2.index("o[0] += s;"), text2.index("o[1] += next;"), text2.index("o[2] += t;")
    assert cube0 < text2.index("for (int s = 0; s < 2; ++s) {", cube0) < vec1 < text2.index("for (int s = 0; s < 2; ++s) {", vec1) < cube2
    assert "<<<pto::host::LaunchBlocks(4, (hipStream_t)(stream)), pto::kBlockThreads, pto::host::LaunchLds((const void *)(kern), 4096), (hipStream_t)(stream)>>>" in text
    assert "__global__ __launch_bounds__(pto::kBlockThreads) AICORE void kern" in text
    assert text.startswith("#define PTO_TILE_COPY_WRITEBACK 1\n#define PTO_VEC_TILES_IN_MEMORY 1\n#define __DAV_VEC__ 1\n")
    begin, end, launch = text.index("PTO_DEVICE_CODE_BEGIN"), text.index("PTO_DEVICE_CODE_END"), text.index("void Launch")
    assert begin < text.index("AICORE inline int counter") and text.index("void kern") < end < launch
    # the kernel expression in front of a launch: plain, with template arguments, with a name pasted by a macro call
    # (tests/npu/a5/src/st/testcase/tmuls_trowsum/tmuls_trowsum_kernel.cpp:59-63) - each gets its static LDS taken off
    for expr in ("kern", "ns::kern<float, 4>", "CONCAT(run, CASENAME)<half, kRows, kCols>"):
        line = "    %s<<<1, nullptr, stream>>>(out);" % expr
        assert mod.kernel_before(line, line.index("<<<")) == expr
    asm = 'uint64_t t; asm volatile("MOV %0, SYS_CNT\\n" : "+l"(t)); asm volatile("MOV %0, PC\\n" : "+l"(pc));'
    assert mod.ASCEND_SREG_READ.sub(lambda m: "%s = %s;" % (m.group(2), "get_sys_cnt()" if m.group(1) == "SYS_CNT" else "0"), asm) == \
        "uint64_t t; t = get_sys_cnt(); pc = 0;"


SNIPPET = r"""
#include <hip/hip_runtime.h>
#include <pto/pto-inst.hpp>
#include <pto/common/constants.hpp>
#include <pto/common/utils.hpp>
#include <pto/common/pto_tile.hpp>
#include <pto/common/memory.hpp>
#include <pto/common/type.hpp>
using namespace pto;
PTO_DEVICE_CODE_BEGIN
template <typename AccT, typename LeftT, typename RightT>
AICORE inline void ByValue(AccT c, LeftT a, RightT b) { TMATMUL(c, a, b); }
__global__ void k(float *out, half *src)
{
    using MatA = Tile<TileType::Mat, half, 128, 64, BLayout::ColMajor, 128, 64, SLayout::RowMajor>;
    using MatB = Tile<TileType::Mat, half, 64, 256, BLayout::RowMajor, 64, 256, SLayout::ColMajor>;
    MatA am; MatB bm;
    TASSIGN(am, 0x0);
    TASSIGN(bm, 0x0 + 128 * 64 * 2);
    MatA am2 = am;               // Mat tiles are handles: copies are fine
    TileLeft<half, 128, 64> a; TileRight<half, 64, 256> b; TileAcc<float, 128, 256> c;
    GlobalTensor<half, pto::Shape<1, 1, 1, 128, 64>, pto::Stride<1, 1, 1, 64, 1>> ga(src);
    GlobalTensor<half, pto::Shape<1, 1, 1, 64, 256>, pto::Stride<1, 1, 1, 1, 64>, Layout::DN> gb(src + 128 * 64);
    TLOAD(am2, ga); TLOAD(bm, gb);
    set_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0); wait_flag(PIPE_MTE2, PIPE_MTE1, EVENT_ID0);
    TEXTRACT(a, am, 0, 0); TEXTRACT(b, bm, 0, 0);
    ByValue(c, a, b);
    GlobalTensor<float, pto::Shape<1, 1, 1, 128, 256>, pto::Stride<1, 1, 1, 256, 1>> gc(out);
    TSTORE(gc, c);
    static_assert(CeilDivision(7, 2) == 4 && CeilAlignment(7, 4) == 8, "utils.hpp");
}
PTO_DEVICE_CODE_END
"""


def test_register_tile_by_value_is_a_compile_error(tmp_path):
    rc, err = _hipcc_snippet(tmp_path, SNIPPET)
    assert rc != 0 and "[PTO][SA] a register tile" in err, err


def test_register_tile_by_value_compiles_in_write_back_mode(tmp_path):
    """With PTO_TILE_COPY_WRITEBACK the spelling of gemm_performance_kernel.cpp:28 is accepted (the copy hands its
    values back to the tile it was copied from)."""
    rc, err = _hipcc_snippet(tmp_path, SNIPPET, defines=["PTO_TILE_COPY_WRITEBACK=1"])
    assert rc == 0, err


MOVED_MAT = r"""
#include <hip/hip_runtime.h>
#include <pto/pto-inst.hpp>
using namespace pto;
PTO_DEVICE_CODE_BEGIN
template <typename ChunkT, typename WholeT>
AICORE inline void Chunks(ChunkT &chunk, WholeT &whole, half *src)
{
    GlobalTensor<half, pto::Shape<1, 1, 1, 128, 64>, pto::Stride<1, 1, 1, 64, 1>> g(src);
    for (int k = 0; k < KCHUNKS; ++k) {
        TASSIGN(chunk, (uint64_t)whole.data() + k * 128 * 64 * 2);
        TLOAD(chunk, g);
    }
}
__global__ void k(half *src)
{
    using Whole = Tile<TileType::Mat, half, 128, 128, BLayout::ColMajor, 128, 128, SLayout::RowMajor>;
    using Chunk = Tile<TileType::Mat, half, 128, 64, BLayout::ColMajor, 128, 64, SLayout::RowMajor>;
    Whole w; Chunk c;
    TASSIGN(w, 0x0);
    Chunks(c, w, src);
}
PTO_DEVICE_CODE_END
"""


def test_mat_tile_moved_through_data_pointer_is_a_compile_error(tmp_path):
    """The walk of pto_macro_matmul.hpp:176-177 (one Mat tile re-addressed to data() + k * chunk bytes): accepted for one
    chunk (offset 0 of the image is the image), stopped at compile time for two."""
    rc, err = _hipcc_snippet(tmp_path, MOVED_MAT, defines=["KCHUNKS=1"])
    assert rc == 0, err
    rc, err = _hipcc_snippet(tmp_path, MOVED_MAT, defines=["KCHUNKS=2"])
    assert rc != 0 and "[PTO][SA] TASSIGN: a Mat tile that has an address is moved" in err, err


VEC_BEYOND = r"""
#include <hip/hip_runtime.h>
#include <pto/pto-inst.hpp>
using namespace pto;
PTO_DEVICE_CODE_BEGIN
__global__ void k(float *out)
{
    Tile<TileType::Vec, float, 64, 64, BLayout::RowMajor, 64, 64> t;
    TASSIGN(t, VEC_ADDR);
    TEXPANDS(t, 1.0f);
    GlobalTensor<float, pto::Shape<1, 1, 1, 64, 64>, pto::Stride<1, 1, 1, 64, 1>> g(out);
    TSTORE(g, t);
}
PTO_DEVICE_CODE_END
"""


def test_vec_tile_beyond_unified_buffer_is_a_compile_error(tmp_path):
    """A Vec tile in the unified buffer has to end inside the workgroup's share of it (512 KiB), and below the accumulator
    images (from 256 KiB) when those live there too."""
    ok = ["PTO_VEC_TILES_IN_MEMORY=1", "VEC_ADDR=0x7C000"]          # ends at 512 KiB exactly
    rc, err = _hipcc_snippet(tmp_path, VEC_BEYOND, defines=ok)
    assert rc == 0, err
    rc, err = _hipcc_snippet(tmp_path, VEC_BEYOND, defines=["PTO_VEC_TILES_IN_MEMORY=1", "VEC_ADDR=0x7C040"])
    assert rc != 0 and "[PTO][SA] TASSIGN: the Vec tile ends beyond" in err, err
    rc, err = _hipcc_snippet(tmp_path, VEC_BEYOND, defines=ok + ["PTO_ACC_TILES_IN_MEMORY=1"])
    assert rc != 0 and "[PTO][SA] TASSIGN: the Vec tile ends beyond" in err, err


def test_forwarding_headers_exist():
    for name in ("pto_tile.hpp", "memory.hpp", "type.hpp", "utils.hpp", "pto_instr.hpp", "constants.hpp", "event.hpp"):
        assert os.path.exists(os.path.join(ROOT, "include", "pto", "common", name)), name
