"""The reference's own kernel sources, compiled against include/pto (pto-isa_amd/build.py: build_ported, only where the
reference tree is mounted; the libraries travel with the tree), run on the GPU and are held to the same bar as the
native kernels."""
import ctypes as C
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PORTED = os.path.join(ROOT, "build", "ported")

pytestmark = pytest.mark.gpu


def _ported(name):
    path = os.path.join(PORTED, name)
    if not os.path.exists(path):
        # a run that is meant to cover the ported kernels (PTO_REQUIRE_PORTED=1) must not pass without them
        assert os.environ.get("PTO_REQUIRE_PORTED") != "1", "%s is missing and PTO_REQUIRE_PORTED=1" % path
        pytest.skip("%s not built (reference tree absent at build time)" % name)
    return C.CDLL(path)


def test_reference_gemm_performance_kernel_6144(oracle):
    """gemm_performance_kernel.cpp (LaunchGEMME2E<uint16_t>, sizes fixed at m = n = k = 6144, 24 blocks), stepKa = stepKb
    = 1: every element against the native GEMM (tolerance 2e-3 of the largest |C|; both are fp32-accumulated MFMA sums
    in different orders), 8 rows against the oracle's port of the CPU simulation."""
    import torch
    import gpu_util as G
    from pto_amd import datagen
    lib = _ported("libpto_ported_gemm.so")
    fn = lib._Z13LaunchGEMME2EItEvPhS0_S0_Pv      # template void LaunchGEMME2E<uint16_t>(uint8_t*, uint8_t*, uint8_t*, void*)
    fn.argtypes = [C.c_void_p] * 4
    fn.restype = None
    m = n = k = 6144
    a, b = datagen.gemm_inputs(m, n, k)
    ta, tb = G.to_dev(a), G.to_dev(b)
    tc = torch.full((m, n), float("nan"), dtype=torch.float32, device=G.DEV)
    print("ported gemm launch", flush=True)
    fn(tc.data_ptr(), ta.data_ptr(), tb.data_ptr(), None)
    torch.cuda.synchronize()
    got = tc.cpu().numpy()
    native = G.gemm(a, b)
    scale = np.abs(native).max()
    assert np.isfinite(got).all()
    assert np.abs(got - native).max() <= 2e-3 * scale
    rows = np.array([0, 1, 127, 128, 1535, 1536, 4097, 6143])
    want = oracle.gemm_f16f32(a[rows], b, base_k=64)
    assert np.abs(got[rows] - want).max() <= 2e-3 * np.abs(want).max()


@pytest.mark.parametrize("S0,S1,causal,tile_s1,preload", [(128, 1024, False, 256, 4), (128, 2048, False, 256, 4),
                                                          (128, 8192, False, 256, 4), (512, 2048, False, 256, 4),
                                                          (256, 2048, True, 256, 2), (256, 2048, False, 128, 4),
                                                          (256, 1024, True, 128, 4), (512, 2048, True, 128, 2)])
def test_reference_flash_attention_kernel(oracle, S0, S1, causal, tile_s1, preload):
    """fa_performance_kernel.cpp: runTFA with its Cube / Vec stage functions, stage macros, TPipe FIFOs in global memory and
    Vec tiles as views of a unified buffer, launched through its own LaunchTFA<S0, 128, S1, 128, 128, TILE_S1, QK_PRELOAD, 8,
    false, CAUSAL, 4> with the workspace its host program allocates (main.cpp:126-207).  The first four cases are the
    reference generator's default schedule (score tiles of 256 keys made of two 128-wide cube tiles, preload 4) at 1024, 2048
    and 8192 keys.  O [S0, 128] fp32 against a dense
    float64 softmax (2e-3 of the largest |O|) and against the oracle's restatement of the streaming recurrence with the same
    key tile and the NPU's round-half-away cast of P (5e-4: rounding only).  Data as the reference's generator draws them
    (scripts/gen_data.py:26-35: seed 7, N(0,1) * 1.5 / 1.2 / 1)."""
    import torch
    lib = _ported("libpto_ported_fa.so")
    name = ("_Z9LaunchTFAILi%dELi128ELi%dELi128ELi128ELi%dELi%dELi8ELb0ELb%dELi4EEvPtS0_S0_S0_S0_PfS1_S1_S1_S1_S1_S1_P12ihipStream_tPh"
            % (S0, S1, tile_s1, preload, int(causal)))
    fn = getattr(lib, name)
    fn.restype, fn.argtypes = None, [C.c_void_p] * 14
    head, cube_s0, fifo = 128, 128, 8
    rng = np.random.default_rng(7)
    q = (rng.standard_normal((S0, head)) * 1.5).astype(np.float16)
    k = (rng.standard_normal((S1, head)) * 1.2).astype(np.float16)
    v = rng.standard_normal((S1, head)).astype(np.float16)
    dev = "cuda:0"
    tq, tk, tv = (torch.from_numpy(t.view(np.int16)).to(dev) for t in (q, k, v))
    blocks = S0 // cube_s0
    z = lambda n, dt: torch.zeros(n, dtype=dt, device=dev)
    ffts, p_fifo, expmax_fifo = z(64, torch.int16), z(blocks * fifo * cube_s0 * tile_s1, torch.int16), z(blocks * fifo * cube_s0, torch.float32)
    gsum, expmax, oparts = z(S0, torch.float32), z(S0, torch.float32), z(S0 * head, torch.float32)
    qk_fifo, pv_fifo = z(blocks * fifo * cube_s0 * tile_s1, torch.float32), z(blocks * fifo * cube_s0 * head, torch.float32)
    o = torch.full((S0, head), float("nan"), dtype=torch.float32, device=dev)
    print("ported flash attention launch", S0, S1, causal, flush=True)
    fn(ffts.data_ptr(), tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), p_fifo.data_ptr(), expmax_fifo.data_ptr(), gsum.data_ptr(),
       expmax.data_ptr(), o.data_ptr(), oparts.data_ptr(), qk_fifo.data_ptr(), pv_fifo.data_ptr(), None, None)
    torch.cuda.synchronize()
    got = o.cpu().numpy()
    s = q.astype(np.float64) @ k.astype(np.float64).T / np.sqrt(head)
    if causal:
        s = np.where(np.triu(np.ones((S0, S1), dtype=bool), 1), -np.inf, s)
    p = np.exp(s - s.max(axis=1, keepdims=True))
    want = (p / p.sum(axis=1, keepdims=True)) @ v.astype(np.float64)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= 2e-3 * np.abs(want).max()
    oo, _, _ = oracle.fa_stream_f16(q, k, v, tile_s1=tile_s1, causal=causal, q_offset=0, round_away=True)
    assert np.abs(got - oo).max() <= 5e-4 * np.abs(oo).max()


@pytest.mark.parametrize("ties", [False, True])
def test_reference_topk_kernel(oracle, ties):
    """topk_kernel.cpp (launchTopk<float>: 4800 rows of 1024 scores, row stride 1280, top 1000, 48 blocks): TLOAD -> TSORT32 ->
    TMRGSORT (one source with block lengths 64 and 256, then two lists merged in place) -> TMOV -> TGATHER P0101 / P1010 ->
    TSTORE, every tile a view of the unified buffer.  Scores and indices bit-exact against the native row sort and the
    oracle (the order of the reference's generator, scripts/gen_data.py:55-64: np.lexsort((idx, -row))[:topk]); data as the
    generator draws them, and with many equal scores (where TMRGSORT's order among equals -- list number, then position --
    and TSORT32's -- index -- agree because the indices increase with the column)."""
    import torch
    import gpu_util as G
    from pto_amd import capi, datagen
    lib = _ported("libpto_ported_topk.so")
    fn = lib._Z10launchTopkIfEvPhS0_S0_S0_Pv        # template void launchTopk<float>(uint8_t*, uint8_t*, uint8_t*, uint8_t*, void*)
    fn.argtypes, fn.restype = [C.c_void_p] * 5, None
    rows, cols, ld, k = 4800, 1024, 1280, 1000
    src, idx = datagen.topk_inputs(rows, cols, ld, distinct=37 if ties else 0)
    ts, ti = G.to_dev(src), G.to_dev(idx)
    out_s = torch.full((rows, k), float("nan"), dtype=torch.float32, device=G.DEV)
    out_i = torch.full((rows, k), -1, dtype=torch.int32, device=G.DEV)
    print("ported top-k launch", ties, flush=True)
    fn(out_s.data_ptr(), out_i.data_ptr(), ts.data_ptr(), ti.data_ptr(), None)
    torch.cuda.synchronize()
    got_s, got_i = out_s.cpu().numpy(), out_i.cpu().numpy().view(np.uint32)
    nat_s = torch.zeros((rows, k), dtype=torch.float32, device=G.DEV)
    nat_i = torch.zeros((rows, k), dtype=torch.int32, device=G.DEV)
    capi.check(capi.load().pto_topk_f32(G.stream(), nat_s.data_ptr(), nat_i.data_ptr(), ts.data_ptr(), ti.data_ptr(), rows, cols, ld, k), "topk")
    torch.cuda.synchronize()
    assert np.array_equal(got_s.view(np.uint32), nat_s.cpu().numpy().view(np.uint32))
    assert np.array_equal(got_i, nat_i.cpu().numpy().view(np.uint32))
    sel = np.array([0, 1, 2399, 4799])
    want_s, want_i = oracle.topk_f32(src[sel], idx, cols, k)
    assert np.array_equal(got_s[sel].view(np.uint32), want_s.view(np.uint32)) and np.array_equal(got_i[sel], want_i)


def test_reference_mxfp8_matmul_kernel(oracle):
    """mxmatmul_performance_kernel.cpp of a5/matmul_mxfp8_performance (LaunchMxMatmul: m = n = k = 6144, e5m2 operands, e8m0
    scales per 32 k, bf16 output, 32 blocks of 1536 x 768) with stepKa = stepKb = 1: TLOAD of operand and scale panels ->
    TEXTRACT -> TMATMUL_MX -> TSTORE.  Every element against the native MX GEMM (both round an fp32 sum of different
    order to bf16: one bf16 step of the largest |C| at most, and nearly all equal), 8 rows against the oracle."""
    import torch
    import gpu_util as G
    from pto_amd import capi, datagen
    lib = _ported("libpto_ported_mxfp8.so")
    fn = lib._Z14LaunchMxMatmulPhS_S_S_S_Pv         # void LaunchMxMatmul(uint8_t*, uint8_t*, uint8_t*, uint8_t*, uint8_t*, void*)
    fn.argtypes, fn.restype = [C.c_void_p] * 6, None
    m = n = k = 6144
    a, b, sa, sb = datagen.mx_inputs(m, n, k, 1)
    ta, tb, tsa, tsb = (torch.from_numpy(x).to(G.DEV) for x in (a, b, sa, sb))
    tc = torch.full((m, n), -1, dtype=torch.int16, device=G.DEV)
    print("ported mxfp8 launch", flush=True)
    fn(tc.data_ptr(), ta.data_ptr(), tb.data_ptr(), tsa.data_ptr(), tsb.data_ptr(), None)
    torch.cuda.synchronize()
    got = tc.view(torch.bfloat16).float().cpu().numpy()
    native = torch.zeros((m, n), dtype=torch.int16, device=G.DEV)
    capi.check(capi.load().pto_gemm_mxfp8(G.stream(), native.data_ptr(), ta.data_ptr(), tb.data_ptr(), tsa.data_ptr(), tsb.data_ptr(),
                                          m, n, k, 1, 0), "pto_gemm_mxfp8")
    torch.cuda.synchronize()
    nat = native.view(torch.bfloat16).float().cpu().numpy()
    assert np.isfinite(got).all()
    scale = np.abs(nat).max()
    assert np.abs(got - nat).max() <= scale * 2.0 ** -7
    assert np.mean(got == nat) > 0.99
    rows = np.array([0, 127, 128, 1535, 1536, 3000, 4607, 6143])
    want = oracle.mx_gemm(a[rows], b, sa[rows], sb, 1)
    assert np.abs(got[rows] - want).max() <= 2.0 ** -7 * np.abs(want).max()


def test_reference_mxfp4_matmul_kernel(oracle):
    """mxmatmul_performance_kernel.cpp of a5/matmul_mxfp4_performance (LaunchMxMatmul: m, k, n = 2040, 8192, 8100, e2m1
    operands two per byte, bf16 output, 32 blocks of 512 x 1024 in 256 x 256 tiles) with stepKa = stepKb = 1.  The last row
    block has 248 valid rows and the last column block 164 valid columns: every tile of the kernel carries run-time valid
    extents (`tile = TileT(validRows, validCols)` on TASSIGNed tiles, TLOAD / TEXTRACT / TMATMUL_MX / TSTORE on them).  On
    the generator's data every sum is exact in fp32, so every element equals the native kernel's bf16 result; nothing is
    written outside C."""
    import torch
    import gpu_util as G
    from pto_amd import capi, datagen
    lib = _ported("libpto_ported_mxfp4.so")
    fn = lib._Z14LaunchMxMatmulPhS_S_S_S_Pv         # void LaunchMxMatmul(uint8_t*, uint8_t*, uint8_t*, uint8_t*, uint8_t*, void*)
    fn.argtypes, fn.restype = [C.c_void_p] * 6, None
    m, k, n = 2040, 8192, 8100
    a, b, sa, sb = datagen.mx_inputs(m, n, k, 4)
    ta, tb, tsa, tsb = (torch.from_numpy(x).to(G.DEV) for x in (a, b, sa, sb))
    guard = 4096                                     # elements before and after C that must keep their pattern
    buf = torch.full((m * n + 2 * guard,), 0x7FC1, dtype=torch.int16, device=G.DEV)
    tc = buf[guard:guard + m * n].view(m, n)
    print("ported mxfp4 launch", flush=True)
    fn(tc.data_ptr(), ta.data_ptr(), tb.data_ptr(), tsa.data_ptr(), tsb.data_ptr(), None)
    torch.cuda.synchronize()
    got = tc.cpu().numpy().view(np.uint16)
    edges = torch.cat((buf[:guard], buf[guard + m * n:])).cpu().numpy()
    assert np.all(edges == 0x7FC1)
    native = G.gemm_mx(a, b, sa, sb, 4, c_fp32=False)
    assert np.array_equal(got, native)
    rows = np.array([0, 255, 256, 511, 512, 1791, 1792, 2039])
    want = oracle.mx_gemm(a[rows], b, sa[rows], sb, 4)
    u = np.ascontiguousarray(want, dtype=np.float32).view(np.uint32).astype(np.uint64)
    assert np.array_equal(got[rows], ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16))    # RNE to bf16
