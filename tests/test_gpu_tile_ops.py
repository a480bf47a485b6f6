"""GPU parity of the single-tile PTO programs (one workgroup each) through the C ABI:
softmax / rescale stages of the attention path, TTRI masks, mask-form TGATHER, MGATHER, TLOAD with
padding and 5-D views, TEXTRACT windows, TMATMUL_BIAS with fp16 and bf16 operands ordered by Events."""
import numpy as np
import pytest
import torch

from pto_amd import capi

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype in (np.uint16, np.float16):
        return torch.from_numpy(a.view(np.int16)).to(DEV)
    return torch.from_numpy(a).to(DEV)


def st():
    return torch.cuda.current_stream().cuda_stream


def softmax_step_oracle(oracle, x, m_in, s_in, scale, first, ties_away):
    """The oracle's row reductions and exp (exp in double, fp32 results), composed as the reference's macro does."""
    lib = oracle.lib()
    x = x.astype(np.float32)
    lmax = x.max(axis=1)
    if first:
        m = lmax
        alpha = np.ones_like(m)
    else:
        m = np.maximum(m_in, lmax)
        alpha = np.exp(((m_in - m) * np.float32(scale)).astype(np.float64)).astype(np.float32)
    p = np.exp((((x - m[:, None]) * np.float32(scale)).astype(np.float32)).astype(np.float64)).astype(np.float32)
    rs = np.zeros(x.shape[0], dtype=np.float32)
    for j in range(x.shape[1]):          # sequential fp32 row sum (cpu/TRowSum.hpp:17-39)
        rs = rs + p[:, j]
    s = rs if first else alpha * s_in + rs
    cvt = lib.po_f32_to_f16_rna if ties_away else lib.po_f32_to_f16_rne
    h = np.array([cvt(int(b)) for b in p.reshape(-1).view(np.uint32)], dtype=np.uint16).reshape(p.shape)
    return h, m, s, alpha, p


@pytest.mark.parametrize("first", [1, 0])
@pytest.mark.parametrize("mode", [capi.CAST_RINT, capi.CAST_ROUND])
def test_softmax_step(oracle, first, mode):
    lib = capi.load_st()
    rng = np.random.default_rng(3 + first)
    x = (rng.standard_normal((64, 256)) * 4).astype(np.float32)
    m_in = (rng.standard_normal(64) * 2 + 6).astype(np.float32)      # some rows keep the old max, some raise it
    s_in = (rng.random(64) * 50 + 1).astype(np.float32)
    scale = np.float32(1.0 / np.sqrt(128.0))
    tx, tm, ts = dev(x), dev(m_in), dev(s_in)
    xe = torch.zeros((64, 256), dtype=torch.int16, device=DEV)
    mo, so, ao = (torch.full((64,), float("nan"), device=DEV) for _ in range(3))
    capi.check(lib.pto_st_softmax_step_f32_64x256(st(), xe.data_ptr(), mo.data_ptr(), so.data_ptr(), ao.data_ptr(),
                                                  tx.data_ptr(), tm.data_ptr(), ts.data_ptr(), float(scale), first, mode), "softmax")
    torch.cuda.synchronize()
    h, m, s, alpha, p = softmax_step_oracle(oracle, x, m_in, s_in, scale, first, mode == capi.CAST_ROUND)
    assert np.array_equal(mo.cpu().numpy(), m)                      # max: exact
    assert np.allclose(ao.cpu().numpy(), alpha, rtol=2e-6, atol=0)  # exp: device exp vs exp in double
    assert np.allclose(so.cpu().numpy(), s, rtol=1e-5, atol=0)      # sum order differs (chunks of 8, then sequential)
    got = xe.cpu().numpy().view(np.uint16).view(np.float16).astype(np.float32)
    want = h.view(np.float16).astype(np.float32)
    # P agrees to an fp16 ulp (the exp differs in the last fp32 bit before rounding)
    assert np.max(np.abs(got - want) / np.maximum(want, 2.0**-14)) <= 2.0**-10


@pytest.mark.parametrize("last", [0, 1])
def test_gu_step(last):
    lib = capi.load_st()
    rng = np.random.default_rng(5)
    o = rng.standard_normal((64, 128)).astype(np.float32)
    pv = rng.standard_normal((64, 128)).astype(np.float32)
    a = rng.random(64).astype(np.float32)
    s = (rng.random(64) * 10 + 1).astype(np.float32)
    out = torch.zeros((64, 128), device=DEV)
    to, tpv, ta, ts = dev(o), dev(pv), dev(a), dev(s)      # named: the buffers must outlive the launch
    capi.check(lib.pto_st_gu_step_f32_64x128(st(), out.data_ptr(), to.data_ptr(), tpv.data_ptr(), ta.data_ptr(),
                                             ts.data_ptr(), last), "gu")
    torch.cuda.synchronize()
    # The device compiler may contract the multiply and the add of two adjacent tile instructions into one
    # fused multiply-add, so each element must equal either rounding: the two-step one or the fused one.
    unfused = (o * a[:, None] + pv).astype(np.float32)
    fused = (o.astype(np.float64) * a[:, None].astype(np.float64) + pv.astype(np.float64)).astype(np.float32)
    if last:
        unfused, fused = (unfused / s[:, None]).astype(np.float32), (fused / s[:, None]).astype(np.float32)
    got = out.cpu().numpy()
    assert np.all((got == unfused) | (got == fused))


@pytest.mark.parametrize("upper,diag", [(1, 1), (1, 37), (1, -5), (0, 0), (0, 20)])
def test_tri_mask(oracle, upper, diag):
    lib = capi.load_st()
    x = np.random.default_rng(7).standard_normal((64, 128)).astype(np.float32)
    out = torch.zeros((64, 128), device=DEV)
    tx = dev(x)
    capi.check(lib.pto_st_tri_mask_f32_64x128(st(), out.data_ptr(), tx.data_ptr(), diag, -3.40282e38, upper), "tri")
    torch.cuda.synchronize()
    r, c = np.arange(64)[:, None], np.arange(128)[None, :]
    one = (c >= diag + r) if upper else (c < diag + r + 1)
    want = x + np.where(one, np.float32(-3.40282e38), np.float32(0.0)).astype(np.float32)
    assert np.array_equal(out.cpu().numpy(), want.astype(np.float32))


@pytest.mark.parametrize("pattern,sl,div", [(1, slice(0, None, 2), 2), (2, slice(1, None, 2), 2), (3, slice(0, None, 4), 4),
                                            (4, slice(1, None, 4), 4), (5, slice(2, None, 4), 4), (6, slice(3, None, 4), 4),
                                            (7, slice(None), 1)])
def test_tgather_mask(oracle, pattern, sl, div):
    lib = capi.load_st()
    src = np.random.default_rng(pattern).integers(0, 2**16, size=(16, 64), dtype=np.uint16)
    out = torch.zeros((16, 64 // div), dtype=torch.int16, device=DEV)
    tsrc = dev(src)
    capi.check(lib.pto_st_tgather_mask_b16_16x64(st(), out.data_ptr(), tsrc.data_ptr(), pattern), "tgather mask")
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(np.uint16)
    assert np.array_equal(got, src[:, sl])
    want, n = oracle.tgather_mask(oracle.make_layout(16, 64 // div), src.reshape(-1), oracle.make_layout(16, 64), 16, 64, pattern)
    assert np.array_equal(got.reshape(-1), want)


def test_mgather_elements(oracle):
    lib = capi.load_st()
    rng = np.random.default_rng(11)
    gm = rng.integers(0, 2**16, size=65536, dtype=np.uint16)
    idx = rng.integers(0, 65536, size=(8, 128), dtype=np.int32)
    out = torch.zeros((8, 128), dtype=torch.int16, device=DEV)
    tgm, tidx = dev(gm), dev(idx)
    capi.check(lib.pto_st_mgather_b16_8x128(st(), out.data_ptr(), tgm.data_ptr(), tidx.data_ptr(), 65536), "mgather")
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint16), gm[idx])


def test_tload_pad_and_valid_region(oracle):
    lib = capi.load_st()
    x = np.arange(200, dtype=np.float32)
    img = torch.zeros((16, 32), device=DEV)
    tx = dev(x)
    capi.check(lib.pto_st_tload_pad_f32_16x32(st(), img.data_ptr(), tx.data_ptr()), "tload pad")
    torch.cuda.synchronize()
    L = oracle.make_layout(16, 32, oracle.BL_ROW, oracle.SL_NONE, 4)
    want = oracle.tload(L, np.float32, x, [1, 1, 1, 10, 20], [200, 200, 200, 20, 1], 10, 20, pad=np.inf)
    assert np.array_equal(img.cpu().numpy().reshape(-1), want)


def test_tload_tstore_5d(oracle):
    lib = capi.load_st()
    gm = np.arange(2000, dtype=np.float32)
    dense = torch.zeros((24, 8), device=DEV)
    strided = torch.full((2000,), -1.0, device=DEV)
    tgm = dev(gm)
    capi.check(lib.pto_st_tload_5d_f32(st(), dense.data_ptr(), strided.data_ptr(), tgm.data_ptr()), "5d")
    torch.cuda.synchronize()
    L = oracle.make_layout(24, 8, oracle.BL_ROW, oracle.SL_NONE, 4)
    want = oracle.tload(L, np.float32, gm, [1, 2, 3, 4, 8], [1000, 400, 100, 10, 1])
    assert np.array_equal(dense.cpu().numpy().reshape(-1), want)
    back = np.full(2000, -1.0, dtype=np.float32)
    oracle.tstore(back, [1, 2, 3, 4, 8], [1000, 400, 100, 10, 1], want, L)
    assert np.array_equal(strided.cpu().numpy(), back)


def test_mat_tile_walked_through_data_pointer_ends_the_kernel(capfd):
    """TASSIGN of a Mat tile that has an address to `data() + n` of another: n == 0 is the image itself, n != 0 is a part of
    a swizzled image and not a tile (the reference's L1 layout allows it, pto_macro_matmul.hpp:176-177) - the kernel
    says so and ends there, in every wave, instead of computing on other data."""
    lib = capi.load_st()
    for chunks, reached in ((1, 1), (2, 0)):
        flags = torch.zeros(2, dtype=torch.int32, device="cuda")
        capi.check(lib.pto_st_mat_view_walk(st(), flags.data_ptr(), chunks), "walk")
        torch.cuda.synchronize()
        assert flags.cpu().tolist() == [1, reached], (chunks, flags.cpu().tolist())
    out = capfd.readouterr().out
    assert "[PTO][RT] TASSIGN: a Mat tile at LDS offset 0 is moved to 16384" in out, out


@pytest.mark.parametrize("col0,row0", [(0, 0), (64, 128), (192, 192), (8, 40)])
def test_textract_windows(oracle, col0, row0):
    """dst[i,j] = src[r0+i, c0+j] for windows that are not the suffix (the reference CPU simulation only
    takes the suffix; the ISA definition is the oracle's mode 1)."""
    lib = capi.load_st()
    rng = np.random.default_rng(13)
    a = rng.integers(-8, 8, size=(128, 256)).astype(np.float16)
    b = rng.integers(-8, 8, size=(256, 256)).astype(np.float16)      # logical [k, n]
    b_t = np.ascontiguousarray(b.T)                                  # stored [n][k]
    eye_b = np.zeros((256, 64), dtype=np.float16)                    # [n][k] of a 64 x 256 identity
    eye_b[np.arange(64), np.arange(64)] = 1
    eye_a = np.zeros((128, 64), dtype=np.float16)
    eye_a[np.arange(64), np.arange(64)] = 1
    ol, orr = torch.zeros((128, 256), device=DEV), torch.zeros((128, 256), device=DEV)
    ta, tb, teb, tea = dev(a), dev(b_t), dev(eye_b), dev(eye_a)
    capi.check(lib.pto_st_textract_windows_f16(st(), ol.data_ptr(), orr.data_ptr(), ta.data_ptr(), tb.data_ptr(),
                                               teb.data_ptr(), tea.data_ptr(), col0, row0), "textract")
    torch.cuda.synchronize()
    gl, gr = ol.cpu().numpy(), orr.cpu().numpy()
    assert np.array_equal(gl[:, :64], a[:, col0:col0 + 64].astype(np.float32)) and not gl[:, 64:].any()
    assert np.array_equal(gr[:64], b[row0:row0 + 64].astype(np.float32)) and not gr[64:].any()
    o = oracle
    Ls, Ld = o.make_layout(128, 256, o.BL_COL, o.SL_ROW, 2), o.make_layout(128, 64, o.BL_COL, o.SL_ROW, 2)
    src = o.tload(Ls, np.uint16, a.view(np.uint16), [1, 1, 1, 128, 256], [0, 0, 0, 256, 1])
    win = o.textract(Ld, 128, 64, src, Ls, 128, 256, 0, col0, mode=1)
    plain = np.zeros((128, 64), dtype=np.uint16)
    o.tstore(plain, [1, 1, 1, 128, 64], [0, 0, 0, 64, 1], win, Ld)
    assert np.array_equal(plain.view(np.float16).astype(np.float32), gl[:, :64])


@pytest.mark.parametrize("bf16", [0, 1])
@pytest.mark.parametrize("with_bias", [0, 1])
def test_matmul_bias_and_bf16(oracle, bf16, with_bias):
    lib = capi.load_st()
    rng = np.random.default_rng(17)
    a = rng.integers(1, 5, size=(128, 64)).astype(np.float32)
    b = rng.integers(1, 5, size=(64, 256)).astype(np.float32)
    bias = rng.integers(1, 10, size=256).astype(np.float32)
    if bf16:
        ta = torch.from_numpy(a).to(torch.bfloat16).to(DEV)
        tb = torch.from_numpy(np.ascontiguousarray(b.T)).to(torch.bfloat16).to(DEV)
    else:
        ta, tb = dev(a.astype(np.float16)), dev(np.ascontiguousarray(b.T).astype(np.float16))
    out = torch.zeros((128, 256), device=DEV)
    tbias = dev(bias)
    capi.check(lib.pto_st_matmul_bias_128x64x256(st(), out.data_ptr(), ta.data_ptr(), tb.data_ptr(),
                                                 tbias.data_ptr() if with_bias else 0, bf16), "matmul bias")
    torch.cuda.synchronize()
    want = a @ b + (bias if with_bias else 0)
    assert np.array_equal(out.cpu().numpy(), want.astype(np.float32))
    if not bf16 and with_bias:
        o = oracle
        La, Lb = o.make_layout(128, 64, o.BL_COL, o.SL_ROW, 2), o.make_layout(64, 256, o.BL_ROW, o.SL_COL, 2)
        Lc = o.make_layout(128, 256, o.BL_COL, o.SL_ROW, 4, 1024)
        tA = o.tload(La, np.uint16, a.astype(np.float16).view(np.uint16), [1, 1, 1, 128, 64], [0, 0, 0, 64, 1])
        tB = o.tload(Lb, np.uint16, b.astype(np.float16).view(np.uint16), [1, 1, 1, 64, 256], [0, 0, 0, 256, 1])
        acc = o.tmatmul(tA, La, tB, Lb, Lc, 128, 256, 64, bias=bias)
        ref = np.zeros((128, 256), dtype=np.float32)
        o.tstore(ref, [1, 1, 1, 128, 256], [0, 0, 0, 256, 1], acc, Lc)
        assert np.array_equal(out.cpu().numpy(), ref)


@pytest.mark.parametrize("lds_fifo", [0, 1])
def test_tpush_tpop_pipeline(lds_fifo):
    """Accumulator -> FIFO -> Vec tile and Vec -> FIFO -> Mat tile hand-offs; integer-valued data, so every
    product, sum and the fp16 cast are exact and the result must equal numpy's."""
    lib = capi.load_st()
    rng = np.random.default_rng(31 + lds_fifo)
    a = rng.integers(-2, 3, size=(64, 64)).astype(np.float32)
    b = rng.integers(-2, 3, size=(2, 64, 128)).astype(np.float32)
    v = rng.integers(-2, 3, size=(2, 128, 64)).astype(np.float32)
    ta = dev(a.astype(np.float16))
    tb = dev(np.ascontiguousarray(b.transpose(0, 2, 1)).astype(np.float16))    # [t][n][k]
    tv = dev(np.ascontiguousarray(v.transpose(0, 2, 1)).astype(np.float16))    # [t][n][k]
    qk = torch.zeros(2 * 64 * 128, device=DEV)
    pf = torch.zeros(2 * 64 * 128, dtype=torch.int16, device=DEV)
    out = torch.zeros((64, 64), device=DEV)
    capi.check(lib.pto_st_pushpop_f16_64x64x128(st(), out.data_ptr(), ta.data_ptr(), tb.data_ptr(), tv.data_ptr(),
                                                0 if lds_fifo else qk.data_ptr(), pf.data_ptr(), lds_fifo), "pushpop")
    torch.cuda.synchronize()
    want = np.zeros((64, 64), dtype=np.float32)
    for t in range(2):
        p = ((a @ b[t]) * np.float32(0.25)).astype(np.float16).astype(np.float32)
        want += p @ v[t]
    assert np.array_equal(out.cpu().numpy(), want)
    # the FIFO slots hold what was pushed: slot t = tile t (depth 2)
    pslots = pf.cpu().numpy().view(np.float16).reshape(2, 64, 128).astype(np.float32)
    for t in range(2):
        assert np.array_equal(pslots[t], ((a @ b[t]) * np.float32(0.25)))
    if not lds_fifo:
        qslots = qk.cpu().numpy().reshape(2, 64, 128)
        for t in range(2):
            assert np.array_equal(qslots[t], a @ b[t])


@pytest.mark.parametrize("via_lds", [0, 1])
@pytest.mark.parametrize("fmt_a,fmt_b", [(0, 0), (1, 1), (0, 1), (1, 0)])
def test_tmatmul_mx_single_tile(oracle, fmt_a, fmt_b, via_lds):
    """TMATMUL_MX and its accumulating form on two 128-wide k halves (two MFMA k steps each), mixed operand formats,
    scale tiles loaded from memory (MX_A_ND / MX_B_DN) and windowed, or staged in Mat tiles of block scales and
    TEXTRACTed: exact on integer operands, <= 2e-3 on random ones."""
    from pto_amd import datagen
    lib = capi.load_st()
    for dist, lo, hi in (("integer", 125, 130), ("uniform", 120, 135), ("bytes", 110, 140)):
        a, _, sa, _ = datagen.mx_inputs(128, 128, 256, fmt_a, dist=dist, scale_lo=lo, scale_hi=hi)
        _, b, _, sb = datagen.mx_inputs(128, 128, 256, fmt_b, dist=dist, scale_lo=lo, scale_hi=hi)
        out = torch.full((128, 128), float("nan"), device=DEV)
        ta, tb, tsa, tsb = (torch.from_numpy(x).to(DEV) for x in (a, b, sa, sb))
        capi.check(lib.pto_st_matmul_mx_128x256x128(st(), out.data_ptr(), ta.data_ptr(), tb.data_ptr(), tsa.data_ptr(),
                                                    tsb.data_ptr(), fmt_a, fmt_b, via_lds), "matmul mx")
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        want = oracle.mx_gemm(a, b, sa, sb, fmt_a, fmt_b)
        if dist == "integer":
            assert np.array_equal(got, want), (dist, fmt_a, fmt_b)
        else:
            assert np.max(np.abs(got - want)) <= 2e-3 * np.max(np.abs(want)), (dist, fmt_a, fmt_b)


@pytest.mark.parametrize("fmt", [0, 1])
def test_tmatmul_mx_bias_form(oracle, fmt):
    """TMATMUL_MX(c, a, aScale, b, bScale, bias) with a [1, n] Bias tile (the reference's bias form, pto_instr.hpp:444-451;
    its generator adds the bias row to every row of the product: tmatmul_mx/gen_data.py): integer operands and an integer
    bias row, exact."""
    from pto_amd import datagen
    lib = capi.load_st()
    a, b, sa, sb = datagen.mx_inputs(128, 128, 256, fmt, dist="integer", scale_lo=126, scale_hi=130)
    bias = np.random.default_rng(9).integers(-10, 10, size=128).astype(np.float32)
    out = torch.full((128, 128), float("nan"), device=DEV)
    ta, tb, tsa, tsb, tbias = (torch.from_numpy(x).to(DEV) for x in (a, b, sa, sb, bias))
    capi.check(lib.pto_st_matmul_mx_bias_128x256x128(st(), out.data_ptr(), ta.data_ptr(), tb.data_ptr(), tsa.data_ptr(), tsb.data_ptr(),
                                                     tbias.data_ptr(), fmt, fmt), "matmul mx bias")
    torch.cuda.synchronize()
    want = oracle.mx_gemm(a, b, sa, sb, fmt, fmt) + bias[None, :]
    assert np.array_equal(out.cpu().numpy(), want.astype(np.float32))


def test_tmatmul_int8_to_int32(oracle):
    """int8 x int8 -> int32 (v_mfma_i32_32x32x32_i8), TMATMUL then TMATMUL_ACC over two k halves: exact."""
    lib = capi.load_st()
    rng = np.random.default_rng(23)
    a = rng.integers(-128, 128, size=(128, 128), dtype=np.int8)
    b = rng.integers(-128, 128, size=(128, 256), dtype=np.int8)
    a[0, :] = -128
    b[:, 0] = -128                                               # the extreme product, 128 times
    out = torch.full((128, 256), -1, dtype=torch.int32, device=DEV)
    ta, tb = torch.from_numpy(a).to(DEV), torch.from_numpy(np.ascontiguousarray(b.T)).to(DEV)
    capi.check(lib.pto_st_matmul_s8_128x128x256(st(), out.data_ptr(), ta.data_ptr(), tb.data_ptr(), 0), "matmul s8")
    torch.cuda.synchronize()
    want = a.astype(np.int32) @ b.astype(np.int32)
    assert np.array_equal(out.cpu().numpy(), want)
    out_relu = torch.full((128, 256), -1, dtype=torch.int32, device=DEV)
    capi.check(lib.pto_st_matmul_s8_128x128x256(st(), out_relu.data_ptr(), ta.data_ptr(), tb.data_ptr(), 1), "matmul s8 relu")
    torch.cuda.synchronize()
    assert np.array_equal(out_relu.cpu().numpy(), np.maximum(want, 0)) and (want < 0).any()
    o = oracle
    La, Lb = o.make_layout(128, 128, o.BL_COL, o.SL_ROW, 1), o.make_layout(128, 256, o.BL_ROW, o.SL_COL, 1)
    Lc = o.make_layout(128, 256, o.BL_COL, o.SL_ROW, 4, 1024)
    tA = o.tload(La, np.int8, a, [1, 1, 1, 128, 128], [0, 0, 0, 128, 1])
    tB = o.tload(Lb, np.int8, b, [1, 1, 1, 128, 256], [0, 0, 0, 256, 1])
    acc = o.tmatmul(tA, La, tB, Lb, Lc, 128, 256, 128)
    ref = np.zeros((128, 256), dtype=np.int32)
    o.tstore(ref, [1, 1, 1, 128, 256], [0, 0, 0, 256, 1], acc, Lc)
    assert np.array_equal(out.cpu().numpy(), ref)


def test_tmatmul_fp32(oracle):
    """fp32 x fp32 -> fp32 (v_mfma_f32_32x32x2_f32): exact on integers, fp32 rounding only otherwise."""
    lib = capi.load_st()
    rng = np.random.default_rng(29)
    for integer in (True, False):
        if integer:
            a = rng.integers(-9, 10, size=(128, 32)).astype(np.float32)
            b = rng.integers(-9, 10, size=(32, 256)).astype(np.float32)
        else:
            a = rng.standard_normal((128, 32)).astype(np.float32)
            b = rng.standard_normal((32, 256)).astype(np.float32)
        out = torch.full((128, 256), float("nan"), device=DEV)
        ta, tb = dev(a), dev(np.ascontiguousarray(b.T))
        capi.check(lib.pto_st_matmul_f32_128x32x256(st(), out.data_ptr(), ta.data_ptr(), tb.data_ptr(), 0), "matmul f32")
        out_relu = torch.full((128, 256), float("nan"), device=DEV)
        capi.check(lib.pto_st_matmul_f32_128x32x256(st(), out_relu.data_ptr(), ta.data_ptr(), tb.data_ptr(), 1), "matmul f32 relu")
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        assert np.array_equal(out_relu.cpu().numpy(), np.maximum(got, 0))
        want = a.astype(np.float64) @ b.astype(np.float64)
        if integer:
            assert np.array_equal(got, want.astype(np.float32))
        else:
            assert np.max(np.abs(got - want)) <= 1e-5 * np.max(np.abs(want))
            o = oracle
            La, Lb = o.make_layout(128, 32, o.BL_COL, o.SL_ROW, 4), o.make_layout(32, 256, o.BL_ROW, o.SL_COL, 4)
            Lc = o.make_layout(128, 256, o.BL_COL, o.SL_ROW, 4, 1024)
            tA = o.tload(La, np.float32, a, [1, 1, 1, 128, 32], [0, 0, 0, 32, 1])
            tB = o.tload(Lb, np.float32, b, [1, 1, 1, 32, 256], [0, 0, 0, 256, 1])
            acc = o.tmatmul(tA, La, tB, Lb, Lc, 128, 256, 32)
            ref = np.zeros((128, 256), dtype=np.float32)
            o.tstore(ref, [1, 1, 1, 128, 256], [0, 0, 0, 256, 1], acc, Lc)
            assert np.max(np.abs(got - ref)) <= 1e-5 * np.max(np.abs(ref))
