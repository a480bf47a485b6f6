"""Pins the oracle's arithmetic functions (CPU only): TMATMUL, TCVT, TGATHER/MGATHER, attention.

What each check can catch is stated beside it; none re-types the oracle's own formula.
"""
import ctypes as C
import os

import numpy as np
import pytest
import torch

from pto_amd import datagen


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _gemm_layouts(o, M, K, N):
    La = o.make_layout(M, K, o.BL_COL, o.SL_ROW, 2)
    Lb = o.make_layout(K, N, o.BL_ROW, o.SL_COL, 2)
    Lc = o.make_layout(M, N, o.BL_COL, o.SL_ROW, 4, 1024)
    return La, Lb, Lc


def _tile_matmul(o, a, b, acc_tile=None):
    """a [M,K] fp16, b [N,K] fp16 through TLOAD -> TMATMUL -> (Acc tile storage, layouts)."""
    M, K = a.shape
    N = b.shape[0]
    La, Lb, Lc = _gemm_layouts(o, M, K, N)
    ta = o.tload(La, np.uint16, a.view(np.uint16), [1, 1, 1, M, K], [0, 0, 0, K, 1])
    tb = o.tload(Lb, np.uint16, b.view(np.uint16), [1, 1, 1, K, N], [0, 0, 0, 1, K])
    return o.tmatmul(ta, La, tb, Lb, Lc, M, N, K, acc=acc_tile), Lc


def _acc_to_nd(o, acc, Lc):
    out = np.zeros((Lc.rows, Lc.cols), dtype=acc.dtype)
    o.tstore(out, [1, 1, 1, Lc.rows, Lc.cols], [0, 0, 0, Lc.cols, 1], acc, Lc)
    return out


# ------------------------------------------------------------------ matmul
def test_matmul_integer_inputs_exact(oracle):
    """Integer-valued operands make every fp32 partial sum exact, so a transposed operand, a dropped
    k term or a wrong layout offset changes the result (recipe of tmatmul/gen_data.py:40-41)."""
    a, b = datagen.gemm_inputs_integer(48, 80, 96)
    acc, Lc = _tile_matmul(oracle, a, b)
    want = a.astype(np.int64) @ b.astype(np.int64).T
    assert np.array_equal(_acc_to_nd(oracle, acc, Lc), want.astype(np.float32))


def test_matmul_acc_adds_partial(oracle):
    a, b = datagen.gemm_inputs_integer(32, 32, 64)
    acc1, Lc = _tile_matmul(oracle, a, b)
    acc2, _ = _tile_matmul(oracle, a, b, acc_tile=acc1)
    assert np.array_equal(acc2, 2 * acc1)


def test_matmul_random_vs_fp64(oracle):
    a, b = datagen.gemm_inputs(64, 48, 256)
    acc, Lc = _tile_matmul(oracle, a, b)
    want = a.astype(np.float64) @ b.astype(np.float64).T
    got = _acc_to_nd(oracle, acc, Lc)
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1.0)) < 1e-5


def test_gemm_composite_equals_op_by_op(oracle):
    """The whole-GEMM routine must give the same bits as TLOAD/TEXTRACT/TMATMUL[_ACC]/TSTORE per K-step."""
    o = oracle
    M, N, K, KS = 32, 48, 256, 64
    a, b = datagen.gemm_inputs(M, N, K)
    La, Lb, Lc = _gemm_layouts(o, M, KS, N)
    acc = None
    for k0 in range(0, K, KS):
        ta = o.tload(La, np.uint16, a.view(np.uint16).reshape(-1)[k0:], [1, 1, 1, M, KS], [0, 0, 0, K, 1])
        tb = o.tload(Lb, np.uint16, b.view(np.uint16).reshape(-1)[k0:], [1, 1, 1, KS, N], [0, 0, 0, 1, K])
        acc = o.tmatmul(ta, La, tb, Lb, Lc, M, N, KS, acc=acc)
    assert np.array_equal(_acc_to_nd(o, acc, Lc), o.gemm_f16f32(a, b, base_k=KS))
    # and the K-step changes the rounding sequence, i.e. base_k is really honoured
    assert not np.array_equal(o.gemm_f16f32(a, b, base_k=KS), o.gemm_f16f32(a, b, base_k=K))


def test_gemm_row_subset(oracle):
    a, b = datagen.gemm_inputs(64, 32, 128)
    full = oracle.gemm_f16f32(a, b, base_k=64)
    part = oracle.gemm_f16f32(a, b, base_k=64, row0=16, row1=40)
    assert np.array_equal(part[16:40], full[16:40]) and not part[:16].any() and not part[40:].any()


@pytest.mark.parametrize("name,M,K,N,KS", [("ref_gemm_128x64x256_ks64", 128, 64, 256, 64),
                                           ("ref_gemm_128x256x256_ks64", 128, 256, 256, 64),
                                           ("ref_gemm_128x512x128_ks64", 128, 512, 128, 64),
                                           ("ref_gemm_256x256x256_ks256", 256, 256, 256, 256)])
def test_ref_gemm_tile_path(oracle, ref, name, M, K, N, KS):
    """Compiled reference TLOAD->TEXTRACT->TMATMUL[_ACC]->TSTORE vs the restatement.  Integer inputs: exact.
    Random inputs: the reference's vectorize pragma may reorder the k-sum, so compare to 1e-5 and report."""
    for gen, exact in ((datagen.gemm_inputs_integer, True), (datagen.gemm_inputs, False)):
        a, b = gen(M, N, K)
        c = np.zeros((M, N), dtype=np.float32)
        getattr(ref, name)(_p(c), _p(a), _p(b))
        mine = oracle.gemm_f16f32(a, b, base_k=KS)
        if exact:
            assert np.array_equal(c, mine)
        else:
            assert np.max(np.abs(c - mine)) <= 1e-5 * max(1.0, np.max(np.abs(mine)))


def test_ref_matmul_st_cases(oracle, ref):
    """Shapes of the reference's tmatmul ST (tmatmul/gen_data.py:91-99), valid regions inside padded tiles."""
    o = oracle
    rng = np.random.default_rng(19)
    # fp16 40x50x60
    a = rng.integers(1, 5, size=(40, 50)).astype(np.float16)
    b = rng.integers(1, 5, size=(50, 60)).astype(np.float16)
    out = np.zeros((40, 60), dtype=np.float32)
    ref.ref_matmul_f16_40x50x60(_p(out), _p(a), _p(b))
    assert np.array_equal(out, (a.astype(np.float32) @ b.astype(np.float32)))
    La = o.make_layout(48, 64, o.BL_COL, o.SL_ROW, 2)
    Lb = o.make_layout(64, 64, o.BL_ROW, o.SL_COL, 2)
    Lc = o.make_layout(48, 64, o.BL_COL, o.SL_ROW, 4, 1024)
    ta = o.tload(La, np.uint16, a.view(np.uint16), [1, 1, 1, 40, 50], [0, 0, 0, 50, 1], 40, 50)
    tb = o.tload(Lb, np.uint16, b.view(np.uint16), [1, 1, 1, 50, 60], [0, 0, 0, 60, 1], 50, 60)
    acc = o.tmatmul(ta, La, tb, Lb, Lc, 40, 60, 50)
    mine = np.zeros((40, 60), dtype=np.float32)
    o.tstore(mine, [1, 1, 1, 40, 60], [0, 0, 0, 60, 1], acc, Lc, 40, 60)
    assert np.array_equal(mine, out)
    # int8 6x7x8
    a8 = rng.integers(-5, 5, size=(6, 7)).astype(np.int8)
    b8 = rng.integers(-5, 5, size=(7, 8)).astype(np.int8)
    o32 = np.zeros((6, 8), dtype=np.int32)
    ref.ref_matmul_s8_6x7x8(_p(o32), _p(a8), _p(b8))
    assert np.array_equal(o32, a8.astype(np.int32) @ b8.astype(np.int32))
    La = o.make_layout(32, 32, o.BL_COL, o.SL_ROW, 1)
    Lb = o.make_layout(32, 32, o.BL_ROW, o.SL_COL, 1)
    Lc = o.make_layout(32, 32, o.BL_COL, o.SL_ROW, 4, 1024)
    ta = o.tload(La, np.int8, a8, [1, 1, 1, 6, 7], [0, 0, 0, 7, 1], 6, 7)
    tb = o.tload(Lb, np.int8, b8, [1, 1, 1, 7, 8], [0, 0, 0, 8, 1], 7, 8)
    acc = o.tmatmul(ta, La, tb, Lb, Lc, 6, 8, 7)
    mine = np.zeros((6, 8), dtype=np.int32)
    o.tstore(mine, [1, 1, 1, 6, 8], [0, 0, 0, 8, 1], acc, Lc, 6, 8)
    assert np.array_equal(mine, o32)
    # fp32 120x110x50 (random): reference vs restatement vs fp64
    af = rng.uniform(-1, 1, size=(120, 110)).astype(np.float32)
    bf = rng.uniform(-1, 1, size=(110, 50)).astype(np.float32)
    of = np.zeros((120, 50), dtype=np.float32)
    ref.ref_matmul_f32_120x110x50(_p(of), _p(af), _p(bf))
    La = o.make_layout(128, 112, o.BL_COL, o.SL_ROW, 4)
    Lb = o.make_layout(112, 64, o.BL_ROW, o.SL_COL, 4)
    Lc = o.make_layout(128, 64, o.BL_COL, o.SL_ROW, 4, 1024)
    ta = o.tload(La, np.float32, af, [1, 1, 1, 120, 110], [0, 0, 0, 110, 1], 120, 110)
    tb = o.tload(Lb, np.float32, bf, [1, 1, 1, 110, 50], [0, 0, 0, 50, 1], 110, 50)
    acc = o.tmatmul(ta, La, tb, Lb, Lc, 120, 50, 110)
    mine = np.zeros((120, 50), dtype=np.float32)
    o.tstore(mine, [1, 1, 1, 120, 50], [0, 0, 0, 50, 1], acc, Lc, 120, 50)
    assert np.allclose(mine, of, rtol=0, atol=2e-5)
    assert np.allclose(mine, af.astype(np.float64) @ bf.astype(np.float64), rtol=0, atol=1e-4)
    # bias 26x100x94
    a = rng.integers(1, 5, size=(26, 100)).astype(np.float16)
    b = rng.integers(1, 5, size=(100, 94)).astype(np.float16)
    bias = rng.integers(1, 10, size=94).astype(np.float32)
    out = np.zeros((26, 94), dtype=np.float32)
    ref.ref_matmul_bias_f16_26x100x94(_p(out), _p(a), _p(b), _p(bias))
    assert np.array_equal(out, a.astype(np.float32) @ b.astype(np.float32) + bias)
    La = o.make_layout(32, 112, o.BL_COL, o.SL_ROW, 2)
    Lb = o.make_layout(112, 96, o.BL_ROW, o.SL_COL, 2)
    Lc = o.make_layout(32, 96, o.BL_COL, o.SL_ROW, 4, 1024)
    ta = o.tload(La, np.uint16, a.view(np.uint16), [1, 1, 1, 26, 100], [0, 0, 0, 100, 1], 26, 100)
    tb = o.tload(Lb, np.uint16, b.view(np.uint16), [1, 1, 1, 100, 94], [0, 0, 0, 94, 1], 100, 94)
    acc = o.tmatmul(ta, La, tb, Lb, Lc, 26, 94, 100, bias=bias)
    mine = np.zeros((26, 94), dtype=np.float32)
    o.tstore(mine, [1, 1, 1, 26, 94], [0, 0, 0, 94, 1], acc, Lc, 26, 94)
    assert np.array_equal(mine, out)


# ---------------------------------------------------------------- conversion
def _boundary_patterns():
    """Every exponent with mantissas at, just below and just above each fp16 rounding boundary."""
    exps = np.arange(0, 256, dtype=np.uint32) << 23
    mants = np.array([0, 1, 0xfff, 0x1000, 0x1001, 0x1fff, 0x2000, 0x2001, 0x2fff, 0x3000, 0x3001,
                      0x7fe000, 0x7fefff, 0x7ff000, 0x7ff001, 0x7fffff, 0x400000, 0x3fffff, 0x400001,
                      0x200000, 0x600000, 0x100000, 0x080000, 0x7fc000, 0x7f8000], dtype=np.uint32)
    pos = (exps[:, None] | mants[None, :]).reshape(-1)
    return np.concatenate([pos, pos | np.uint32(0x80000000)])


def test_tcvt_f32_f16_matches_numpy_rne(oracle):
    """numpy's float32->float16 is IEEE round-to-nearest-even (what tcvt/gen_data.py:25-26 uses as golden).
    Boundary patterns + 16M strided patterns; NaNs compared by payload policy separately."""
    bits = np.concatenate([_boundary_patterns(), np.arange(0, 2**32, 251, dtype=np.uint64).astype(np.uint32)])
    x = bits.view(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = oracle.tcvt_f32_f16(x)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    gn = got[nan]
    assert np.all((gn & 0x7c00) == 0x7c00) and np.all((gn & 0x0200) != 0)      # quiet NaN
    assert np.array_equal(gn >> 15, (bits[nan] >> 31).astype(np.uint16))        # sign kept
    assert np.array_equal(gn & 0x1ff, ((bits[nan] >> 13) & 0x1ff).astype(np.uint16))  # top payload kept


@pytest.mark.skipif(os.environ.get("PTO_SLOW") != "1", reason="exhaustive 2^32 sweep: set PTO_SLOW=1")
def test_tcvt_f32_f16_exhaustive(oracle):
    for hi in range(0, 2**32, 2**26):
        bits = np.arange(hi, hi + 2**26, dtype=np.uint64).astype(np.uint32)
        x = bits.view(np.float32)
        with np.errstate(over="ignore", invalid="ignore"):
            want = x.astype(np.float16).view(np.uint16)
        got = oracle.tcvt_f32_f16(x)
        nan = np.isnan(x)
        assert np.array_equal(got[~nan], want[~nan])


def test_tcvt_f32_f16_known_answers(oracle):
    ka = {0x00000000: 0x0000, 0x80000000: 0x8000, 0x3f800000: 0x3c00, 0x477fe000: 0x7bff, 0x477fefff: 0x7bff,
          0x477ff000: 0x7c00, 0x47800000: 0x7c00, 0x7f800000: 0x7c00, 0xff800000: 0xfc00,
          0x33800000: 0x0001, 0x33000000: 0x0000, 0x33000001: 0x0001, 0x33c00000: 0x0002,  # 2^-24, 2^-25 (tie->0), 1.5*2^-24 (tie->2)
          0x387fe000: 0x0400, 0x387fc000: 0x03ff, 0x38800000: 0x0400,
          0x3f801000: 0x3c00, 0x3f803000: 0x3c02, 0x3f801001: 0x3c01, 0x7fc00000: 0x7e00}
    for b, h in ka.items():
        assert oracle.lib().po_f32_to_f16_rne(b) == h, hex(b)
    # ties away from zero differ from RNE exactly on ties with an even kept mantissa
    assert oracle.lib().po_f32_to_f16_rna(0x3f801000) == 0x3c01
    assert oracle.lib().po_f32_to_f16_rna(0x3f803000) == 0x3c02
    assert oracle.lib().po_f32_to_f16_rna(0x33000000) == 0x0001
    assert oracle.lib().po_f32_to_f16_rna(0x3f800fff) == 0x3c00


def test_tcvt_f32_bf16_matches_torch(oracle):
    """torch's float32->bfloat16 is round-to-nearest-even; parity with the reference itself is unpinned
    (its bfloat16_t is _Float16 with this toolchain)."""
    bits = np.concatenate([_boundary_patterns(), np.arange(0, 2**32, 257, dtype=np.uint64).astype(np.uint32),
                           np.array([0x3f808000, 0x3f818000, 0x3f807fff, 0x3f808001, 0x7f7fffff, 0x7f7f8000],
                                    dtype=np.uint32)])
    x = bits.view(np.float32)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = oracle.tcvt_f32_bf16(x)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    gn = got[nan]
    assert np.all((gn & 0x7f80) == 0x7f80) and np.all((gn & 0x0040) != 0)
    assert np.array_equal(gn & 0x803f, ((bits[nan] >> 16) & 0x803f).astype(np.uint16))


def test_f16_to_f32_all_values(oracle):
    h = np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)
    got = oracle.tcvt_f16_f32(h).view(np.uint32)
    want = h.view(np.float16).astype(np.float32).view(np.uint32)
    nan = np.isnan(h.view(np.float16))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(got[nan].view(np.float32)))
    # and fp16 -> fp32 -> fp16 is the identity, which ties the two directions together
    back = oracle.tcvt_f32_f16(got.view(np.float32))
    assert np.array_equal(back[~nan], h[~nan])


def test_ref_tcvt(oracle, ref):
    """Compiled reference TLOAD->TCVT(CAST_RINT)->TSTORE, bit for bit, NaNs included."""
    x = datagen.tcvt_input(64, 1024, inject=0.05).reshape(-1)
    out = np.zeros(x.size, dtype=np.uint16)
    ref.ref_tcvt_f32_f16(_p(out), _p(x), C.c_size_t(x.size))
    assert np.array_equal(out, oracle.tcvt_f32_f16(x))
    # the ST's own range: values in [0, 4.41) (tcvt/gen_data.py:61-71)
    y = (np.random.default_rng(0).random(4096, dtype=np.float32) * 4.41).astype(np.float32)
    ref.ref_tcvt_f32_f16(_p(out), _p(y), C.c_size_t(4096))
    assert np.array_equal(out[:4096], y.astype(np.float16).view(np.uint16))
    # fp16 -> fp32
    h = np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)
    f = np.zeros(65536, dtype=np.float32)
    ref.ref_tcvt_f16_f32(_p(f), _p(h), C.c_size_t(65536))
    mine = oracle.tcvt_f16_f32(h)
    nan = np.isnan(f)
    assert np.array_equal(f[~nan].view(np.uint32), mine[~nan].view(np.uint32))


def test_tcvt_round_modes_to_int(oracle):
    """float -> int32 is off the accelerated path; pinned by known answers only (the compiled reference
    crashes in this conversion with this toolchain, so it is not compared)."""
    z = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 2.4, -2.6], dtype=np.float32)
    assert oracle.tcvt_f32_s32(z, 1).tolist() == [0, 2, 2, 0, -2, -2, 2, -3]      # CAST_RINT
    assert oracle.tcvt_f32_s32(z, 2).tolist() == [1, 2, 3, -1, -2, -3, 2, -3]     # CAST_ROUND
    assert oracle.tcvt_f32_s32(z, 3).tolist() == [0, 1, 2, -1, -2, -3, 2, -3]     # CAST_FLOOR
    assert oracle.tcvt_f32_s32(z, 4).tolist() == [1, 2, 3, 0, -1, -2, 3, -2]      # CAST_CEIL
    assert oracle.tcvt_f32_s32(z, 5).tolist() == [0, 1, 2, 0, -1, -2, 2, -2]      # CAST_TRUNC
    assert oracle.tcvt_f32_s32(z, 6).tolist() == [1, 1, 3, -1, -1, -3, 2, -3]     # CAST_ODD


# ------------------------------------------------------------------- gather
def test_tgather_index_is_numpy_take(oracle):
    o = oracle
    rng = np.random.default_rng(5)
    src = rng.integers(0, 2**16, size=(16, 1024), dtype=np.uint16)
    idx = rng.integers(0, 16 * 1024, size=(16, 128), dtype=np.int32)
    idx[0, :4] = [-1, 16 * 1024, 2**31 - 1, -2**31]          # out of range -> 0
    L0 = o.make_layout(16, 1024)
    L1 = o.make_layout(16, 128, elem_bytes=4)
    Ld = o.make_layout(16, 128)
    got = o.tgather_index(Ld, src.reshape(-1), L0, idx.reshape(-1), L1, 16, 128).reshape(16, 128)
    ok = (idx >= 0) & (idx < src.size)
    want = np.where(ok, src.reshape(-1)[np.clip(idx, 0, src.size - 1)], 0)
    assert np.array_equal(got, want)


def test_tgather_mask_is_strided_slice(oracle):
    o = oracle
    src = np.arange(16 * 64, dtype=np.uint16).reshape(16, 64)
    Ls = o.make_layout(16, 64)
    for pat, sl, div in [(1, slice(0, None, 2), 2), (2, slice(1, None, 2), 2), (3, slice(0, None, 4), 4),
                         (4, slice(1, None, 4), 4), (5, slice(2, None, 4), 4), (6, slice(3, None, 4), 4),
                         (7, slice(None), 1)]:
        Ld = o.make_layout(16, 64 // div)
        got, n = o.tgather_mask(Ld, src.reshape(-1), Ls, 16, 64, pat)
        assert n == 16 * 64 // div
        assert np.array_equal(got.reshape(16, -1), src[:, sl])


def test_gather_rows_equals_mgather_with_expanded_indices(oracle):
    """The row gather of the benchmark is MGATHER with idx[i,j] = idx[i]*cols + j."""
    o = oracle
    table, idx = datagen.gather_inputs(64, 128, 8)
    want = table[idx]
    assert np.array_equal(o.gather_rows(table, idx), want)
    full = (idx[:, None].astype(np.int64) * 128 + np.arange(128)[None, :]).astype(np.int32)
    Ld = o.make_layout(8, 128)
    Li = o.make_layout(8, 128, elem_bytes=4)
    got = o.mgather(Ld, table.reshape(-1), full.reshape(-1), Li, 8, 128).reshape(8, 128)
    assert np.array_equal(got, want)
    bad = np.array([3, -1, 64, 5], dtype=np.int32)
    out = o.gather_rows(table, bad)
    assert np.array_equal(out[0], table[3]) and not out[1].any() and not out[2].any()


def test_ref_gather(oracle, ref):
    o = oracle
    rng = np.random.default_rng(9)
    src = rng.integers(0, 2**16, size=(16, 1024), dtype=np.uint16)
    idx = rng.integers(-50, 16 * 1024 + 50, size=(16, 128), dtype=np.int32)
    out = np.zeros((16, 128), dtype=np.uint16)
    ref.ref_tgather_index_f16_16x1024_16x128(_p(out), _p(src), _p(idx))
    got = o.tgather_index(o.make_layout(16, 128), src.reshape(-1), o.make_layout(16, 1024), idx.reshape(-1),
                          o.make_layout(16, 128, elem_bytes=4), 16, 128)
    assert np.array_equal(out.reshape(-1), got)
    srcf = rng.standard_normal((32, 64)).astype(np.float32)
    idxf = rng.integers(0, 32 * 64, size=(32, 64), dtype=np.int32)
    outf = np.zeros((32, 64), dtype=np.float32)
    ref.ref_tgather_index_f32_32x64_32x64(_p(outf), _p(srcf), _p(idxf))
    assert np.array_equal(outf, srcf.reshape(-1)[idxf])
    # mask forms
    s16 = rng.integers(0, 2**16, size=(16, 64), dtype=np.uint16)
    o16 = np.zeros((16, 32), dtype=np.uint16)
    ref.ref_tgather_mask_f16_16x64_p0101(_p(o16), _p(s16))
    got, _ = o.tgather_mask(o.make_layout(16, 32), s16.reshape(-1), o.make_layout(16, 64), 16, 64, 1)
    assert np.array_equal(o16.reshape(-1), got) and np.array_equal(o16, s16[:, 0::2])
    s32 = rng.standard_normal((8, 64)).astype(np.float32)
    o32 = np.zeros((8, 16), dtype=np.float32)
    ref.ref_tgather_mask_f32_8x64_p1000(_p(o32), _p(s32))
    assert np.array_equal(o32, s32[:, 3::4])
    o64 = np.zeros((8, 64), dtype=np.float32)
    ref.ref_tgather_mask_f32_8x64_p1111(_p(o64), _p(s32))
    assert np.array_equal(o64, s32)
    # MGATHER
    gm = rng.integers(0, 2**16, size=65536, dtype=np.uint16)
    mi = rng.integers(0, 65536, size=(8, 128), dtype=np.int32)
    mo = np.zeros((8, 128), dtype=np.uint16)
    ref.ref_mgather_f16_8x128(_p(mo), _p(gm), _p(mi))
    assert np.array_equal(mo, gm[mi])
    got = o.mgather(o.make_layout(8, 128), gm, mi.reshape(-1), o.make_layout(8, 128, elem_bytes=4), 8, 128)
    assert np.array_equal(got, mo.reshape(-1))


# ---------------------------------------------------------------- attention
def _dense_attention_fp64(q, k, v, causal=False, q_offset=0):
    q, k, v = (t.astype(np.float64) for t in (q, k, v))
    s = q @ k.T / np.sqrt(q.shape[1])
    if causal:
        i = np.arange(q.shape[0])[:, None] + q_offset
        j = np.arange(k.shape[0])[None, :]
        s = np.where(j > i, -np.inf, s)
    m = s.max(axis=1, keepdims=True)
    p = np.exp(s - m)
    l = p.sum(axis=1, keepdims=True)
    return (p / l) @ v, (m + np.log(l)).reshape(-1)


def test_fa_auto_matches_fp64_golden(oracle):
    """Recipe of tflashattn/gen_data.py:31-58: S=64, D=32, seed 20251220, scale 0.02, fp64 golden, eps 2e-4."""
    rng = np.random.default_rng(20251220)
    q, k, v = ((rng.standard_normal((64, 32), dtype=np.float32) * 0.02).astype(np.float32) for _ in range(3))
    got = oracle.fa_auto_f32(q, k, v)
    want, _ = _dense_attention_fp64(q, k, v)
    ok, md, nbad = oracle.result_cmp(want.astype(np.float32), got, 2e-4)
    assert ok and nbad == 0 and md < 1e-6
    # larger magnitudes exercise the max subtraction (a missing subtraction overflows exp)
    q2 = (q * 3000).astype(np.float32)
    got2 = oracle.fa_auto_f32(q2, (k * 50).astype(np.float32), v)
    want2, _ = _dense_attention_fp64(q2, (k * 50).astype(np.float32), v)
    assert np.all(np.isfinite(got2)) and np.max(np.abs(got2 - want2)) < 1e-5


@pytest.mark.parametrize("name,S,D", [("ref_fa_auto_64x32", 64, 32), ("ref_fa_auto_128x64", 128, 64)])
def test_ref_fa_auto(oracle, ref, name, S, D):
    rng = np.random.default_rng(20251220)
    q, k, v = (rng.standard_normal((S, D), dtype=np.float32) for _ in range(3))
    out = np.zeros((S, D), dtype=np.float32)
    getattr(ref, name)(_p(out), _p(q), _p(k), _p(v))
    mine = oracle.fa_auto_f32(q, k, v)
    # vectorised row sums in the compiled reference may associate differently: a few ulp
    assert np.max(np.abs(out - mine)) < 2e-6
    want, _ = _dense_attention_fp64(q, k, v)
    assert np.max(np.abs(out - want)) < 1e-5


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("S0,S1,D,T", [(64, 256, 64, 64), (128, 512, 128, 256), (48, 200, 64, 128)])
def test_fa_stream_vs_dense_fp64(oracle, S0, S1, D, T, causal):
    q, k, v = datagen.fa_inputs(1, 1, S0, S1, D, scale=1.0)
    q, k, v = q[0, 0], k[0, 0], v[0, 0]
    q_off = S1 - S0 if causal else 0
    o, m, l = oracle.fa_stream_f16(q, k, v, tile_s1=T, causal=causal, q_offset=q_off)
    want, lse = _dense_attention_fp64(q, k, v, causal, q_off)
    rel = np.max(np.abs(o - want)) / np.max(np.abs(want))
    assert rel < 2e-3                                 # P is rounded to fp16: ~5e-4 expected
    got_lse = m.astype(np.float64) / np.sqrt(D) + np.log(l.astype(np.float64))
    assert np.max(np.abs(got_lse - lse)) < 1e-4


def test_fa_stream_invariants(oracle):
    q, k, v = datagen.fa_inputs(1, 1, 64, 512, 64)
    q, k, v = q[0, 0], k[0, 0], v[0, 0]
    a, ma, la = oracle.fa_stream_f16(q, k, v, tile_s1=64)
    b, mb, lb = oracle.fa_stream_f16(q, k, v, tile_s1=512)
    # tiling changes only rounding: running max equal, sums/outputs close
    assert np.array_equal(ma, mb)
    assert np.max(np.abs(la - lb) / lb) < 1e-5 and np.max(np.abs(a - b)) < 2e-3
    # causal: row i must not depend on keys > i
    o1, _, _ = oracle.fa_stream_f16(q, k[:64], v[:64], tile_s1=32, causal=True)
    k2, v2 = k[:64].copy(), v[:64].copy()
    k2[40:] = 0
    v2[40:] = 7
    o2, _, _ = oracle.fa_stream_f16(q, k2, v2, tile_s1=32, causal=True)
    assert np.array_equal(o1[:40], o2[:40]) and not np.array_equal(o1[40:], o2[40:])
    # constant V -> output is that constant for every row (softmax weights sum to 1)
    vc = np.full_like(v, 0.5)
    oc, _, _ = oracle.fa_stream_f16(q, k, vc, tile_s1=128)
    assert np.max(np.abs(oc - 0.5)) < 1e-3
    # ties-away vs RNE for the P cast differs only at rounding level
    orne, _, _ = oracle.fa_stream_f16(q, k, v, tile_s1=64, round_away=False)
    assert np.max(np.abs(orne - a)) < 1e-3


def test_result_cmp_semantics(oracle):
    e = np.ones(1000, dtype=np.float32)
    a = e.copy()
    a[0] = 1.01
    ok, md, nbad = oracle.result_cmp(e, a, 1e-3)
    assert ok and nbad == 1 and abs(md - 0.01) < 1e-6     # 1 bad <= floor(1000*1e-3)
    a[1] = 1.01
    ok, _, nbad = oracle.result_cmp(e, a, 1e-3)
    assert not ok and nbad == 2


# ------------------------------------------------------------------ MX GEMM
def _torch_fp8_table(fmt):
    import torch
    dt = torch.float8_e5m2 if fmt else torch.float8_e4m3fn
    return torch.arange(256, dtype=torch.int32).to(torch.uint8).view(dt).to(torch.float32).numpy()


@pytest.mark.parametrize("fmt", [0, 1])
def test_fp8_decode_matches_an_independent_implementation(oracle, fmt):
    """The oracle's and the data generator's fp8 decoders against torch's float8_e4m3fn / float8_e5m2 (all 256 bytes)."""
    from pto_amd import datagen
    want = _torch_fp8_table(fmt)
    got = oracle.fp8_table(fmt)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))      # signed zeros and infinities included
    gen = datagen.fp8_values(fmt).astype(np.float32)
    assert np.array_equal(np.isnan(gen), np.isnan(want)) and np.array_equal(gen[ok], want[ok])
    # known values: largest finite, smallest subnormal, one
    if fmt == 0:
        assert got[0x7E] == 448.0 and got[0x01] == 2.0 ** -9 and got[0x38] == 1.0
    else:
        assert got[0x7B] == 57344.0 and got[0x01] == 2.0 ** -16 and got[0x3C] == 1.0 and np.isinf(got[0x7C])


@pytest.mark.parametrize("fmt", [0, 1])
def test_fp8_encode_round_trips_and_rounds_to_nearest(fmt):
    import torch
    from pto_amd import datagen
    tab = datagen.fp8_values(fmt)
    finite = np.flatnonzero(np.isfinite(tab) & (np.arange(256) != 0x80))
    assert np.array_equal(datagen.fp8_encode(tab[finite], fmt), finite.astype(np.uint8))
    x = np.random.Generator(np.random.Philox(key=5)).uniform(-5, 5, size=4096)
    got = tab[datagen.fp8_encode(x, fmt)]
    dt = torch.float8_e5m2 if fmt else torch.float8_e4m3fn
    want = torch.from_numpy(x).to(dt).to(torch.float64).numpy()
    # nearest value either way; only exact ties may differ (torch rounds them to even)
    assert np.all(np.abs(got - x) <= np.abs(want - x) + 1e-12)


@pytest.mark.parametrize("fmt", [0, 1])
def test_mx_gemm_oracle_closed_forms(oracle, fmt):
    from pto_amd import datagen
    m, n, k = 24, 40, 128
    a, b, sa, sb = datagen.mx_inputs(m, n, k, fmt, dist="integer")
    tab = _torch_fp8_table(fmt).astype(np.float64)          # decoded independently of the oracle
    ad = tab[a] * np.repeat(np.exp2(sa.astype(np.float64) - 127), 32, axis=1)
    bd = tab[b] * np.repeat(np.exp2(sb.astype(np.float64) - 127), 32, axis=1)
    got = oracle.mx_gemm(a, b, sa, sb, fmt)
    assert np.array_equal(got, (ad @ bd.T).astype(np.float32))                   # integers: exact
    # raising every scale of A by one doubles C; of one k block of B: adds that block's contribution once more
    assert np.array_equal(oracle.mx_gemm(a, b, sa + 1, sb, fmt), 2 * got)
    sb2 = sb.copy()
    sb2[:, 2] += 1
    extra = ad[:, 64:96] @ bd[:, 64:96].T
    assert np.array_equal(oracle.mx_gemm(a, b, sa, sb2, fmt), (ad @ bd.T + extra).astype(np.float32))
    # mixed operand formats
    a1, _, _, _ = datagen.mx_inputs(m, n, k, 1 - fmt, dist="integer")
    ad1 = _torch_fp8_table(1 - fmt).astype(np.float64)[a1] * np.repeat(np.exp2(sa.astype(np.float64) - 127), 32, axis=1)
    assert np.array_equal(oracle.mx_gemm(a1, b, sa, sb, 1 - fmt, fmt), (ad1 @ bd.T).astype(np.float32))
    # the generator's distribution, against a float64 matmul
    a, b, sa, sb = datagen.mx_inputs(m, n, k, fmt)
    ad = tab[a] * np.repeat(np.exp2(sa.astype(np.float64) - 127), 32, axis=1)
    bd = tab[b] * np.repeat(np.exp2(sb.astype(np.float64) - 127), 32, axis=1)
    assert np.allclose(oracle.mx_gemm(a, b, sa, sb, fmt), ad @ bd.T, rtol=1e-6, atol=1e-4)


def test_fp4_decode_and_mx_gemm_oracle_fp4(oracle):
    """float4_e2m1: the published value set (OCP MX: 0, 0.5, 1, 1.5, 2, 3, 4, 6), the bit-field formula, packing order, and
    the oracle's fp4 GEMM against a float64 matmul of independently decoded operands."""
    from pto_amd import datagen
    want = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6, -0.0, -0.5, -1, -1.5, -2, -3, -4, -6], dtype=np.float32)
    got = oracle.fp8_table(4)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(datagen.fp4_values().astype(np.float32), want)
    # formula: sign | 2-bit exponent (bias 1) | 1-bit mantissa, e = 0 subnormal
    for v in range(16):
        e, f = (v >> 1) & 3, v & 1
        mag = 0.5 * f if e == 0 else (1 + f / 2) * 2.0 ** (e - 1)
        assert abs(got[v]) == mag
    nib = np.arange(64, dtype=np.uint8).reshape(2, 32) % 16
    packed = datagen.fp4_pack(nib)
    assert packed[0, 0] == (nib[0, 0] | (nib[0, 1] << 4)) and np.array_equal(datagen.fp4_unpack(packed), nib)
    assert np.array_equal(datagen.fp8_encode(np.array([-6, -5, -1.2, 0, 0.2, 0.3, 2.4, 2.6, 5, 9]), 4),
                          np.array([15, 15, 10, 0, 0, 1, 4, 5, 6, 7], dtype=np.uint8))
    m, n, k = 16, 24, 128
    a, b, sa, sb = datagen.mx_inputs(m, n, k, 4, dist="bytes", scale_lo=120, scale_hi=135)
    assert a.shape == (m, k // 2)
    ad = want.astype(np.float64)[datagen.fp4_unpack(a)] * np.repeat(np.exp2(sa.astype(np.float64) - 127), 32, axis=1)
    bd = want.astype(np.float64)[datagen.fp4_unpack(b)] * np.repeat(np.exp2(sb.astype(np.float64) - 127), 32, axis=1)
    assert np.allclose(oracle.mx_gemm(a, b, sa, sb, 4), ad @ bd.T, rtol=1e-6, atol=0)
    a, b, sa, sb = datagen.mx_inputs(m, n, k, 4, dist="integer")
    ad = want.astype(np.float64)[datagen.fp4_unpack(a)] * np.repeat(np.exp2(sa.astype(np.float64) - 127), 32, axis=1)
    bd = want.astype(np.float64)[datagen.fp4_unpack(b)] * np.repeat(np.exp2(sb.astype(np.float64) - 127), 32, axis=1)
    assert np.array_equal(oracle.mx_gemm(a, b, sa, sb, 4), (ad @ bd.T).astype(np.float32))


# -------------------------------------------------------------------- top-k
def test_topk_oracle_matches_the_reference_golden_recipe(oracle):
    """np.lexsort((idx, -row))[:k], the recipe of kernels/manual/a2a3/topk/scripts/gen_data.py:55-64, on its distribution, on
    rows with many ties, signed zeros and infinities, and with indices that are not the column numbers."""
    from pto_amd import datagen
    rows, cols, ld, k = 12, 300, 320, 123
    for distinct in (0, 5):
        src, idx = datagen.topk_inputs(rows, cols, ld, distinct=distinct)
        src[1, ::7] = -0.0
        src[2, ::5] = np.inf
        src[3, 1::6] = -np.inf
        r = np.random.Generator(np.random.Philox(key=3))
        for index in (idx, r.permutation(5000)[:cols].astype(np.uint32)):
            s, i = oracle.topk_f32(src, index, cols, k)
            for row in range(rows):
                v = src[row, :cols]
                order = np.lexsort((index, -v))[:k]
                assert np.array_equal(i[row], index[order])
                assert np.array_equal(s[row].view(np.uint32), v[order].view(np.uint32))
    # known answer
    s, i = oracle.topk_f32(np.array([[1.0, 3.0, 2.0, 3.0, -1.0, 9.0]], dtype=np.float32), np.arange(5, dtype=np.uint32), 5, 3)
    assert s.tolist() == [[3.0, 3.0, 2.0]] and i.tolist() == [[1, 3, 2]]


# ------------------------------------------------------------ multi-latent attention (the Auto-mode demo)
MLA_GOLD = os.path.join(os.path.dirname(__file__), "golden", "ref_mla.npz")


def _rel_to_max(got, want):
    return float(np.max(np.abs(got.astype(np.float64) - want)) / np.max(np.abs(want)))


@pytest.mark.parametrize("case,scales", [("demo_scale", (0.02, 0.02)), ("peaked", (1.0, 0.5))])
def test_mla_oracle_vs_reference_outputs(oracle, case, scales):
    """The float64 restatement against what the reference's CPU simulation produced for the same program (committed
    outputs; also the compiled reference itself where it is built): an fp32 chain of five matmuls and a softmax
    agrees with float64 to ~1e-6 of the largest output; a wrong scale, transposed weight or missing stage does not."""
    args = datagen.mla_inputs(1, 2, *scales)
    want = oracle.mla_attention(*args)
    gold = np.load(MLA_GOLD)["mla_" + case]
    assert _rel_to_max(gold, want.astype(np.float64)) < 5e-6
    assert oracle.mla_verify_allclose(gold, want) == 0          # the demo's own acceptance test
    r = oracle.ref()
    if r is not None:
        q, k, v, wq, wk, wv, wo = args
        for h in range(2):
            o = np.zeros((64, 32), dtype=np.float32)
            r.ref_mla_auto_64x32x16(_p(o), _p(np.ascontiguousarray(q[0, h])), _p(np.ascontiguousarray(k[0, h])),
                                    _p(np.ascontiguousarray(v[0, h])), _p(wq), _p(wk), _p(wv), _p(wo))
            assert np.array_equal(o, gold[0, h])


def test_mla_oracle_closed_forms(oracle):
    from scipy.special import softmax
    q, k, v, wq, wk, wv, wo = datagen.mla_inputs(2, 3, 1.0, 0.5, seed=5)
    # no key projection: all scores are zero, the softmax is uniform, every position gets mean(V) Wv Wo
    out = oracle.mla_attention(q, k, v, wq, np.zeros_like(wk), wv, wo)
    want = (v.astype(np.float64).mean(axis=2, keepdims=True) @ wv.astype(np.float64)) @ wo.astype(np.float64)
    assert np.max(np.abs(out - np.broadcast_to(want, out.shape))) < 1e-6
    # associativity: P (V (Wv Wo)) with a library softmax of Q (Wq Wk^T) K^T / sqrt(R)
    out = oracle.mla_attention(q, k, v, wq, wk, wv, wo)
    q64, k64, v64 = (t.astype(np.float64) for t in (q, k, v))
    sc = q64 @ (wq.astype(np.float64) @ wk.astype(np.float64).T) @ np.swapaxes(k64, 2, 3) / 4.0
    want = softmax(sc, axis=-1) @ (v64 @ (wv.astype(np.float64) @ wo.astype(np.float64)))
    assert np.max(np.abs(out - want)) < 1e-6 * np.max(np.abs(want))
    # one key far ahead of the others: the output row is that key's value row projected
    q1, k1 = np.zeros_like(q), np.zeros_like(k)
    q1[..., 0], k1[:, :, 17, 0] = 40.0, 40.0
    w1 = np.zeros_like(wq)
    w1[0, 0] = 1.0
    out = oracle.mla_attention(q1, k1, v, w1, w1, wv, wo)
    want = (v64[:, :, 17:18] @ wv.astype(np.float64)) @ wo.astype(np.float64)
    assert np.max(np.abs(out - np.broadcast_to(want, out.shape))) < 1e-6
    # the acceptance test counts what it should
    assert oracle.mla_verify_allclose(np.array([1.0, 2.0, np.nan, 0.0]), np.array([1.0001, 2.1, 0.0, 0.0])) == 2


# ---------------------------------------------------------------- MXFP8 quantisation (TQUANT<QuantType::MXFP8>)
def _e4m3_grid():
    tab = datagen.fp8_values(0)
    vals = np.sort(np.unique(tab[np.isfinite(tab)]))
    return tab, vals


def test_fp8_e4m3_encoder_against_torch_and_the_value_table(oracle):
    """The oracle's fp32 -> e4m3fn encoder: every representable value maps to its own byte, every midpoint between two
    neighbours goes to the one with the even code (ties) and its fp32 neighbours to the nearer value, random values agree
    with torch's float8_e4m3fn cast, magnitudes above 448 saturate, NaN keeps its sign."""
    import torch
    tab, vals = _e4m3_grid()
    mids = ((vals[:-1] + vals[1:]) / 2).astype(np.float32)            # exact in fp32
    rng = np.random.default_rng(3)
    x = np.concatenate([vals.astype(np.float32), mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)),
                        rng.uniform(-448, 448, 30000).astype(np.float32), (rng.standard_normal(30000) * 0.02).astype(np.float32)])
    got = oracle.fp8_e4m3_encode(x)
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(got, want)
    # nearest value by brute force over the table (independent of any cast); at a tie the even code
    dec = tab[got].astype(np.float64)
    best = np.min(np.abs(x.astype(np.float64)[:, None] - vals[None, :]), axis=1)
    assert np.array_equal(np.abs(dec - x.astype(np.float64)), best)
    tie = oracle.fp8_e4m3_encode(mids)
    assert not (tie & 1).any()
    sat = oracle.fp8_e4m3_encode(np.array([448, 448.5, 479, 480, 1e30, np.inf, -449, -np.inf], dtype=np.float32))
    assert list(sat) == [0x7e] * 6 + [0xfe] * 2
    nan = oracle.fp8_e4m3_encode(np.array([np.nan, -np.nan], dtype=np.float32))
    assert list(nan & 0x7f) == [0x7f, 0x7f]


def test_quant_mxfp8_oracle_closed_forms(oracle):
    """Scale byte = floor(log2(amax)) + 119; elements = e4m3(x * 2^(127 - scale byte)) computed with torch's cast; the
    largest element of a group lands in [256, 448]; dequantised values are within 2^-4 relative (half a step of a 3-bit
    mantissa) of every element that is not far below its group's maximum; scaling a group by a power of two moves only
    the scale byte."""
    import torch
    rows, cols = 37, 1024
    x = datagen.quant_input(rows, cols, specials=False)
    q, s, amax, scale = oracle.quant_mxfp8(x, with_stats=True)
    g = np.abs(x).reshape(rows, cols // 32, 32).max(axis=2)
    assert np.array_equal(amax, g)
    _, ex = np.frexp(g)
    assert np.array_equal(s, (ex - 1 + 119).astype(np.uint8))
    assert np.array_equal(scale, np.exp2(127.0 - s.astype(np.float64)).astype(np.float32))
    y = np.clip(x.astype(np.float64) * np.repeat(np.exp2(127.0 - s.astype(np.float64)), 32, axis=1), -448, 448).astype(np.float32)
    assert np.array_equal(q, torch.from_numpy(y).to(torch.float8_e4m3fn).view(torch.uint8).numpy())
    tab = datagen.fp8_values(0)
    top = np.abs(tab[q]).reshape(rows, cols // 32, 32).max(axis=2)
    assert top.min() >= 256 and top.max() <= 448
    deq = tab[q] * np.repeat(np.exp2(s.astype(np.float64) - 127.0), 32, axis=1)
    big = np.abs(x) >= np.repeat(g, 32, axis=1) * 2.0 ** -7          # normal e4m3 range below the group's top
    clipped = np.abs(y) >= 448
    err = np.abs(deq - x)[big & ~clipped] / np.abs(x)[big & ~clipped]
    assert err.max() <= 2.0 ** -4
    q2, s2 = oracle.quant_mxfp8(x * np.float32(2.0 ** 5))
    assert np.array_equal(q2, q) and np.array_equal(s2.astype(int), s.astype(int) + 5)


def test_quant_mxfp8_oracle_special_groups(oracle):
    """Zero and tiny groups: scale byte 0, factor 2^127; groups with an infinity or NaN: scale byte 0xff, NaN -> NaN,
    infinities -> +-448, finite -> signed zero; an element at -0 stays -0."""
    z = np.zeros((1, 32), dtype=np.float32)
    q, s = oracle.quant_mxfp8(z)
    assert s[0, 0] == 0 and not q.any()
    t = np.full((1, 32), 2.0 ** -125, dtype=np.float32)
    t[0, 1] = -2.0 ** -121
    q, s, _, scale = oracle.quant_mxfp8(t, with_stats=True)
    assert s[0, 0] == 0 and scale[0, 0] == np.float32(2.0 ** 127)
    assert q[0, 0] == 0x48 and q[0, 1] == 0xe8          # 2^-125 * 2^127 = 4 -> 0.1001.000; -2^-121 * 2^127 = -64 -> 1.1101.000
    w = np.ones((1, 64), dtype=np.float32)
    w[0, 3], w[0, 4], w[0, 5], w[0, 6] = np.inf, -np.inf, np.nan, -5.0
    w[0, 40] = -0.0
    q, s = oracle.quant_mxfp8(w)
    assert s[0, 0] == 0xff and s[0, 1] == 127 - 8
    assert q[0, 3] == 0x7e and q[0, 4] == 0xfe and (q[0, 5] & 0x7f) == 0x7f and q[0, 6] == 0x80 and q[0, 0] == 0
    assert q[0, 40] == 0x80 and q[0, 41] == 0x78         # 1.0 * 2^8 = 256 -> 0.1111.000
