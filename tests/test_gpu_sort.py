"""GPU parity of TSORT32 and TMRGSORT (single-tile programs through the C ABI): bit-exact against the oracle and, where
the two agree by construction, against the committed outputs of the reference's CPU simulation."""
import os

import numpy as np
import pytest
import torch

import sort_cases as sc
from pto_amd import capi

pytestmark = pytest.mark.gpu

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_sort.npz"))


def _dev(a):
    from gpu_util import to_dev
    return to_dev(a)


def _st():
    from gpu_util import stream
    return stream()


@pytest.mark.parametrize("dtype,vr,vc,seed", sc.SORT32_CASES)
def test_tsort32(oracle, dtype, vr, vc, seed):
    lib = capi.load_st()
    src, idx, out0 = sc.sort32_inputs(dtype, vr, vc, seed)
    ts, ti, to = _dev(src), _dev(idx), _dev(out0)
    capi.check(lib.pto_st_tsort32_8x128(_st(), to.data_ptr(), ts.data_ptr(), ti.data_ptr(), vr, vc, 0 if dtype == "f32" else 1), "tsort32")
    torch.cuda.synchronize()
    got = to.cpu().numpy().view(np.uint32)
    want = oracle.tsort32(out0, src, idx, vr, vc).view(np.uint32)              # index as its bit pattern (the NPU form)
    # equal scores of different sign of zero may come out in either bit pattern only if they tie on the index too;
    # the inputs have no such pair, so the comparison is on bits
    assert np.array_equal(got, want)
    if dtype == "s32":                                                         # for int32 tiles the CPU simulation's form is the same
        assert np.array_equal(got, GOLD["sort32_%d" % seed].view(np.uint32))


@pytest.mark.parametrize("valid_cols,block_len,seed", sc.BLOCK_CASES)
def test_tmrgsort_blocks(oracle, valid_cols, block_len, seed):
    lib = capi.load_st()
    src, out0 = sc.block_inputs(valid_cols, block_len, seed)
    ts, to = _dev(src), _dev(out0)
    capi.check(lib.pto_st_tmrgsort_blocks_f32_1x1024(_st(), to.data_ptr(), ts.data_ptr(), valid_cols, block_len), "tmrgsort blocks")
    torch.cuda.synchronize()
    got = to.cpu().numpy().view(np.uint32)
    assert np.array_equal(got, oracle.tmrgsort_blocks(out0, src, valid_cols, block_len).view(np.uint32))
    assert np.array_equal(got, GOLD["blocks_%d" % seed])


@pytest.mark.parametrize("counts,out_structs,exhausted,seed", sc.LIST_CASES)
def test_tmrgsort_lists(oracle, counts, out_structs, exhausted, seed):
    lib = capi.load_st()
    lists, out0 = sc.list_inputs(counts, seed)
    tl = [_dev(l) for l in lists]
    to = _dev(out0)
    tex = torch.full((4,), -1, dtype=torch.int32, device="cuda:0")
    ptrs = [t.data_ptr() for t in tl] + [0] * (4 - len(tl))
    cols = [2 * n for n in counts] + [0] * (4 - len(counts))
    capi.check(lib.pto_st_tmrgsort_lists_f32(_st(), to.data_ptr(), tex.data_ptr(), *ptrs, *cols, 2 * out_structs, len(counts), exhausted),
               "tmrgsort lists")
    torch.cuda.synchronize()
    got, ex = to.cpu().numpy().view(np.uint32), tex.cpu().numpy().view(np.uint32)
    want, want_ex = oracle.tmrgsort_lists(out0, lists, cols[:len(counts)], 2 * out_structs, exhausted)
    assert np.array_equal(ex, want_ex)
    assert np.array_equal(got, want.view(np.uint32))
    assert np.array_equal(got, GOLD["lists_%d" % seed]) and np.array_equal(ex, GOLD["lists_%d_executed" % seed])


@pytest.mark.parametrize("dtype,vr,vc,seed", sc.SORT32_CASES_16)
def test_tsort32_16bit(oracle, dtype, vr, vc, seed):
    """fp16 / int16 scores: structures of four elements (score, 0, index & 0xffff, index >> 16), the index as its bits."""
    lib = capi.load_st()
    src, idx, out0 = sc.sort32_inputs_16(dtype, vr, vc, seed)
    ts, ti, to = _dev(src.view(np.int16)), _dev(idx), _dev(out0.view(np.int16))
    capi.check(lib.pto_st_tsort32_8x128(_st(), to.data_ptr(), ts.data_ptr(), ti.data_ptr(), vr, vc, 2 if dtype == "f16" else 3), "tsort32")
    torch.cuda.synchronize()
    got = to.cpu().numpy().view(np.uint16)
    assert np.array_equal(got, oracle.tsort32(out0, src, idx, vr, vc).view(np.uint16))
    if dtype == "s16" and vc <= 32:          # there the CPU simulation's by-value form is the same thing
        assert np.array_equal(got, GOLD["sort32_%d" % seed])


@pytest.mark.parametrize("dtype,valid_cols,block_len,seed", sc.BLOCK_CASES_16)
def test_tmrgsort_blocks_16bit(oracle, dtype, valid_cols, block_len, seed):
    lib = capi.load_st()
    src, out0 = sc.block_inputs_16(dtype, valid_cols, block_len, seed)
    ts, to = _dev(src.view(np.int16)), _dev(out0.view(np.int16))
    capi.check(lib.pto_st_tmrgsort_blocks_16_1x2048(_st(), to.data_ptr(), ts.data_ptr(), valid_cols, block_len, sc.DT16[dtype]), "tmrgsort blocks")
    torch.cuda.synchronize()
    got = to.cpu().numpy().view(np.uint16)
    assert np.array_equal(got, oracle.tmrgsort_blocks(out0, src, valid_cols, block_len).view(np.uint16))
    assert np.array_equal(got, GOLD["blocks_%d" % seed])


@pytest.mark.parametrize("dtype,counts,out_structs,exhausted,seed", sc.LIST_CASES_16)
def test_tmrgsort_lists_16bit(oracle, dtype, counts, out_structs, exhausted, seed):
    lib = capi.load_st()
    lists, out0 = sc.list_inputs_16(dtype, counts, seed)
    tl = [_dev(l.view(np.int16)) for l in lists]
    to = _dev(out0.view(np.int16))
    tex = torch.full((4,), -1, dtype=torch.int32, device="cuda:0")
    ptrs = [t.data_ptr() for t in tl] + [0] * (4 - len(tl))
    cols = [4 * n for n in counts] + [0] * (4 - len(counts))
    capi.check(lib.pto_st_tmrgsort_lists_16(_st(), to.data_ptr(), tex.data_ptr(), *ptrs, *cols, 4 * out_structs, len(counts), exhausted,
                                            sc.DT16[dtype]), "tmrgsort lists")
    torch.cuda.synchronize()
    got, ex = to.cpu().numpy().view(np.uint16), tex.cpu().numpy().view(np.uint32)
    want, want_ex = oracle.tmrgsort_lists(out0, lists, cols[:len(counts)], 4 * out_structs, exhausted)
    assert np.array_equal(ex, want_ex)
    assert np.array_equal(got, want.view(np.uint16))
    assert np.array_equal(got, GOLD["lists_%d" % seed]) and np.array_equal(ex, GOLD["lists_%d_executed" % seed])


@pytest.mark.parametrize("n", range(len(sc.PART_CASES)))
def test_tpart(oracle, n):
    lib = capi.load_st()
    op, dv, av, bv = sc.PART_CASES[n]
    a, b, out0 = sc.part_inputs(n)
    ta, tb, to = _dev(a), _dev(b), _dev(out0)
    capi.check(lib.pto_st_tpart_f32_64x128(_st(), to.data_ptr(), ta.data_ptr(), tb.data_ptr(), op, *dv, *av, *bv), "tpart")
    torch.cuda.synchronize()
    got = to.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), oracle.tpart(out0, a, b, op, dv, av, bv).view(np.uint32))
    assert np.array_equal(got[::3].view(np.uint32), GOLD["part_%d" % n].view(np.uint32))


@pytest.mark.parametrize("n", range(len(sc.SCATTER_CASES)))
def test_tscatter_and_mscatter(oracle, n):
    lib = capi.load_st()
    vr, vc, kind = sc.SCATTER_CASES[n]
    src, idx, out0 = sc.scatter_inputs(vr, vc, kind, n)
    ts, ti, to = _dev(src), _dev(idx), _dev(out0)
    capi.check(lib.pto_st_scatter_f32_64x128(_st(), to.data_ptr(), ts.data_ptr(), ti.data_ptr(), vr, vc, 0), "tscatter")
    torch.cuda.synchronize()
    got = to.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), oracle.tscatter(out0, src, idx, vr, vc).view(np.uint32))      # incl. "last row wins"
    assert np.array_equal(got[::3].view(np.uint32), GOLD["tscatter_%d" % n].view(np.uint32))
    msrc, midx, mem0 = sc.mscatter_inputs(vr, vc, n)
    ts, ti, tm = _dev(msrc), _dev(midx), _dev(mem0)
    capi.check(lib.pto_st_scatter_f32_64x128(_st(), tm.data_ptr(), ts.data_ptr(), ti.data_ptr(), vr, vc, 1), "mscatter")
    torch.cuda.synchronize()
    mgot = tm.cpu().numpy()
    assert np.array_equal(mgot.view(np.uint32), oracle.mscatter(mem0, msrc, midx, vr, vc).view(np.uint32))
    assert np.array_equal(mgot[::3].view(np.uint32), GOLD["mscatter_%d" % n].view(np.uint32))


@pytest.mark.parametrize("n", range(len(sc.GATHERB_CASES)))
def test_tgatherb(oracle, n):
    lib = capi.load_st()
    vr, vc, kind = sc.GATHERB_CASES[n]
    src, off, out0 = sc.gatherb_inputs(kind, n)
    ts, tf, to = _dev(src), _dev(off), _dev(out0)
    capi.check(lib.pto_st_tgatherb_f32_16x128(_st(), to.data_ptr(), ts.data_ptr(), tf.data_ptr(), vr, vc), "tgatherb")
    torch.cuda.synchronize()
    got = to.cpu().numpy().view(np.uint32)
    assert np.array_equal(got, oracle.tgatherb(out0, src, off, vr, vc).view(np.uint32))
    assert np.array_equal(got, GOLD["gatherb_%d" % n].view(np.uint32))


@pytest.mark.parametrize("n", range(len(sc.CI_CASES)))
def test_tci(oracle, n):
    lib = capi.load_st()
    start, desc, vc = sc.CI_CASES[n]
    out0 = np.full(1024, -5, dtype=np.int32)
    to = _dev(out0)
    capi.check(lib.pto_st_tci_s32_1x1024(_st(), to.data_ptr(), start, desc, vc), "tci")
    torch.cuda.synchronize()
    got = to.cpu().numpy()
    assert np.array_equal(got, oracle.tci(out0, start, desc, vc)) and np.array_equal(got, GOLD["tci_%d" % n])


def test_sort_programs_reject_bad_arguments():
    lib = capi.load_st()
    p = torch.zeros(2048, device="cuda:0").data_ptr()
    assert lib.pto_st_tsort32_8x128(0, p, p, p, 9, 32, 0) == capi.ERR_BAD_ARG
    assert lib.pto_st_tpart_f32_64x128(0, p, p, p, 3, 64, 128, 64, 128, 64, 128) == capi.ERR_BAD_ARG
    assert lib.pto_st_tpart_f32_64x128(0, p, p, p, 0, 65, 128, 64, 128, 64, 128) == capi.ERR_BAD_ARG
    assert lib.pto_st_tmrgsort_blocks_f32_1x1024(0, p, p, 2048, 64) == capi.ERR_BAD_ARG
    assert lib.pto_st_tmrgsort_lists_f32(0, p, p, p, p, 0, 0, 64, 64, 64, 0, 256, 3, 0) == capi.ERR_BAD_ARG      # third list missing
    assert lib.pto_st_tmrgsort_lists_f32(0, p, p, p, p, p, p, 63, 64, 64, 64, 256, 4, 0) == capi.ERR_BAD_ARG      # odd column count
