"""Pins the oracle's TSORT32 / TMRGSORT restatements (CPU only) against the committed outputs of the reference's CPU
simulation (tests/golden/ref_sort.npz; the compiled reference itself where it is built) and against numpy's sorts."""
import ctypes as C
import os

import numpy as np
import pytest

import sort_cases as sc

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_sort.npz"))


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


@pytest.mark.parametrize("dtype,vr,vc,seed", sc.SORT32_CASES)
def test_tsort32_vs_reference_and_lexsort(oracle, dtype, vr, vc, seed):
    src, idx, out0 = sc.sort32_inputs(dtype, vr, vc, seed)
    # the CPU simulation stores the index converted by value
    got = oracle.tsort32(out0, src, idx, vr, vc, index_as_value=True)
    assert np.array_equal(got.view(np.uint32), GOLD["sort32_%d" % seed].view(np.uint32))
    r = oracle.ref()
    if r is not None:
        o = out0.copy()
        (r.ref_tsort32_f32_8x128 if dtype == "f32" else r.ref_tsort32_s32_8x128)(_p(o), _p(src), _p(idx), vr, vc)
        assert np.array_equal(o.view(np.uint32), got.view(np.uint32))
    # the bit-pattern form against numpy: per group, lexsort by (-score, index), position last
    bits = oracle.tsort32(out0, src, idx, vr, vc)
    for row in range(vr):
        for j in range(0, vc, 32):
            n = min(32, vc - j)
            s = src[row, j:j + n].astype(np.float64)
            order = np.lexsort((np.arange(n), idx[row, j:j + n], -s))
            assert np.array_equal(bits[row, 2 * j:2 * (j + n):2], src[row, j + order])      # values (-0 == +0 may swap bits)
            assert np.array_equal(bits[row, 2 * j + 1:2 * (j + n):2].view(np.uint32), idx[row, j + order])
    # untouched: rows beyond the valid ones and columns beyond twice the valid ones
    assert np.array_equal(bits[vr:], out0[vr:]) and np.array_equal(bits[:, 2 * vc:], out0[:, 2 * vc:])


@pytest.mark.parametrize("valid_cols,block_len,seed", sc.BLOCK_CASES)
def test_tmrgsort_blocks_vs_reference_and_stable_sort(oracle, valid_cols, block_len, seed):
    src, out0 = sc.block_inputs(valid_cols, block_len, seed)
    got = oracle.tmrgsort_blocks(out0, src, valid_cols, block_len)
    assert np.array_equal(got.view(np.uint32), GOLD["blocks_%d" % seed])
    r = oracle.ref()
    if r is not None:
        o = out0.copy()
        r.ref_tmrgsort_blocks_f32_1x1024(_p(o), _p(src), valid_cols, block_len)
        assert np.array_equal(o.view(np.uint32), got.view(np.uint32))
    # merging sorted blocks = a stable sort of their concatenation by descending score
    group = 4 * block_len
    done = valid_cols // group * group
    for c in range(0, done, group):
        st = src[c:c + group].reshape(-1, 2)
        order = np.argsort(-st[:, 0], kind="stable")
        assert np.array_equal(got[c:c + group].view(np.uint32), st[order].reshape(-1).view(np.uint32))
    assert np.array_equal(got[done:], out0[done:])


@pytest.mark.parametrize("dtype,vr,vc,seed", sc.SORT32_CASES_16)
def test_tsort32_16bit_vs_reference_and_lexsort(oracle, dtype, vr, vc, seed):
    """2-byte scores: the by-value form (with the CPU simulation's group offset 2 j) against the compiled reference's
    committed outputs; the bit-pattern form, four elements a structure at 4 j, against numpy's lexsort."""
    src, idx, out0 = sc.sort32_inputs_16(dtype, vr, vc, seed)
    got = oracle.tsort32(out0, src, idx, vr, vc, index_as_value=True)
    assert np.array_equal(got.view(np.uint16), GOLD["sort32_%d" % seed])
    r = oracle.ref()
    if r is not None:
        o = out0.copy()
        (r.ref_tsort32_f16_8x128 if dtype == "f16" else r.ref_tsort32_s16_8x128)(_p(o), _p(src), _p(idx), vr, vc)
        assert np.array_equal(o.view(np.uint16), got.view(np.uint16))
    bits = oracle.tsort32(out0, src, idx, vr, vc)
    if dtype == "s16" and vc <= 32:          # integer conversions keep the bits and one group has nothing to overlap: the two forms agree
        assert np.array_equal(bits, got)
    for row in range(vr):
        for j in range(0, vc, 32):
            n = min(32, vc - j)
            order = np.lexsort((np.arange(n), idx[row, j:j + n], -src[row, j:j + n].astype(np.float64)))
            st = bits[row, 4 * j:4 * (j + n)].reshape(n, 4)
            assert np.array_equal(st[:, 0], src[row, j + order])
            assert not st[:, 1].view(np.uint16).any()
            assert np.array_equal(st[:, 2:].copy().view(np.uint16).astype(np.uint32) @ np.array([1, 65536], dtype=np.uint32),
                                  idx[row, j + order])
    assert np.array_equal(bits[vr:], out0[vr:]) and np.array_equal(bits[:, 4 * vc:], out0[:, 4 * vc:])


@pytest.mark.parametrize("dtype,valid_cols,block_len,seed", sc.BLOCK_CASES_16)
def test_tmrgsort_blocks_16bit_vs_reference_and_stable_sort(oracle, dtype, valid_cols, block_len, seed):
    src, out0 = sc.block_inputs_16(dtype, valid_cols, block_len, seed)
    got = oracle.tmrgsort_blocks(out0, src, valid_cols, block_len)
    assert np.array_equal(got.view(np.uint16), GOLD["blocks_%d" % seed])
    r = oracle.ref()
    if r is not None:
        o = out0.copy()
        r.ref_tmrgsort_blocks_16_1x2048(_p(o), _p(src), valid_cols, block_len, sc.DT16[dtype])
        assert np.array_equal(o.view(np.uint16), got.view(np.uint16))
    done = 0
    if block_len % 4 == 0:                   # a block length that is not whole structures merges nothing
        group = 4 * block_len
        done = valid_cols // group * group
        for c in range(0, done, group):
            st = src[c:c + group].reshape(-1, 4)
            order = np.argsort(-st[:, 0].astype(np.float64), kind="stable")      # uint16 scores order as unsigned numbers
            assert np.array_equal(got[c:c + group].view(np.uint16), st[order].reshape(-1).view(np.uint16))
    assert np.array_equal(got[done:], out0[done:])


@pytest.mark.parametrize("dtype,counts,out_structs,exhausted,seed", sc.LIST_CASES_16)
def test_tmrgsort_lists_16bit_vs_reference_and_stable_sort(oracle, dtype, counts, out_structs, exhausted, seed):
    lists, out0 = sc.list_inputs_16(dtype, counts, seed)
    got, ex = oracle.tmrgsort_lists(out0, lists, [4 * n for n in counts], 4 * out_structs, exhausted)
    assert np.array_equal(got.view(np.uint16), GOLD["lists_%d" % seed])
    assert np.array_equal(ex, GOLD["lists_%d_executed" % seed])
    r = oracle.ref()
    if r is not None:
        o, e = out0.copy(), np.zeros(4, dtype=np.uint32)
        ptrs = [_p(l) for l in lists] + [None] * (4 - len(lists))
        cols = [4 * n for n in counts] + [0] * (4 - len(counts))
        r.ref_tmrgsort_lists_16(_p(o), _p(e), *ptrs, *cols, 4 * out_structs, len(counts), exhausted, sc.DT16[dtype])
        assert np.array_equal(o.view(np.uint16), got.view(np.uint16)) and np.array_equal(e, ex)
    cat = np.concatenate([l[:4 * n].reshape(-1, 4) for l, n in zip(lists, counts)])
    full = cat[np.argsort(-cat[:, 0].astype(np.float64), kind="stable")] if len(cat) else cat
    taken = int(ex.sum())
    assert taken <= min(out_structs, len(cat))
    assert np.array_equal(got[:4 * taken].view(np.uint16), full[:taken].reshape(-1).view(np.uint16))
    assert np.array_equal(got[4 * taken:], out0[4 * taken:])


@pytest.mark.parametrize("counts,out_structs,exhausted,seed", sc.LIST_CASES)
def test_tmrgsort_lists_vs_reference_and_stable_sort(oracle, counts, out_structs, exhausted, seed):
    lists, out0 = sc.list_inputs(counts, seed)
    got, ex = oracle.tmrgsort_lists(out0, lists, [2 * n for n in counts], 2 * out_structs, exhausted)
    assert np.array_equal(got.view(np.uint32), GOLD["lists_%d" % seed])
    assert np.array_equal(ex, GOLD["lists_%d_executed" % seed])
    r = oracle.ref()
    if r is not None:
        o, e = out0.copy(), np.zeros(4, dtype=np.uint32)
        ptrs = [_p(l) for l in lists] + [None] * (4 - len(lists))
        cols = [2 * n for n in counts] + [0] * (4 - len(counts))
        r.ref_tmrgsort_lists_f32(_p(o), _p(e), *ptrs, *cols, 2 * out_structs, len(counts), exhausted)
        assert np.array_equal(o.view(np.uint32), got.view(np.uint32)) and np.array_equal(e, ex)
    # the merged prefix is a prefix of the stable sort of the concatenation; the counts say where it stops
    cat = np.concatenate([l[:2 * n].reshape(-1, 2) for l, n in zip(lists, counts)])
    full = cat[np.argsort(-cat[:, 0], kind="stable")] if len(cat) else cat
    taken = int(ex.sum())
    assert taken <= min(out_structs, len(cat))
    assert np.array_equal(got[:2 * taken].view(np.uint32), full[:taken].reshape(-1).view(np.uint32))
    assert np.array_equal(got[2 * taken:], out0[2 * taken:])
    if not exhausted:
        assert taken == min(out_structs, len(cat))
    elif taken < min(out_structs, len(cat)):
        assert any(int(ex[b]) == n for b, n in enumerate(counts))        # it stopped because a list ran empty


@pytest.mark.parametrize("n", range(len(sc.PART_CASES)))
def test_tpart_vs_reference(oracle, n):
    """TPARTADD / TPARTMAX / TPARTMIN against the reference's CPU simulation (committed outputs, every third row; all
    rows where the compiled reference is built) and against the definition applied region by region."""
    op, dv, av, bv = sc.PART_CASES[n]
    a, b, out0 = sc.part_inputs(n)
    got = oracle.tpart(out0, a, b, op, dv, av, bv)
    assert np.array_equal(got[::3].view(np.uint32), GOLD["part_%d" % n].view(np.uint32))
    r = oracle.ref()
    if r is not None:
        o = out0.copy()
        r.ref_tpart_f32_64x128(_p(o), _p(a), _p(b), op, *dv, *av, *bv)
        assert np.array_equal(o.view(np.uint32), got.view(np.uint32))
    f = [np.add, np.maximum, np.minimum][op]
    rr, cc = min(dv[0], av[0], bv[0]), min(dv[1], av[1], bv[1])
    assert np.array_equal(got[:rr, :cc], f(a[:rr, :cc], b[:rr, :cc]))                    # both valid
    assert np.array_equal(got[dv[0]:], out0[dv[0]:]) and np.array_equal(got[:, dv[1]:], out0[:, dv[1]:])   # outside dst: untouched
    none = np.zeros((64, 128), dtype=bool)
    none[:dv[0], :dv[1]] = True
    none[:av[0], :av[1]] = False
    none[:bv[0], :bv[1]] = False
    assert np.all(got[none] == 0)                                                          # neither source valid


@pytest.mark.parametrize("n", range(len(sc.SCATTER_CASES)))
def test_scatter_vs_reference(oracle, n):
    """TSCATTER / MSCATTER against the reference's CPU simulation (committed outputs, every third element row / word;
    everything where the compiled reference is built), and as the inverse of a gather where the indices are a permutation."""
    vr, vc, kind = sc.SCATTER_CASES[n]
    src, idx, out0 = sc.scatter_inputs(vr, vc, kind, n)
    got = oracle.tscatter(out0, src, idx, vr, vc)
    assert np.array_equal(got[::3].view(np.uint32), GOLD["tscatter_%d" % n].view(np.uint32))
    msrc, midx, mem0 = sc.mscatter_inputs(vr, vc, n)
    mgot = oracle.mscatter(mem0, msrc, midx, vr, vc)
    assert np.array_equal(mgot[::3].view(np.uint32), GOLD["mscatter_%d" % n].view(np.uint32))
    r = oracle.ref()
    if r is not None:
        o = out0.copy()
        r.ref_tscatter_f32_64x128(_p(o), _p(src), _p(idx), vr, vc)
        assert np.array_equal(o.view(np.uint32), got.view(np.uint32))
        m = mem0.copy()
        r.ref_mscatter_f32_64x128(_p(m), _p(msrc), _p(midx), vr, vc)
        assert np.array_equal(m.view(np.uint32), mgot.view(np.uint32))
    if kind == "perm" and vr == 64:          # a gather with the same indices undoes the scatter
        assert np.array_equal(np.take_along_axis(got[:, :vc], idx[:, :vc].astype(np.int64), axis=0), src[:, :vc])
    assert np.array_equal(mgot[midx[:vr, :vc]], msrc[:vr, :vc])
    touched = np.zeros(8192, dtype=bool)
    touched[midx[:vr, :vc].ravel()] = True
    assert np.all(mgot[~touched] == mem0[~touched])


@pytest.mark.parametrize("n", range(len(sc.CI_CASES)))
def test_tci_vs_reference(oracle, n):
    start, desc, vc = sc.CI_CASES[n]
    got = oracle.tci(np.full(1024, -5, dtype=np.int32), start, desc, vc)
    assert np.array_equal(got, GOLD["tci_%d" % n])
    want = (np.int64(start) + (-1 if desc else 1) * np.arange(vc, dtype=np.int64)).astype(np.int32)    # closed form, wraps
    assert np.array_equal(got[:vc], want) and np.all(got[vc:] == -5)


@pytest.mark.parametrize("n", range(len(sc.GATHERB_CASES)))
def test_tgatherb_vs_reference(oracle, n):
    vr, vc, kind = sc.GATHERB_CASES[n]
    src, off, out0 = sc.gatherb_inputs(kind, n)
    got = oracle.tgatherb(out0, src, off, vr, vc)
    assert np.array_equal(got.view(np.uint32), GOLD["gatherb_%d" % n].view(np.uint32))
    r = oracle.ref()
    if r is not None:
        o = out0.copy()
        r.ref_tgatherb_f32_16x128(_p(o), _p(src), _p(off), vr, vc)
        assert np.array_equal(o.view(np.uint32), got.view(np.uint32))
    if kind == "aligned":        # aligned block starts: a plain gather of 8-element blocks
        blocks = src.reshape(-1, 8)
        assert np.array_equal(got[:vr, :vc].reshape(vr, vc // 8, 8), blocks[(off[:vr, :vc // 8] // 32).astype(np.int64)])
    assert np.array_equal(got[vr:], out0[vr:]) and np.array_equal(got[:, vc:], out0[:, vc:])
