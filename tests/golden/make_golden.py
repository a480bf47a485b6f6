"""Writes tests/golden/ref_vectors.npz, ref_vec_ext.npz, ref_mla.npz and ref_sort.npz: outputs of the COMPILED REFERENCE (oracle/_ref, built from the
reference's CPU-simulation headers) on seeded inputs.  Run in the build container, where the reference
tree is mounted; the fixture lets the oracle be checked against the reference where the tree is absent.

    python tests/golden/make_golden.py

Inputs are regenerated from seeds by the tests (pto_amd.datagen / numpy default_rng), only the
reference's outputs are stored.
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [ROOT, os.path.join(ROOT, "pto-isa_amd")]

from oracle import oracle  # noqa: E402
from pto_amd import datagen  # noqa: E402


def p(a):
    return a.ctypes.data_as(C.c_void_p)


def cases(ref):
    out = {}
    a, b = datagen.gemm_inputs(128, 128, 512)
    c = np.zeros((128, 128), dtype=np.float32)
    ref.ref_gemm_128x512x128_ks64(p(c), p(a), p(b))
    out["gemm_128x512x128_ks64"] = c
    a, b = datagen.gemm_inputs(128, 256, 64)
    c = np.zeros((128, 256), dtype=np.float32)
    ref.ref_gemm_128x64x256_ks64(p(c), p(a), p(b))
    out["gemm_128x64x256_ks64"] = c
    x = datagen.tcvt_input(64, 256, inject=0.05).reshape(-1)
    h = np.zeros(x.size, dtype=np.uint16)
    ref.ref_tcvt_f32_f16(p(h), p(x), C.c_size_t(x.size))
    out["tcvt_f32_f16_64x256"] = h
    rng = np.random.default_rng(9)
    src = rng.integers(0, 2**16, size=(16, 1024), dtype=np.uint16)
    idx = rng.integers(-50, 16 * 1024 + 50, size=(16, 128), dtype=np.int32)
    g = np.zeros((16, 128), dtype=np.uint16)
    ref.ref_tgather_index_f16_16x1024_16x128(p(g), p(src), p(idx))
    out["tgather_index_f16_16x1024_16x128"] = g
    rng = np.random.default_rng(20251220)
    q, k, v = (rng.standard_normal((64, 32), dtype=np.float32) for _ in range(3))
    o = np.zeros((64, 32), dtype=np.float32)
    ref.ref_fa_auto_64x32(p(o), p(q), p(k), p(v))
    out["fa_auto_64x32"] = o
    x = np.arange(128 * 256, dtype=np.uint16).reshape(128, 256)
    e = np.zeros((128, 64), dtype=np.uint16)
    ref.ref_textract_suffix_128x256_0_192(p(e), p(x))
    out["textract_suffix_128x256_0_192"] = e
    return out


def vec_ext_cases(ref):
    """Outputs of the compiled reference for the further Vec instructions -> ref_vec_ext.npz."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from vec_ext_cases import ALL_OPS, vec_inputs
    out = {}
    for op in ALL_OPS:
        a, b, vec, k = vec_inputs(op)
        o = np.zeros((64, 128), dtype=np.float32)
        ref.ref_vec_op_f32_64x128(p(o), p(a), p(b), None if vec is None else p(vec), C.c_float(float(k)), oracle.VOP[op])
        out["vec_" + op] = o[::4].copy()  # every fourth row keeps the fixture small
    return out


MLA_CASES = {"demo_scale": (0.02, 0.02), "peaked": (1.0, 0.5)}


def mla_cases(ref):
    """The reference's CPU simulation running the multi-latent attention program on two heads -> ref_mla.npz."""
    out = {}
    for name, (xs, ws) in MLA_CASES.items():
        q, k, v, wq, wk, wv, wo = datagen.mla_inputs(1, 2, xs, ws)
        o = np.zeros_like(q)
        for h in range(2):
            oh = np.zeros((64, 32), dtype=np.float32)
            ref.ref_mla_auto_64x32x16(p(oh), p(np.ascontiguousarray(q[0, h])), p(np.ascontiguousarray(k[0, h])),
                                      p(np.ascontiguousarray(v[0, h])), p(wq), p(wk), p(wv), p(wo))
            o[0, h] = oh
        out["mla_" + name] = o
    return out


def sort_cases(ref):
    """TSORT32 / TMRGSORT outputs of the reference's CPU simulation for the seeded cases of tests/sort_cases.py -> ref_sort.npz."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import sort_cases as sc
    out = {}
    for dtype, vr, vc, seed in sc.SORT32_CASES:
        src, idx, o = sc.sort32_inputs(dtype, vr, vc, seed)
        (ref.ref_tsort32_f32_8x128 if dtype == "f32" else ref.ref_tsort32_s32_8x128)(p(o), p(src), p(idx), vr, vc)
        out["sort32_%d" % seed] = o
    for valid_cols, block_len, seed in sc.BLOCK_CASES:
        src, o = sc.block_inputs(valid_cols, block_len, seed)
        ref.ref_tmrgsort_blocks_f32_1x1024(p(o), p(src), valid_cols, block_len)
        out["blocks_%d" % seed] = o.view(np.uint32)
    for counts, out_structs, exhausted, seed in sc.LIST_CASES:
        lists, o = sc.list_inputs(counts, seed)
        ex = np.zeros(4, dtype=np.uint32)
        ptrs = [p(l) for l in lists] + [None] * (4 - len(lists))
        cols = [2 * n for n in counts] + [0] * (4 - len(counts))
        ref.ref_tmrgsort_lists_f32(p(o), p(ex), *ptrs, *cols, 2 * out_structs, len(counts), exhausted)
        out["lists_%d" % seed] = o.view(np.uint32)
        out["lists_%d_executed" % seed] = ex
    for dtype, vr, vc, seed in sc.SORT32_CASES_16:
        src, idx, o = sc.sort32_inputs_16(dtype, vr, vc, seed)
        (ref.ref_tsort32_f16_8x128 if dtype == "f16" else ref.ref_tsort32_s16_8x128)(p(o), p(src), p(idx), vr, vc)
        out["sort32_%d" % seed] = o.view(np.uint16)
    for dtype, valid_cols, block_len, seed in sc.BLOCK_CASES_16:
        src, o = sc.block_inputs_16(dtype, valid_cols, block_len, seed)
        ref.ref_tmrgsort_blocks_16_1x2048(p(o), p(src), valid_cols, block_len, sc.DT16[dtype])
        out["blocks_%d" % seed] = o.view(np.uint16)
    for dtype, counts, out_structs, exhausted, seed in sc.LIST_CASES_16:
        lists, o = sc.list_inputs_16(dtype, counts, seed)
        ex = np.zeros(4, dtype=np.uint32)
        ptrs = [p(l) for l in lists] + [None] * (4 - len(lists))
        cols = [4 * n for n in counts] + [0] * (4 - len(counts))
        ref.ref_tmrgsort_lists_16(p(o), p(ex), *ptrs, *cols, 4 * out_structs, len(counts), exhausted, sc.DT16[dtype])
        out["lists_%d" % seed] = o.view(np.uint16)
        out["lists_%d_executed" % seed] = ex
    for n, (op, dv, av, bv) in enumerate(sc.PART_CASES):
        a, b, o = sc.part_inputs(n)
        ref.ref_tpart_f32_64x128(p(o), p(a), p(b), op, *dv, *av, *bv)
        out["part_%d" % n] = o[::3].copy()      # every third row keeps the fixture small
    for n, (vr, vc, kind) in enumerate(sc.SCATTER_CASES):
        src, idx, o = sc.scatter_inputs(vr, vc, kind, n)
        ref.ref_tscatter_f32_64x128(p(o), p(src), p(idx), vr, vc)
        out["tscatter_%d" % n] = o[::3].copy()
        src, idx, mem = sc.mscatter_inputs(vr, vc, n)
        ref.ref_mscatter_f32_64x128(p(mem), p(src), p(idx), vr, vc)
        out["mscatter_%d" % n] = mem[::3].copy()
    for n, (vr, vc, kind) in enumerate(sc.GATHERB_CASES):
        src, off, o = sc.gatherb_inputs(kind, n)
        ref.ref_tgatherb_f32_16x128(p(o), p(src), p(off), vr, vc)
        out["gatherb_%d" % n] = o
    for n, (start, desc, vc) in enumerate(sc.CI_CASES):
        o = np.full(1024, -5, dtype=np.int32)
        ref.ref_tci_s32_1x1024(p(o), start, desc, vc)
        out["tci_%d" % n] = o
    return out


if __name__ == "__main__":
    oracle.build(ref=True)
    r = oracle.ref()
    if r is None:
        sys.exit("reference tree not present: cannot regenerate the fixture")
    np.savez_compressed(os.path.join(HERE, "ref_vectors.npz"), **cases(r))
    print("wrote", os.path.join(HERE, "ref_vectors.npz"))
    np.savez_compressed(os.path.join(HERE, "ref_vec_ext.npz"), **vec_ext_cases(r))
    print("wrote", os.path.join(HERE, "ref_vec_ext.npz"))
    np.savez_compressed(os.path.join(HERE, "ref_mla.npz"), **mla_cases(r))
    print("wrote", os.path.join(HERE, "ref_mla.npz"))
    np.savez_compressed(os.path.join(HERE, "ref_sort.npz"), **sort_cases(r))
    print("wrote", os.path.join(HERE, "ref_sort.npz"))
