"""Host side of the run of the reference's per-instruction NPU test kernels (tests/st_ref_cases.py): every launcher
instantiation that the built libraries export parses into a launch plan whose buffers hold the valid region, and the
numpy formula of its test yields that region.  No GPU."""
import os
import re

import numpy as np
import pytest

import st_ref_cases as S

CASES = S.cases()


def test_case_table_covers_every_built_test():
    if not os.path.isdir(S.ST_DIR):
        pytest.skip("build/ported/st not built (reference tree absent at build time)")
    man = S.manifest()
    assert {S.lib_of(t) for t in S.SPECS} <= set(man)
    # every exported launcher of a listed test is a case: none is dropped by the symbol patterns
    for test, spec in S.SPECS.items():
        launchers = [d for d in man[S.lib_of(test)]["launchers"].values() if re.match(r"void %s%s<" % (re.escape(spec["fn"]), "2?" if "P<two>" in spec["tail"] else ("(?:Half)?" if "P<half>" in spec["tail"] else (r"\w*" if test == "tci" else ""))), d)]
        # cases whose L1 tiles exceed a compute unit's LDS: fp32 cases of 64 + 128 KiB; tiles of 176 to 400 KiB
        skipped = {"textract:launchTEXTRACT_COMPACT": 4, "tstore_mat2gm": 3}.get(test, 0)
        assert launchers and len(launchers) == sum(1 for c in CASES if c[0] == test) + skipped, test


@pytest.mark.parametrize("test,mangled,demangled", CASES, ids=[c[2][5:].split("(")[0] for c in CASES])
def test_plan_and_formula(test, mangled, demangled):
    pl = S.plan(test, demangled)
    assert len(pl.outs) == len(pl.regions)
    for (dt, (rows, ld)), (vr, vc) in zip(pl.outs, pl.regions):
        assert vr <= rows and vc <= ld
    ins = S.make_inputs(pl, seed=1)
    assert [a.shape for a in ins] == [tuple(e[1]) for e in pl.ins] and all(a.dtype == e[0] for a, e in zip(ins, pl.ins))
    with np.errstate(all="ignore"):
        wants = S.expected(pl, ins)
    assert len(wants) == len(pl.outs)
    for want, (vr, vc), (dt, _) in zip(wants, pl.regions, pl.outs):
        want = np.asarray(want)
        assert want.shape == (vr, vc) or (pl.flat_prefix is not None and want.ndim == 1 and want.size in (pl.flat_prefix, want.size if pl.flat_prefix < 0 else -1))
        if dt.kind == "f" and pl.compare is None:
            assert np.isfinite(want.astype(np.float64)).all()


def test_fix_pipe_model_known_answers():
    """The numpy model of the quantising conversions against values worked out by hand from the word layout of the
    reference's generator (tests/npu/a2a3/src/st/testcase/tmov_acc2mat/gen_data.py:27-100)."""
    f32 = lambda x: int(np.float32(x).view(np.uint32))
    acc = np.array([[100, -3, 10, -200, 5]], dtype=np.int32)
    signed = 1 << 46
    # scale 2, signed: 200 -> 127, -6, 20, -400 -> -256 -> -128, 10
    assert S.fix_quant_model(acc, np.uint64(f32(2.0) | signed), "int8_t").tolist() == [[127, -6, 20, -128, 10]]
    # unsigned: negatives clamp to 0, 200 stays
    assert S.fix_quant_model(acc, np.uint64(f32(2.0)), "uint8_t").tolist() == [[200, 0, 20, 0, 10]]
    # halves round to even: -1.5 -> -2, 2.5 -> 2; offset 3 is added after the rounding
    assert S.fix_quant_model(acc, np.uint64(f32(0.5) | signed | (3 << 37)), "int8_t").tolist() == [[53, 1, 8, -97, 5]]
    # one word per column
    words = np.array([f32(1.0) | signed, f32(2.0) | signed, f32(0.5) | signed, f32(1.0) | signed, f32(1.5) | signed], dtype=np.uint64)
    assert S.fix_quant_model(acc, words, "int8_t").tolist() == [[100, -6, 5, -128, 8]]
    # the scale keeps 10 mantissa bits: 1 + 2^-10 survives, 1 + 2^-11 is cut to 1
    big = np.array([[2048, 2048]], dtype=np.float32)
    got = S.fix_quant_model(big, np.array([f32(1 + 2.0**-10), f32(1 + 2.0**-11)], dtype=np.uint64), "half")
    assert got.tolist() == [[2050.0, 2048.0]]
    assert S.fix_quant_model(np.array([[1e6, -1e6]], dtype=np.float32), np.uint64(f32(1.0)), "half").tolist() == [[65504.0, -65504.0]]
    # int32 -> int16: shift by n + 1 (arithmetic), then clamp
    acc16 = np.array([[1000, -1000, 1 << 20, -(1 << 20)]], dtype=np.int32)
    assert S.fix_quant_model(acc16, np.uint64(1 << 32), "int16_t").tolist() == [[250, -250, 32767, -32768]]
    # the word the kernels build from their float argument
    assert S.fix_scalar_word(2.0, "int8_t") == np.uint64(0x40000000 | signed) and S.fix_scalar_word(2.0, "uint8_t") == np.uint64(0x40000000)
    assert S.fix_scalar_word(2.0, "int16_t") == np.uint64(1 << 32) and S.fix_scalar_word(2.0, "half") == np.uint64(0x40000000)
    # NZ image: [col blocks][row blocks][16][bc]
    mat = np.arange(32 * 32).reshape(32, 32)
    nz = S._nz(mat, 16)
    assert nz.shape == (64, 16) and nz[0].tolist() == list(range(16)) and nz[1].tolist() == list(range(32, 48)) and nz[32].tolist() == list(range(16, 32))
