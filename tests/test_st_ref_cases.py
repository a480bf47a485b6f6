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
        pytest.skip("oracle/_ref/st not built (reference tree absent at build time)")
    man = S.manifest()
    assert {S.lib_of(t) for t in S.SPECS} <= set(man)
    # every exported launcher of a listed test is a case: none is dropped by the symbol patterns
    for test, spec in S.SPECS.items():
        launchers = [d for d in man[S.lib_of(test)]["launchers"].values() if re.match(r"void %s%s<" % (re.escape(spec["fn"]), "2?" if "P<two>" in spec["tail"] else ("(?:Half)?" if "P<half>" in spec["tail"] else "")), d)]
        skipped = 4 if test == "textract:launchTEXTRACT_COMPACT" else 0     # fp32 cases of 64 + 128 KiB of L1 tiles
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
