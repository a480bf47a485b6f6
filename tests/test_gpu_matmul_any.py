"""TMOV / TEXTRACT / TMATMUL / TMATMUL_ACC / TMATMUL_BIAS / TGEMV / TSTORE on ragged tiles, on the GPU through the C ABI
(pto_st_matmul_ragged), for the shapes of the reference's own CPU and NPU tests of these instructions and for tiles of mixed
storage.  int8 exact; floating point against a float64 product with the tolerance of an fp32 accumulation over k (2e-3
relative to the row-by-column magnitude, as for the other matmul tests), and against the compiled reference where it is built."""
import ctypes as C

import numpy as np
import pytest

import matmul_any_cases as M
from pto_amd import capi

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case_id", sorted(M.CASES))
def test_matmul_ragged(case_id):
    import torch
    lib = capi.load_st()
    kind, m, k, n, form = M.CASES[case_id]
    (a, b, bias), values = M.inputs(case_id)
    dev = "cuda:0"
    view = {np.dtype(np.float16): np.int16, np.dtype(np.uint16): np.int16}

    def to_dev(x):
        return torch.from_numpy(x.view(view.get(x.dtype, x.dtype))).to(dev)
    out_dt = np.int32 if kind == "s8" else np.float32
    sentinel = 12345
    t_out = to_dev(np.full((m + 1, n), sentinel, dtype=out_dt))           # one row more than the kernel may touch
    ta, tb = to_dev(a), to_dev(b)
    tbias = to_dev(bias) if bias is not None else None
    print("case", case_id, M.CASES[case_id], flush=True)
    capi.check(lib.pto_st_matmul_ragged(None, t_out.data_ptr(), ta.data_ptr(), tb.data_ptr(),
                                        tbias.data_ptr() if tbias is not None else None, case_id), "matmul_ragged")
    torch.cuda.synchronize()
    got = t_out.cpu().numpy()
    want = M.expected(case_id, values)
    assert np.all(got[m] == sentinel)
    if kind == "s8":
        assert np.array_equal(got[:m].astype(np.int64), want)
    else:
        av, bv, _ = values
        scale = np.abs(av) @ np.abs(bv) * (2 if bias is not None else 1) + 1e-6
        assert np.max(np.abs(got[:m].astype(np.float64) - want) / scale) < 2e-3 * (1e-3 if kind == "f32" else 1)
        # the sequential fp32 accumulation of the general path, or an MFMA's: well inside 1e-5 of the magnitude


def test_unknown_case_is_refused():
    lib = capi.load_st()
    one = C.c_void_p(8)
    assert lib.pto_st_matmul_ragged(None, one, one, one, None, 999) == capi.ERR_UNSUPPORTED
    assert lib.pto_st_matmul_ragged(None, None, one, one, None, 0) == capi.ERR_BAD_ARG
