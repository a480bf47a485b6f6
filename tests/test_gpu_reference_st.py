"""The reference's own per-instruction NPU test kernels (tests/npu/a2a3/src/st/testcase/<op>/<op>_kernel.cpp), compiled
unchanged against include/pto (pto-isa_amd/build.py: build_ported_st, where the reference tree is mounted; the libraries
travel with the tree), run on the GPU: every launcher instantiation a kernel source exports is one case, checked against the
numpy formula of the test's own generator (tests/st_ref_cases.py).  Integer and bitwise results bit-exact, floating-point
results to the rounding of one operation (fp32 2e-6, fp16 1.5e-3 relative)."""
import ctypes as C
import os

import numpy as np
import pytest

import st_ref_cases as S

pytestmark = pytest.mark.gpu

CASES = S.cases()


def test_the_test_kernel_libraries_were_built():
    if not os.path.isdir(S.ST_DIR):
        # a run that is meant to cover the reference's test kernels (PTO_REQUIRE_PORTED=1) must not pass without them
        assert os.environ.get("PTO_REQUIRE_PORTED") != "1", "%s is missing and PTO_REQUIRE_PORTED=1" % S.ST_DIR
        pytest.skip("build/ported/st not built (reference tree absent at build time)")
    assert len(CASES) >= 1100 and {c[0] for c in CASES} == set(S.SPECS)


@pytest.mark.parametrize("test,mangled,demangled", CASES, ids=[c[2][5:].split("(")[0] for c in CASES])
def test_reference_st_kernel(test, mangled, demangled):
    import torch
    pl = S.plan(test, demangled)
    ins = S.make_inputs(pl, seed=len(demangled) + sum(map(ord, demangled)) % 997)
    lib = C.CDLL(os.path.join(S.ST_DIR, S.lib_of(test) + ".so"))
    fn = getattr(lib, mangled)
    dev = "cuda:0"
    view = {np.dtype(np.float16): np.int16, np.dtype(np.uint16): np.int16, np.dtype(np.uint32): np.int32, np.dtype(np.uint64): np.int64}

    def to_dev(a):
        return torch.from_numpy(a.view(view.get(a.dtype, a.dtype))).to(dev)

    def to_dev_padded(a):
        # 4096 zero elements follow every input: the reference's split-k matmul case reads its matrices in blocks of 32
        # columns with the row stride of the valid k (tmatmul_kernel.cpp:212-216, 254-255), which for k = 75 runs past the
        # end of both; zeros there make those reads defined and leave the product what the generator computes
        flat = a.reshape(-1)
        buf = np.zeros(flat.size + 4096, dtype=a.dtype)
        buf[:flat.size] = flat
        return to_dev(buf)
    sentinel = 77
    t_out = [to_dev(np.full(shape, sentinel, dtype=dt)) for dt, shape in pl.outs]
    t_in = [to_dev_padded(a) for a in ins]
    late = pl.ins_after_stream      # buffers that the launcher takes after its stream argument
    args = [C.c_void_p(t.data_ptr()) for t in t_out + t_in[:len(t_in) - late]]
    if pl.scalar and not pl.scalar_after_stream:
        args.append(pl.scalar[0](pl.scalar[1]))
    args.append(C.c_void_p(0))
    if pl.scalar and pl.scalar_after_stream:
        args.append(pl.scalar[0](pl.scalar[1]))
    args += [C.c_void_p(t.data_ptr()) for t in t_in[len(t_in) - late:]]
    fn.restype = None
    print("launch", demangled, flush=True)
    fn(*args)
    torch.cuda.synchronize()
    with np.errstate(all="ignore"):
        wants = S.expected(pl, ins)
    for t, (dt, shape), (vr, vc), want in zip(t_out, pl.outs, pl.regions, wants):
        got = t.cpu().numpy().view(dt)
        if pl.flat_prefix is not None:      # a packed run from the start of the buffer; the rest is not defined
            flat = np.asarray(want).reshape(-1)
            n = flat.size if pl.flat_prefix < 0 else pl.flat_prefix
            assert n == flat.size and n > 0
            if pl.compare is not None:
                assert pl.compare(got.reshape(-1)[:n], flat, ins), demangled
            else:
                assert np.array_equal(got.reshape(-1)[:n], flat.astype(dt)), demangled
            continue
        if pl.compare is not None:
            assert pl.compare(got[:vr, :vc], np.asarray(want), ins), demangled
        elif dt.kind == "f":
            want = np.asarray(want, dtype=np.float64).astype(dt)
            tol = pl.spec.get("tol", {}).get(dt.name, 2e-6 if dt == np.float32 else 1.5e-3)
            atol = pl.spec.get("atol", {}).get(dt.name, tol * 1e-2)
            assert np.allclose(got[:vr, :vc].astype(np.float64), want.astype(np.float64), rtol=tol, atol=atol), demangled
        else:
            assert np.array_equal(got[:vr, :vc], np.asarray(want).astype(dt)), demangled
        # nothing outside the valid region is stored
        rest = np.ones(shape, dtype=bool)
        rest[:vr, :vc] = False
        assert np.all(got[rest] == dt.type(sentinel)), demangled
