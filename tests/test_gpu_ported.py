"""The reference's own kernel sources, compiled against include/pto (pto-isa_amd/build.py: build_ported, only where the
reference tree is mounted; the libraries travel with the tree), run on the GPU and are held to the same bar as the
native kernels."""
import ctypes as C
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PORTED = os.path.join(ROOT, "oracle", "_ref")

pytestmark = pytest.mark.gpu


def _ported(name):
    path = os.path.join(PORTED, name)
    if not os.path.exists(path):
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
