"""Cases of pto_st_matmul_ragged (pto-isa_amd/csrc/pto_optest_matmul.hip): case id -> (operand type, m, k, n, form).
0-5 are the cases of the reference's CPU tests (tests/cpu/st/testcase/tmatmul/tmatmul_kernel.cpp:158-197), 6 and 8-11 those
of its NPU tests (tests/npu/a2a3/src/st/testcase/tmatmul/tmatmul_kernel.cpp:548-575); the rest exercise what the general path
adds: int8 with all extents ragged, bf16 with a bias, whole-block tiles with a valid region inside, mixed storage."""
import numpy as np

CASES = {
    0: ("f16", 40, 50, 60, "plain"),
    1: ("s8", 6, 7, 8, "plain"),
    2: ("f32", 120, 110, 50, "plain"),
    3: ("s8", 8, 7, 6, "bias"),
    4: ("f16", 16, 15, 16, "bias"),
    5: ("f32", 127, 128, 63, "bias"),
    6: ("f16", 31, 120, 58, "plain"),
    7: ("s8", 65, 90, 89, "plain"),
    8: ("f16", 5, 75, 11, "splitk"),
    9: ("f16", 1, 256, 64, "gemv"),
    10: ("f16", 1, 200, 32, "gemv"),
    11: ("f32", 5, 75, 11, "plain"),
    12: ("bf16", 33, 47, 19, "bias"),
    13: ("f16", 60, 50, 58, "plain"),
    14: ("f16", 100, 70, 120, "splitk"),
    15: ("f16", 64, 64, 16, "plain"),
    16: ("f16", 20, 64, 64, "bias"),
}


def bf16_round(x):
    """float32 -> the nearest bfloat16 (ties to even), returned as float32 and as the 16-bit pattern"""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return (r.astype(np.uint32) << 16).view(np.float32), r


def inputs(case_id, seed=0):
    """(a, b, bias or None) as the arrays handed to the kernel, and their values as float64 / int64 for the expectation"""
    kind, m, k, n, form = CASES[case_id]
    rng = np.random.default_rng(1000 * case_id + seed)
    if kind == "s8":
        a = rng.integers(-128, 127, size=(m, k), endpoint=True).astype(np.int8)
        b = rng.integers(-128, 127, size=(k, n), endpoint=True).astype(np.int8)
        bias = rng.integers(-1000, 1000, size=(1, n)).astype(np.int32) if form == "bias" else None
        return (a, b, bias), (a.astype(np.int64), b.astype(np.int64), None if bias is None else bias.astype(np.int64))
    a, b = rng.standard_normal((m, k)).astype(np.float32), rng.standard_normal((k, n)).astype(np.float32)
    bias = rng.standard_normal((1, n)).astype(np.float32) if form == "bias" else None
    bv = None if bias is None else bias.astype(np.float64)
    if kind == "f16":
        a, b = a.astype(np.float16), b.astype(np.float16)
        return (a, b, bias), (a.astype(np.float64), b.astype(np.float64), bv)
    if kind == "bf16":
        (av, ab), (bvv, bb) = bf16_round(a), bf16_round(b)
        return (ab, bb, bias), (av.astype(np.float64), bvv.astype(np.float64), bv)
    return (a, b, bias), (a.astype(np.float64), b.astype(np.float64), bv)


def expected(case_id, values):
    a, b, bias = values
    c = a @ b
    if bias is not None:
        c = 2 * (c + bias)       # the bias program stores the sum of its two results
    return c
