"""GPU parity of the further Vec instructions (unary math, ReLU family, compare / select, row and column
broadcasts and reductions, TFILLPAD, TMOV accumulator -> Vec) through the C ABI, against the oracle."""
import numpy as np
import pytest
import torch

from pto_amd import capi
from vec_ext_cases import ALL_OPS, REDUCE_SHAPES, reduce_inputs, vec_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# device results that may differ from the host's in the last place: library log / exp in double then cast
ULP_OPS = {"LOG": 1, "EXP": 1, "ROWEXPANDEXPDIF": 1, "COLEXPANDEXPDIF": 1}


def dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype in (np.uint16, np.float16):
        return torch.from_numpy(a.view(np.int16)).to(DEV)
    return torch.from_numpy(a).to(DEV)


def st():
    return torch.cuda.current_stream().cuda_stream


def ulp_diff(a, b):
    ia, ib = a.view(np.int32).astype(np.int64), b.view(np.int32).astype(np.int64)
    return np.abs(ia - ib)


@pytest.mark.parametrize("op", ALL_OPS)
def test_vec_op(oracle, op):
    lib = capi.load_st()
    a, b, vec, k = vec_inputs(op)
    ta, tb = dev(a), dev(b)
    tv = dev(vec) if vec is not None else None
    out = torch.full((64, 128), float("nan"), device=DEV)
    capi.check(lib.pto_st_vec_op_f32_64x128(st(), out.data_ptr(), ta.data_ptr(), tb.data_ptr(), tv.data_ptr() if tv is not None else 0,
                                            float(k), oracle.VOP[op]), op)
    torch.cuda.synchronize()
    got, want = out.cpu().numpy(), oracle.vec_op(op, a, b, vec, k)
    if op in ULP_OPS:
        assert ulp_diff(got, want).max() <= ULP_OPS[op], op
        assert (ulp_diff(got, want) > 0).mean() < 0.01, op       # and almost all results are identical
    else:
        assert np.array_equal(got, want, equal_nan=True), op      # bit-exact


def test_vec_op_bad_code():
    lib = capi.load_st()
    out = torch.zeros((64, 128), device=DEV)
    assert lib.pto_st_vec_op_f32_64x128(st(), out.data_ptr(), out.data_ptr(), out.data_ptr(), 0, 0.0, 999) == capi.ERR_BAD_ARG


@pytest.mark.parametrize("op", range(6))
@pytest.mark.parametrize("shape", REDUCE_SHAPES)
def test_reduce(oracle, op, shape):
    lib = capi.load_st()
    vr, vc = shape
    full = reduce_inputs()
    ta = dev(full)
    out = torch.full((128,), -777.0, device=DEV)
    capi.check(lib.pto_st_reduce_f32_64x128(st(), out.data_ptr(), ta.data_ptr(), vr, vc, op), "reduce")
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    n = vr if op < 3 else vc
    want = oracle.reduce(op, full[:vr, :vc])
    if op % 3 == 2:       # sums add in another order than the sequential oracle: fp32 rounding only
        mag = np.abs(full[:vr, :vc]).sum(axis=1 if op < 3 else 0)
        assert np.all(np.abs(got[:n] - want) <= 2.0 ** -20 * mag)
    else:
        assert np.array_equal(got[:n], want)
    assert np.all(got[n:] == -777.0)                               # nothing outside the valid region is written


@pytest.mark.parametrize("mode", range(6))
def test_cmps_sel(oracle, mode):
    lib = capi.load_st()
    a, b, _, _ = vec_inputs("CMP_EQ", seed=mode)
    scalar = np.float32(a[3, 5])
    a[::7, ::3] = scalar
    a[1, 1] = scalar + np.float32(1e-6)
    ta, tb = dev(a), dev(b)
    sel = torch.zeros((64, 128), device=DEV)
    bits = torch.zeros((64, 16), dtype=torch.uint8, device=DEV)
    capi.check(lib.pto_st_cmps_sel_f32_64x128(st(), sel.data_ptr(), bits.data_ptr(), ta.data_ptr(), tb.data_ptr(), float(scalar), mode), "cmps")
    torch.cuda.synchronize()
    obits = oracle.tcmps_packed(a, scalar, mode)
    assert np.array_equal(bits.cpu().numpy(), obits)
    mask = np.zeros((64, 32), dtype=np.uint8)
    mask[:, :16] = obits
    assert np.array_equal(sel.cpu().numpy(), oracle.tsel_packed(mask, 16, a, b))


@pytest.mark.parametrize("pad_kind", [1, 2, 3])
@pytest.mark.parametrize("shape", [(64, 128), (10, 20), (64, 5), (1, 1)])
def test_fillpad(oracle, pad_kind, shape):
    lib = capi.load_st()
    vr, vc = shape
    a = reduce_inputs(3)
    ta = dev(a)
    out = torch.full((64, 128), 5.0, device=DEV)
    capi.check(lib.pto_st_fillpad_f32_64x128(st(), out.data_ptr(), ta.data_ptr(), vr, vc, pad_kind), "fillpad")
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), oracle.tfillpad(a, vr, vc, pad_kind))


@pytest.mark.parametrize("relu", [0, 1])
def test_matmul_tmov_acc_to_vec(oracle, relu):
    lib = capi.load_st()
    rng = np.random.default_rng(21)
    a = rng.integers(-4, 5, size=(64, 64)).astype(np.float32)     # integer values: the fp32 products and sums are exact
    b = rng.integers(-4, 5, size=(64, 128)).astype(np.float32)
    ta, tb = dev(a.astype(np.float16)), dev(np.ascontiguousarray(b.T).astype(np.float16))
    out = torch.zeros((64, 128), device=DEV)
    capi.check(lib.pto_st_matmul_tmov_f16_64x64x128(st(), out.data_ptr(), ta.data_ptr(), tb.data_ptr(), relu, 0.5), "tmov")
    torch.cuda.synchronize()
    want = oracle.tmov_relu((a @ b).astype(np.float32), relu) * np.float32(0.5)
    assert np.array_equal(out.cpu().numpy(), want)


TYPED_OPS = {
    "ABS": lambda a, b, v, k: np.abs(a), "NEG": lambda a, b, v, k: -a, "RELU": lambda a, b, v, k: np.maximum(a, 0),
    "ADD": lambda a, b, v, k: a + b, "SUB": lambda a, b, v, k: a - b, "MUL": lambda a, b, v, k: a * b,
    "MAX": lambda a, b, v, k: np.maximum(a, b), "MIN": lambda a, b, v, k: np.minimum(a, b),
    "ADDS": lambda a, b, v, k: a + k, "SUBS": lambda a, b, v, k: a - k, "MULS": lambda a, b, v, k: a * k,
    "MAXS": lambda a, b, v, k: np.maximum(a, k), "MINS": lambda a, b, v, k: np.minimum(a, k),
    "ROWEXPAND": lambda a, b, v, k: np.broadcast_to(v[:, None], a.shape), "ROWEXPANDSUB": lambda a, b, v, k: a - v[:, None],
    "ROWEXPANDMUL": lambda a, b, v, k: a * v[:, None], "ROWEXPANDADD": lambda a, b, v, k: a + v[:, None],
    "ROWEXPANDMAX": lambda a, b, v, k: np.maximum(a, v[:, None]), "ROWEXPANDMIN": lambda a, b, v, k: np.minimum(a, v[:, None]),
    "COLEXPAND": lambda a, b, v, k: np.broadcast_to(v[None, :], a.shape), "COLEXPANDSUB": lambda a, b, v, k: a - v[None, :],
    "COLEXPANDMUL": lambda a, b, v, k: a * v[None, :], "COLEXPANDADD": lambda a, b, v, k: a + v[None, :],
    "COLEXPANDMAX": lambda a, b, v, k: np.maximum(a, v[None, :]), "COLEXPANDMIN": lambda a, b, v, k: np.minimum(a, v[None, :]),
}


FP16_MATH_OPS = {
    # the CPU simulation evaluates these in double and casts to the element type (ElementOp.h:265-340, TSqrt.hpp:23,
    # TRSqrt.hpp:29-31, TExp.hpp:36); division and reciprocal are one operation in the element type (numpy's float16
    # divides in float32 and rounds once more, which is what a host compiler does with _Float16 as well)
    "SQRT": lambda a, b, k: np.sqrt(np.abs(a).astype(np.float64)).astype(np.float16),
    "RSQRT": lambda a, b, k: (1.0 / np.sqrt(np.abs(a).astype(np.float64))).astype(np.float16),
    "LOG": lambda a, b, k: np.log(np.abs(a).astype(np.float64)).astype(np.float16),
    "EXP": lambda a, b, k: np.exp(a.astype(np.float64)).astype(np.float16),
    "RECIP": lambda a, b, k: (np.float16(1) / a).astype(np.float16),
    "DIV": lambda a, b, k: (a / b).astype(np.float16),
    "DIVS": lambda a, b, k: (a / k).astype(np.float16),
}


@pytest.mark.parametrize("op", sorted(FP16_MATH_OPS))
def test_vec_math_ops_fp16(oracle, op):
    """TSQRT, TRSQRT, TLOG, TEXP, TRECIP, TDIV, TDIVS on fp16 tiles, bit-exact against the rule of the CPU simulation
    (double evaluation + one cast for the transcendental ones), subnormal results and overflow to infinity included."""
    lib = capi.load_st()
    rng = np.random.default_rng(500 + len(op))
    a = (rng.standard_normal((64, 128)) * (3 if op == "EXP" else 40)).astype(np.float16)
    a[0, :8] = np.array([0.0, 6.1e-5, 5.96e-8, 65504.0, 1.0, 0.5, 11.1, 3.0e-5], dtype=np.float16)
    if op == "EXP":
        a[1, :4] = np.array([11.0, 11.1, -17.0, -16.0], dtype=np.float16)   # overflow to inf, subnormal results
    b = (rng.standard_normal((64, 128)) * 8).astype(np.float16)
    b[b == 0] = np.float16(1)
    k = np.float16(1.75)
    src = np.abs(a) if op in ("SQRT", "RSQRT", "LOG") else a
    with np.errstate(over="ignore", invalid="ignore", divide="ignore"):
        want = FP16_MATH_OPS[op](src, b, k)
    ta, tb = dev(src), dev(b)
    out = torch.zeros((64, 128), dtype=torch.int16, device=DEV)
    capi.check(lib.pto_st_vec_op_typed_64x128(st(), out.data_ptr(), ta.data_ptr(), tb.data_ptr(), 0, float(k), oracle.VOP[op], 0), op)
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(np.float16)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint16), want[~nan].view(np.uint16)), op


@pytest.mark.parametrize("dtype", ["f16", "s32"])
@pytest.mark.parametrize("op", sorted(TYPED_OPS))
def test_vec_op_fp16_and_int32(oracle, op, dtype):
    """The arithmetic Vec instructions on fp16 tiles (one IEEE rounding per operation, as numpy's float16) and on int32
    tiles (wrap-around arithmetic): bit-exact."""
    lib = capi.load_st()
    rng = np.random.default_rng(101 + len(op))
    if dtype == "f16":
        a = (rng.standard_normal((64, 128)) * 8).astype(np.float16)
        b = (rng.standard_normal((64, 128)) * 8).astype(np.float16)
        k = np.float16(1.75)
        mk = lambda n: (rng.standard_normal(n) * 4).astype(np.float16)
    else:
        a = rng.integers(-2**31, 2**31, size=(64, 128), dtype=np.int64).astype(np.int32)
        b = rng.integers(-2**31, 2**31, size=(64, 128), dtype=np.int64).astype(np.int32)
        a[0, 0] = -2**31                                        # abs / neg of the most negative value wrap
        k = np.int32(37)
        mk = lambda n: rng.integers(-2**20, 2**20, size=n).astype(np.int32)
    vec = mk(64) if op.startswith("ROW") else (mk(128) if op.startswith("COL") else None)
    with np.errstate(over="ignore", invalid="ignore"):
        want = np.ascontiguousarray(TYPED_OPS[op](a, b, vec, k)).astype(a.dtype)
    ta, tb = dev(a), dev(b)
    tv = dev(vec) if vec is not None else None
    out = torch.zeros((64, 128), dtype=torch.int16 if dtype == "f16" else torch.int32, device=DEV)
    capi.check(lib.pto_st_vec_op_typed_64x128(st(), out.data_ptr(), ta.data_ptr(), tb.data_ptr(), tv.data_ptr() if tv is not None else 0,
                                              float(k), oracle.VOP[op], 0 if dtype == "f16" else 1), op)
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(a.dtype)
    if dtype == "f16":
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan)
        assert np.array_equal(got[~nan].view(np.uint16), want[~nan].view(np.uint16)), op
    else:
        assert np.array_equal(got, want), op


BIT_OPS = ["AND", "OR", "XOR", "SHL", "SHR", "REM", "NOT", "ANDS", "ORS", "XORS", "SHLS", "SHRS", "REMS", "ADDC", "SUBC", "ADDSC", "SUBSC"]
FLOAT_BIT_OPS = ["REM", "REMS", "ADDC", "SUBC", "ADDSC", "SUBSC"]


def c_rem(a, b):
    """C's remainder (sign of the dividend), the rule of the reference's element operation, for integers and floats."""
    if a.dtype.kind == "i":
        a64, b64 = a.astype(np.int64), np.broadcast_to(b, a.shape).astype(np.int64)
        return (a64 - np.trunc(a64 / b64).astype(np.int64) * b64).astype(a.dtype)
    return np.fmod(a.astype(np.float64), np.float64(b) if np.ndim(b) == 0 else b.astype(np.float64)).astype(a.dtype)


@pytest.mark.parametrize("op,dtype", [(op, "s32") for op in BIT_OPS] + [(op, "f32") for op in FLOAT_BIT_OPS])
def test_vec_bitwise_shift_rem_carry(op, dtype):
    """TAND .. TSUBSC against numpy's integer / float rules (wrap-around int32; shifts by 0..31, arithmetic right
    shift; remainder with the dividend's sign; a + b + c evaluated left to right in the element type): bit-exact."""
    lib = capi.load_st()
    rng = np.random.default_rng(300 + BIT_OPS.index(op))
    if dtype == "s32":
        a = rng.integers(-2**31, 2**31, size=(64, 128), dtype=np.int64).astype(np.int32)
        b = rng.integers(-2**31, 2**31, size=(64, 128), dtype=np.int64).astype(np.int32)
        c = rng.integers(-2**31, 2**31, size=(64, 128), dtype=np.int64).astype(np.int32)
        k = np.int32(-1234577 if op in ("ANDS", "ORS", "XORS", "ADDSC", "SUBSC") else 11)
        if op in ("SHL", "SHR"):
            b = rng.integers(0, 32, size=(64, 128)).astype(np.int32)
        if op == "REM":
            b = rng.integers(1, 2**20, size=(64, 128)).astype(np.int32) * rng.choice(np.array([-1, 1], dtype=np.int32), size=(64, 128))
            a[0, :4] = [-2**31, 2**31 - 1, 0, -1]
        if op == "SHL":                                         # a left shift of a negative value: the bits move, as on the device
            want = ((a.astype(np.int64) << b) & 0xffffffff).astype(np.uint32).view(np.int32)
        elif op == "SHLS":
            want = ((a.astype(np.int64) << int(k)) & 0xffffffff).astype(np.uint32).view(np.int32)
    else:
        a = (rng.standard_normal((64, 128)) * 100).astype(np.float32)
        b = (rng.standard_normal((64, 128)) * 7).astype(np.float32)
        b[b == 0] = 1
        c = (rng.standard_normal((64, 128)) * 50).astype(np.float32)
        k = np.float32(3.7)
    with np.errstate(over="ignore"):
        table = {"AND": lambda: a & b, "OR": lambda: a | b, "XOR": lambda: a ^ b, "SHR": lambda: a >> b, "REM": lambda: c_rem(a, b),
                 "NOT": lambda: ~a, "ANDS": lambda: a & k, "ORS": lambda: a | k, "XORS": lambda: a ^ k, "SHRS": lambda: a >> k,
                 "REMS": lambda: c_rem(a, k), "ADDC": lambda: a + b + c, "SUBC": lambda: a - b + c, "ADDSC": lambda: a + k + c,
                 "SUBSC": lambda: a - k + c}
        if op not in ("SHL", "SHLS"):
            want = table[op]().astype(a.dtype)
    ta, tb, tc = dev(a), dev(b), dev(c)
    out = torch.zeros((64, 128), dtype=torch.int32, device=DEV)
    capi.check(lib.pto_st_vec_bitop_64x128(st(), out.data_ptr(), ta.data_ptr(), tb.data_ptr(), tc.data_ptr(), float(k), int(k) if dtype == "s32" else 0,
                                           BIT_OPS.index(op), 1 if dtype == "s32" else 0), op)
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(a.dtype)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), op


def test_vec_bitop_rejects_bad_arguments():
    lib = capi.load_st()
    t = torch.zeros((64, 128), dtype=torch.int32, device=DEV)
    p = t.data_ptr()
    assert lib.pto_st_vec_bitop_64x128(st(), p, p, p, p, 0.0, 0, 17, 1) == capi.ERR_BAD_ARG
    assert lib.pto_st_vec_bitop_64x128(st(), p, p, p, p, 0.0, 0, 0, 0) == capi.ERR_UNSUPPORTED   # TAND on fp32
    assert lib.pto_st_vec_bitop_64x128(st(), p, p, 0, p, 0.0, 0, 0, 1) == capi.ERR_BAD_ARG


def test_ttrans_and_tmov_to_operands():
    """TTRANS is a permutation (bit-exact); TMOV Vec -> Left / Right and Acc -> Left feed matmuls whose small-integer
    inputs make every product and sum exact in fp16 / fp32."""
    lib = capi.load_st()
    rng = np.random.default_rng(55)
    x = rng.standard_normal((64, 128)).astype(np.float32)
    x[0, :3] = [np.nan, np.inf, -0.0]
    tx = dev(x)
    ty = torch.zeros((128, 64), device=DEV)
    capi.check(lib.pto_st_ttrans_f32_64x128(st(), ty.data_ptr(), tx.data_ptr()), "ttrans")
    torch.cuda.synchronize()
    assert np.array_equal(ty.cpu().numpy().view(np.uint32), np.ascontiguousarray(x.T).view(np.uint32))
    a = rng.integers(-2, 3, size=(64, 64)).astype(np.float32)
    b = rng.integers(-2, 3, size=(64, 128)).astype(np.float32)
    ta, tb = dev(a.astype(np.float16)), dev(b.astype(np.float16))
    mid = torch.zeros((64, 128), device=DEV)
    out = torch.zeros((64, 64), device=DEV)
    capi.check(lib.pto_st_matmul_vec_operands_f16_64x64x128(st(), out.data_ptr(), mid.data_ptr(), ta.data_ptr(), tb.data_ptr()), "vec operands")
    torch.cuda.synchronize()
    want_mid = a @ b                                            # |values| <= 256: exact in fp16 as well
    assert np.array_equal(mid.cpu().numpy(), want_mid)
    assert np.array_equal(out.cpu().numpy(), want_mid @ b.T)
