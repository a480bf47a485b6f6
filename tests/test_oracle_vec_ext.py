"""The oracle's further Vec instructions: against numpy closed forms, against the compiled reference
(oracle/_ref, where built) and against its committed outputs (tests/golden/ref_vec_ext.npz)."""
import ctypes as C
import os

import numpy as np
import pytest

from vec_ext_cases import ALL_OPS, REDUCE_SHAPES, numpy_vec_op, reduce_inputs, vec_inputs

GOLD = os.path.join(os.path.dirname(__file__), "golden", "ref_vec_ext.npz")


def p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


@pytest.mark.parametrize("op", ALL_OPS)
def test_vec_op_closed_form(oracle, op):
    a, b, vec, k = vec_inputs(op)
    got = oracle.vec_op(op, a, b, vec, k)
    want = numpy_vec_op(op, a, b, vec, k)
    assert np.array_equal(got, want, equal_nan=True), op          # bit-exact: the same IEEE operations


@pytest.mark.parametrize("op", ALL_OPS)
def test_vec_op_vs_reference(oracle, ref, op):
    a, b, vec, k = vec_inputs(op)
    out = np.zeros((64, 128), dtype=np.float32)
    ref.ref_vec_op_f32_64x128(p(out), p(a), p(b), p(vec), C.c_float(float(k)), oracle.VOP[op])
    assert np.array_equal(oracle.vec_op(op, a, b, vec, k), out, equal_nan=True), op


def test_vec_op_golden(oracle):
    g = np.load(GOLD)
    for op in ALL_OPS:
        a, b, vec, k = vec_inputs(op)
        assert np.array_equal(oracle.vec_op(op, a, b, vec, k)[::4], g["vec_" + op], equal_nan=True), op


@pytest.mark.parametrize("op", range(6))
@pytest.mark.parametrize("shape", REDUCE_SHAPES)
def test_reduce(oracle, op, shape):
    vr, vc = shape
    a = reduce_inputs()[:vr, :vc]
    got = oracle.reduce(op, a)
    axis = 1 if op < 3 else 0
    if op % 3 == 0:
        assert np.array_equal(got, a.max(axis=axis))
    elif op % 3 == 1:
        assert np.array_equal(got, a.min(axis=axis))
    else:                                                       # sequential fp32 sum along the reduced axis
        acc = np.zeros(a.shape[1 - axis], dtype=np.float32)
        for i in range(a.shape[axis]):
            acc = acc + (a[:, i] if axis == 1 else a[i, :])
        assert np.array_equal(got, acc)


@pytest.mark.parametrize("op", range(6))
@pytest.mark.parametrize("shape", REDUCE_SHAPES)
def test_reduce_vs_reference(oracle, ref, op, shape):
    vr, vc = shape
    full = reduce_inputs()
    out = np.zeros(128, dtype=np.float32)
    ref.ref_reduce_f32_64x128(p(out), p(full), vr, vc, op)
    n = vr if op < 3 else vc
    want = oracle.reduce(op, full[:vr, :vc])
    if op % 3 == 2:      # the reference's vectorised row / column loops may add in another order
        assert np.allclose(out[:n], want, rtol=1e-5, atol=1e-5)
    else:
        assert np.array_equal(out[:n], want)


@pytest.mark.parametrize("mode", range(6))
def test_cmps_sel(oracle, mode):
    a, b, _, _ = vec_inputs("CMP_EQ", seed=mode)
    scalar = np.float32(a[3, 5])
    a[::7, ::3] = scalar                                           # exact hits for EQ / NE / LE / GE
    a[1, 1] = scalar + np.float32(1e-6)                              # outside the 1e-9 tolerance
    bits = oracle.tcmps_packed(a, scalar, mode)
    cmpf = [lambda x: np.abs(x.astype(np.float64) - np.float64(scalar)) < 1e-9, lambda x: np.abs(x.astype(np.float64) - np.float64(scalar)) > 1e-9,
            lambda x: x < scalar, lambda x: x <= scalar, lambda x: x > scalar, lambda x: x >= scalar][mode]
    want_bits = np.packbits(cmpf(a), axis=1, bitorder="little")
    assert np.array_equal(bits, want_bits)
    mask = np.zeros((64, 32), dtype=np.uint8)
    mask[:, :16] = bits
    sel = oracle.tsel_packed(mask, 16, a, b)
    assert np.array_equal(sel, np.where(cmpf(a), a, b))


@pytest.mark.parametrize("mode", range(6))
def test_cmps_sel_vs_reference(oracle, ref, mode):
    a, b, _, _ = vec_inputs("CMP_EQ", seed=mode)
    scalar = np.float32(a[3, 5])
    a[::7, ::3] = scalar
    sel = np.zeros((64, 128), dtype=np.float32)
    bits = np.zeros((64, 16), dtype=np.uint8)
    ref.ref_cmps_sel_f32_64x128(p(sel), p(bits), p(a), p(b), C.c_float(float(scalar)), mode)
    obits = oracle.tcmps_packed(a, scalar, mode)
    assert np.array_equal(bits, obits)
    mask = np.zeros((64, 32), dtype=np.uint8)
    mask[:, :16] = obits
    assert np.array_equal(sel, oracle.tsel_packed(mask, 16, a, b))


def test_tsel_mask_rows_when_width_is_not_a_multiple_of_8(oracle):
    """Row i of the mask serves row i of the tiles; the unused high bits of its last byte are skipped
    (npu/a2a3/TSel.hpp:46-57, tsel/gen_data.py:31-47: the NPU test with 54 valid columns)."""
    rng = np.random.default_rng(5)
    a, b = rng.standard_normal((6, 12)).astype(np.float32), rng.standard_normal((6, 12)).astype(np.float32)
    bits = rng.integers(0, 2, size=(6, 12)).astype(bool)
    mask = np.full((6, 32), 0xFF, dtype=np.uint8)
    mask[:, :2] = np.packbits(bits, axis=1, bitorder="little")
    got = oracle.tsel_packed(mask, 2, a, b)
    assert np.array_equal(got, np.where(bits, a, b))


@pytest.mark.parametrize("pad_kind", [1, 2, 3])
@pytest.mark.parametrize("shape", [(64, 128), (10, 20), (64, 5), (1, 1)])
def test_fillpad(oracle, ref, pad_kind, shape):
    vr, vc = shape
    a = reduce_inputs(3)
    got = oracle.tfillpad(a, vr, vc, pad_kind)
    want = np.full((64, 128), [0.0, np.inf, -np.inf][pad_kind - 1], dtype=np.float32)
    want[:vr, :vc] = a[:vr, :vc]
    assert np.array_equal(got, want)
    out = np.zeros((64, 128), dtype=np.float32)
    ref.ref_fillpad_f32_64x128(p(out), p(a), vr, vc, pad_kind)
    assert np.array_equal(out, got)


@pytest.mark.parametrize("relu", [0, 1])
def test_tmov_relu(oracle, ref, relu):
    x = reduce_inputs(4)
    got = oracle.tmov_relu(x, relu)
    assert np.array_equal(got, np.maximum(x, 0) if relu else x)
    out = np.zeros((64, 128), dtype=np.float32)
    ref.ref_tmov_acc_vec_f32_64x128(p(out), p(x), relu)
    assert np.array_equal(out, got)
