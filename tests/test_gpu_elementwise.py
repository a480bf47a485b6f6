"""GPU parity of TCVT and the gathers through the C ABI: bit-exact against the oracle."""
import os

import numpy as np
import pytest
import torch

from pto_amd import capi, datagen

pytestmark = pytest.mark.gpu


def boundary_patterns():
    exps = np.arange(0, 256, dtype=np.uint32) << 23
    mants = np.array([0, 1, 0xfff, 0x1000, 0x1001, 0x1fff, 0x2000, 0x2001, 0x2fff, 0x3000, 0x3001, 0x7fe000, 0x7fefff,
                      0x7ff000, 0x7ff001, 0x7fffff, 0x400000, 0x3fffff, 0x400001, 0x200000, 0x600000, 0x100000,
                      0x080000, 0x7fc000, 0x7f8000, 0x7fff, 0x8000, 0x8001, 0x17fff, 0x18000, 0x18001], dtype=np.uint32)
    pos = (exps[:, None] | mants[None, :]).reshape(-1)
    return np.concatenate([pos, pos | np.uint32(0x80000000)])


def test_tcvt_f16_boundaries_and_strided_sweep(oracle):
    """Every exponent x mantissa pattern around the fp16 rounding boundaries (NaN payloads, +-inf,
    overflow at 65520, subnormal results, ties) and a 2^32 / 1021 strided sweep."""
    from gpu_util import tcvt
    bits = np.concatenate([boundary_patterns(), np.arange(0, 2**32, 1021, dtype=np.uint64).astype(np.uint32)])
    x = bits.view(np.float32)
    assert np.array_equal(tcvt(x, "f16"), oracle.tcvt_f32_f16(x))


def test_tcvt_bf16_boundaries_and_strided_sweep(oracle):
    from gpu_util import tcvt
    bits = np.concatenate([boundary_patterns(), np.arange(0, 2**32, 1021, dtype=np.uint64).astype(np.uint32)])
    x = bits.view(np.float32)
    got = tcvt(x, "bf16")
    assert np.array_equal(got, oracle.tcvt_f32_bf16(x))
    nan = np.isnan(x)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got[~nan], want[~nan])


@pytest.mark.parametrize("n", [0, 1, 7, 8, 8191, 8192, 8193, 3 * 8192 + 5])
def test_tcvt_ragged_sizes(oracle, n):
    from gpu_util import tcvt
    x = datagen.tcvt_input(1, max(n, 8), inject=0.05).reshape(-1)[:n]
    assert np.array_equal(tcvt(x, "f16"), oracle.tcvt_f32_f16(x))
    assert np.array_equal(tcvt(x, "bf16"), oracle.tcvt_f32_bf16(x))


def test_tcvt_golden_fixture():
    from gpu_util import tcvt
    G = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_vectors.npz"))
    x = datagen.tcvt_input(64, 256, inject=0.05).reshape(-1)
    assert np.array_equal(tcvt(x, "f16"), G["tcvt_f32_f16_64x256"])


def test_tcvt_round_modes(oracle):
    """CAST_ROUND (ties away) against the oracle's ties-away conversion; directed modes against
    numpy's nextafter-based definition on finite inputs."""
    from gpu_util import tcvt
    bits = np.concatenate([boundary_patterns(), np.arange(0, 2**32, 65521, dtype=np.uint64).astype(np.uint32)])
    x = bits.view(np.float32)
    got = tcvt(x, "f16", capi.CAST_ROUND)
    want = np.array([oracle.lib().po_f32_to_f16_rna(int(b)) for b in bits[:20000]], dtype=np.uint16)
    assert np.array_equal(got[:20000], want)
    fin = np.isfinite(x) & (np.abs(x) < 65504)
    xf = x[fin].astype(np.float64)
    for mode, pred in ((capi.CAST_FLOOR, lambda h: h <= xf), (capi.CAST_CEIL, lambda h: h >= xf),
                       (capi.CAST_TRUNC, lambda h: np.abs(h) <= np.abs(xf))):
        h = tcvt(x, "f16", mode)[fin].view(np.float16).astype(np.float64)
        assert np.all(pred(h))
        assert np.all(np.abs(h - xf) <= np.maximum(np.abs(xf) * 2.0**-10, 2.0**-24))   # within one fp16 ulp


def test_tcvt_full_size_config(oracle):
    """Config 5 at full size 16384 x 8192 with 0.1% special values: compared in slabs against the oracle."""
    from gpu_util import to_dev, stream
    lib = capi.load()
    x = datagen.tcvt_input(16384, 8192)
    tx = to_dev(x.reshape(-1))
    for kind, fn, ofn in (("f16", lib.pto_tcvt_f32_f16, oracle.tcvt_f32_f16), ("bf16", lib.pto_tcvt_f32_bf16, oracle.tcvt_f32_bf16)):
        th = torch.zeros(x.size, dtype=torch.int16, device="cuda:0")
        capi.check(fn(stream(), th.data_ptr(), tx.data_ptr(), x.size, capi.CAST_RINT), kind)
        torch.cuda.synchronize()
        got = th.cpu().numpy().view(np.uint16).reshape(16384, 8192)
        for r0 in range(0, 16384, 2048):
            assert np.array_equal(got[r0:r0 + 2048], ofn(x[r0:r0 + 2048])), (kind, r0)


@pytest.mark.parametrize("rows,cols,nidx", [(64, 1024, 100), (16, 8, 1), (33, 264, 70), (128, 256, 32), (50, 2048, 31)])
def test_gather_rows_small(oracle, rows, cols, nidx):
    from gpu_util import gather_rows
    table, idx = datagen.gather_inputs(rows, cols, nidx)
    assert np.array_equal(gather_rows(table, idx), oracle.gather_rows(table, idx))
    t32 = np.random.default_rng(1).integers(0, 2**32, size=(rows, cols), dtype=np.uint64).astype(np.uint32)
    assert np.array_equal(gather_rows(t32, idx), oracle.gather_rows(t32, idx))


def test_gather_rows_out_of_range_indices_give_zero_rows(oracle):
    from gpu_util import gather_rows
    table, _ = datagen.gather_inputs(64, 512, 8)
    idx = np.array([0, 63, -1, 64, 5, 2**31 - 1, -2**31, 7], dtype=np.int32)
    got = gather_rows(table, idx)
    assert np.array_equal(got, oracle.gather_rows(table, idx))
    assert not got[2].any() and not got[3].any() and np.array_equal(got[4], table[5])


def test_gather_rows_full_size_config(oracle):
    """Config 5: 65536 int32 row indices over a 16384 x 1024 fp16 table: bit-exact copy."""
    from gpu_util import gather_rows
    table, idx = datagen.gather_inputs(16384, 1024, 65536)
    got = gather_rows(table, idx)
    assert np.array_equal(got, table[idx])
    assert np.array_equal(got[:4096], oracle.gather_rows(table, idx[:4096]))


def test_tgather_index_tile(oracle):
    """Index-form TGATHER on one tile pair (half 16x1024 -> 16x128 of the reference's tgather test),
    with out-of-range indices, against the oracle and the committed reference output."""
    from gpu_util import to_dev, stream
    lib = capi.load()
    rng = np.random.default_rng(9)
    src = rng.integers(0, 2**16, size=(16, 1024), dtype=np.uint16)
    idx = rng.integers(-50, 16 * 1024 + 50, size=(16, 128), dtype=np.int32)
    ts, ti = to_dev(src), to_dev(idx)
    td = torch.full((16, 128), -1, dtype=torch.int16, device="cuda:0")
    capi.check(lib.pto_tgather_index_f16_16x1024_16x128(stream(), td.data_ptr(), ts.data_ptr(), ti.data_ptr()), "tgather")
    torch.cuda.synchronize()
    got = td.cpu().numpy().view(np.uint16)
    o = oracle
    want = o.tgather_index(o.make_layout(16, 128), src.reshape(-1), o.make_layout(16, 1024), idx.reshape(-1),
                           o.make_layout(16, 128, elem_bytes=4), 16, 128).reshape(16, 128)
    assert np.array_equal(got, want)
    G = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_vectors.npz"))
    assert np.array_equal(got, G["tgather_index_f16_16x1024_16x128"])
