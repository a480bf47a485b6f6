"""GPU parity of the MXFP8 quantiser (TQUANT<QuantType::MXFP8>, include/pto/npu/a5/TQuant.hpp:262-322) through the C ABI:
bit-exact element and scale bytes against the oracle, the range invariant at the full size, and the quantised operands
fed to the MXFP8 GEMM."""
import numpy as np
import pytest
import torch

from pto_amd import capi, datagen

pytestmark = pytest.mark.gpu


def quant_gpu(x):
    from gpu_util import to_dev, stream
    lib = capi.load()
    rows, cols = x.shape
    tx = to_dev(x)
    q = torch.full((rows, cols), 0x55, dtype=torch.uint8, device="cuda:0")
    s = torch.full((rows, cols // 32), 0x55, dtype=torch.uint8, device="cuda:0")
    capi.check(lib.pto_quant_mxfp8_f32(stream(), q.data_ptr(), s.data_ptr(), tx.data_ptr(), rows, cols), "pto_quant_mxfp8_f32")
    torch.cuda.synchronize()
    return q.cpu().numpy(), s.cpu().numpy()


@pytest.mark.parametrize("rows,cols", [(1, 32), (3, 64), (8, 1024), (1, 8192), (5, 8192), (7, 1056), (33, 992), (256, 2048), (129, 4128)])
def test_quant_mxfp8_small_vs_oracle(oracle, rows, cols):
    """Whole tiles of 8192 elements, partial last tiles, single groups; scales over 24 binades and the special groups."""
    x = datagen.quant_input(rows, cols)
    q, s = quant_gpu(x)
    wq, ws = oracle.quant_mxfp8(x)
    assert np.array_equal(s, ws)
    assert np.array_equal(q, wq)


def test_quant_mxfp8_every_exponent(oracle):
    """One group per biased exponent 0 .. 255 of the group maximum (denormals, the clamp below 2^-119, infinities)."""
    g = np.zeros((256, 32), dtype=np.float32)
    rng = np.random.default_rng(5)
    for e in range(256):
        top = np.uint32(e << 23 | 0x2b0000).view(np.float32) if e < 255 else np.float32(np.inf)
        small = rng.uniform(-1, 1, 32).astype(np.float32)
        g[e] = small * (top if np.isfinite(top) else np.float32(1e30))
        g[e, e % 32] = top if e % 2 else -top
    q, s = quant_gpu(g.reshape(8, 1024))
    wq, ws = oracle.quant_mxfp8(g.reshape(8, 1024))
    assert np.array_equal(s, ws) and np.array_equal(q, wq)
    assert np.array_equal(ws.reshape(-1)[8:255], np.arange(0, 247, dtype=np.uint8))   # E - 8
    assert ws.reshape(-1)[255] == 0xff and not ws.reshape(-1)[:8].any()


def test_quant_mxfp8_full_size_invariants(oracle):
    """16384 x 8192 (the conversion workload's shape): scale byte = floor(log2(amax)) + 119, the largest element of every
    group lands in [256, 448], and a sample of rows is bit-exact."""
    rows, cols = 16384, 8192
    x = datagen.quant_input(rows, cols, spread=20, specials=False)
    q, s = quant_gpu(x)
    amax = np.abs(x).reshape(rows, cols // 32, 32).max(axis=2)
    _, ex = np.frexp(amax)                                   # amax = f * 2^ex, f in [0.5, 1)
    assert np.array_equal(s, (ex - 1 + 119).astype(np.uint8))
    mag = np.abs(datagen.fp8_values(0))[q].reshape(rows, cols // 32, 32).max(axis=2)
    assert mag.min() >= 256.0 and mag.max() <= 448.0
    pick = np.r_[0:64, rows // 2:rows // 2 + 64, rows - 64:rows]
    wq, ws = oracle.quant_mxfp8(x[pick])
    assert np.array_equal(q[pick], wq) and np.array_equal(s[pick], ws)


def test_quant_mxfp8_feeds_the_mx_gemm(oracle):
    """fp32 A, B -> quantised operands -> pto_gemm_mxfp8: equal to the oracle's GEMM of the same bytes (the GEMM's own bar),
    and close to the fp32 product by what 3 mantissa bits allow."""
    from gpu_util import to_dev, stream
    lib = capi.load()
    m, n, k = 256, 256, 1024
    rng = np.random.default_rng(11)
    a = (rng.standard_normal((m, k)) * np.exp2(rng.integers(-3, 4, size=(m, 1)))).astype(np.float32)
    b = (rng.standard_normal((n, k)) * np.exp2(rng.integers(-3, 4, size=(n, 1)))).astype(np.float32)
    (qa, sa), (qb, sb) = quant_gpu(a), quant_gpu(b)
    c = torch.zeros((m, n), dtype=torch.float32, device="cuda:0")
    ta, tb, tsa, tsb = (to_dev(t) for t in (qa, qb, sa, sb))
    capi.check(lib.pto_gemm_mxfp8(stream(), c.data_ptr(), ta.data_ptr(), tb.data_ptr(), tsa.data_ptr(), tsb.data_ptr(), m, n, k, 0, 1),
               "pto_gemm_mxfp8")
    torch.cuda.synchronize()
    got = c.cpu().numpy().astype(np.float64)
    want = oracle.mx_gemm(qa, qb, sa, sb, 0).astype(np.float64)
    assert np.max(np.abs(got - want)) <= 2e-3 * np.max(np.abs(want))
    exact = a.astype(np.float64) @ b.astype(np.float64).T
    # a 3-bit mantissa rounds with a relative error of up to 2^-4, about 2.7 % rms; a product of two such factors 3.8 %, and
    # a sum of independent terms keeps that ratio (measured 4.0 %)
    ratio = np.sqrt(np.mean((got - exact) ** 2)) / np.sqrt(np.mean(exact ** 2))
    assert 0.02 <= ratio <= 0.06


def test_quant_mxfp8_argument_checks():
    lib = capi.load()
    assert lib.pto_quant_mxfp8_f32(None, None, None, None, 0, 64) == capi.OK
    assert lib.pto_quant_mxfp8_f32(None, None, None, None, 4, 64) == capi.ERR_BAD_ARG
    d = torch.zeros(64, dtype=torch.float32, device="cuda:0")
    o = torch.zeros(64, dtype=torch.uint8, device="cuda:0")
    assert lib.pto_quant_mxfp8_f32(None, o.data_ptr(), o.data_ptr(), d.data_ptr(), 1, 48) == capi.ERR_UNSUPPORTED


@pytest.mark.parametrize("shape,R,C,vr,vc", [(0, 32, 32, 32, 32), (1, 32, 64, 32, 64), (2, 64, 128, 64, 128), (3, 128, 128, 128, 128),
                                             (1, 32, 64, 30, 40), (2, 64, 128, 1, 33), (3, 128, 128, 77, 128)])
def test_tquant_mxfp8_tile_instruction(oracle, shape, R, C, vr, vc):
    """TQUANT<QuantType::MXFP8> on one Vec tile in the ND cases of the reference's test (32 x 32 ... 128 x 128) and with
    partial valid regions (what lies outside counts as zeros): fp8 bytes, exponents, maxima and factors against the oracle."""
    from gpu_util import to_dev, stream
    lib = capi.load_st()
    x = datagen.quant_input(vr, 32 * ((vc + 31) // 32), spread=10, specials=(vr * vc >= 2048))[:, :vc].copy()
    padded = np.zeros((R, C), dtype=np.float32)
    padded[:vr, :vc] = x
    G = R * C // 32
    e8 = torch.full((G,), 0x55, dtype=torch.uint8, device="cuda:0")
    q = torch.full((R, C), 0x55, dtype=torch.uint8, device="cuda:0")
    mx = torch.zeros((G,), dtype=torch.float32, device="cuda:0")
    sc = torch.zeros((R, C), dtype=torch.float32, device="cuda:0")
    capi.check(lib.pto_st_tquant_mxfp8(stream(), e8.data_ptr(), q.data_ptr(), mx.data_ptr(), sc.data_ptr(), to_dev(x).data_ptr(),
                                       shape, vr, vc), "pto_st_tquant_mxfp8")
    torch.cuda.synchronize()
    wq, we, wmax, wscale = oracle.quant_mxfp8(padded, with_stats=True)
    assert np.array_equal(e8.cpu().numpy(), we.reshape(-1))
    assert np.array_equal(q.cpu().numpy(), wq)
    assert np.array_equal(mx.cpu().numpy().view(np.uint32), wmax.reshape(-1).view(np.uint32))
    got_scale = sc.cpu().numpy().reshape(-1)[:G]
    ordinary = we.reshape(-1) != 0xff                      # a group with inf / NaN: the factor is the bit pattern 0xff
    assert np.array_equal(got_scale[ordinary], wscale.reshape(-1)[ordinary])
    assert np.all(got_scale[~ordinary].view(np.uint32) == 0xff)


def test_quant_mxfp8_refuses_pointers_below_the_alignment_of_its_accesses():
    lib = capi.load()
    d = torch.zeros(128, dtype=torch.float32, device="cuda:0")
    o = torch.zeros(128, dtype=torch.uint8, device="cuda:0")
    assert lib.pto_quant_mxfp8_f32(None, o.data_ptr(), o.data_ptr(), d.data_ptr() + 4, 1, 64) == capi.ERR_UNSUPPORTED
    assert lib.pto_quant_mxfp8_f32(None, o.data_ptr() + 2, o.data_ptr(), d.data_ptr(), 1, 64) == capi.ERR_UNSUPPORTED
    assert lib.pto_quant_mxfp8_f32(None, o.data_ptr(), o.data_ptr() + 1, d.data_ptr(), 1, 64) == capi.OK
    torch.cuda.synchronize()
