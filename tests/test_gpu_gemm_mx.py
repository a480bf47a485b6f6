"""GPU parity of the MXFP8 / MXFP4 GEMMs (TLOAD -> TEXTRACT -> TMATMUL_MX -> TSTORE) through the C ABI.

Reference: the oracle's float64 matmul of the dequantised operands (the golden of the reference's tmatmul_mx test
and of its matmul_mxfp8_performance kernel).  Products of two scaled fp8 values are exact in fp32; the GPU adds them in
fp32 in the MFMA's order, so the bar is the GEMM path's: max |gpu - ref| <= 2e-3 * max|ref| (observed ~1e-6), exact on
integer-valued operands.  The bf16 result must be the round-to-nearest-even of the fp32 result, bit for bit."""
import numpy as np
import pytest

from pto_amd import capi, datagen

pytestmark = pytest.mark.gpu

TOL = 2e-3


def rel_err(got, want):
    return float(np.max(np.abs(got - want)) / np.max(np.abs(want)))


def bf16_rne(x):
    """float32 array -> bf16 bit patterns, round to nearest even (finite inputs)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


@pytest.mark.parametrize("fmt", [0, 1, 4])
@pytest.mark.parametrize("m,n,k", [(256, 256, 512), (256, 512, 1024), (512, 256, 1536), (768, 768, 2048)])
def test_mx_gemm_small_vs_oracle(oracle, m, n, k, fmt):
    from gpu_util import gemm_mx
    a, b, sa, sb = datagen.mx_inputs(m, n, k, fmt)
    got = gemm_mx(a, b, sa, sb, fmt)
    want = oracle.mx_gemm(a, b, sa, sb, fmt)
    assert np.all(np.isfinite(got))
    assert rel_err(got, want) <= TOL
    got16 = gemm_mx(a, b, sa, sb, fmt, c_fp32=False)
    assert np.array_equal(got16, bf16_rne(got))


@pytest.mark.parametrize("fmt_a,fmt_b,code", [(0, 1, 2), (1, 0, 3)])
def test_mx_gemm_mixed_fp8_formats(oracle, fmt_a, fmt_b, code):
    """A in e4m3 and B in e5m2 (format 2) and the other way round (3): every finite byte pattern of either format meets the
    other (the byte 0x7c is 320 in e4m3 and +inf in e5m2, so a swapped format pair cannot pass), then integers, exactly."""
    from gpu_util import gemm_mx
    m, n, k = 512, 768, 1024
    a, _, sa, sb = datagen.mx_inputs(m, n, k, fmt_a, dist="bytes")
    _, b, _, _ = datagen.mx_inputs(m, n, k, fmt_b, dist="bytes")
    got = gemm_mx(a, b, sa, sb, code)
    want = oracle.mx_gemm(a, b, sa, sb, fmt_a, fmt_b)
    assert np.all(np.isfinite(got)) and rel_err(got, want) <= TOL
    wrong = oracle.mx_gemm(a, b, sa, sb, fmt_b, fmt_a)
    assert rel_err(got, wrong) > 10 * TOL or not np.all(np.isfinite(wrong))
    ai, _, sa, sb = datagen.mx_inputs(m, n, k, fmt_a, dist="integer")
    _, bi, _, _ = datagen.mx_inputs(m, n, k, fmt_b, dist="integer")
    assert np.array_equal(gemm_mx(ai, bi, sa, sb, code), oracle.mx_gemm(ai, bi, sa, sb, fmt_a, fmt_b))
    got16 = gemm_mx(a, b, sa, sb, code, c_fp32=False)
    assert np.array_equal(got16, bf16_rne(got))


@pytest.mark.parametrize("fmt", [0, 1, 4])
def test_mx_gemm_integer_operands_exact(oracle, fmt):
    """Integers in [-10, 10) (those fp8 can hold) and scales 2^0 .. 2^2: every partial sum is an integer below 2^24,
    exact in fp32 in any order, so a wrong fragment byte order, k-block / scale pairing or dropped step cannot hide."""
    from gpu_util import gemm_mx
    a, b, sa, sb = datagen.mx_inputs(512, 512, 1024, fmt, dist="integer")
    got = gemm_mx(a, b, sa, sb, fmt)
    want = oracle.mx_gemm(a, b, sa, sb, fmt)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("fmt", [0, 1, 4])
def test_mx_gemm_scale_of_every_block_is_applied(oracle, fmt):
    """Operands of all ones: C[i,j] = 32 * sum_kb 2^(sa[i,kb] + sb[j,kb] - 254), scales drawn from a wide range, so the
    result identifies which scale byte met which k block of which row and column."""
    from gpu_util import gemm_mx
    m, n, k = 256, 512, 1024
    one = datagen.fp8_encode(np.ones(1), fmt)[0]
    a = np.full((m, k), one, dtype=np.uint8)
    b = np.full((n, k), one, dtype=np.uint8)
    if fmt == 4:
        a, b = datagen.fp4_pack(a), datagen.fp4_pack(b)
    _, _, sa, sb = datagen.mx_inputs(m, n, k, fmt, scale_lo=123, scale_hi=131)
    got = gemm_mx(a, b, sa, sb, fmt)
    want = 32.0 * (np.exp2(sa.astype(np.float64) - 127) @ np.exp2(sb.astype(np.float64) - 127).T)
    assert np.array_equal(got, want.astype(np.float32))       # multiples of 2^-3 below 2^16: exact in any order
    assert np.array_equal(got, oracle.mx_gemm(a, b, sa, sb, fmt))
    # a wide range of scales (2^-20 .. 2^20 per product): fp32 rounding only
    _, _, sa, sb = datagen.mx_inputs(m, n, k, fmt, scale_lo=117, scale_hi=138)
    got = gemm_mx(a, b, sa, sb, fmt)
    want = 32.0 * (np.exp2(sa.astype(np.float64) - 127) @ np.exp2(sb.astype(np.float64) - 127).T)
    assert np.max(np.abs(got - want) / want) <= 1e-5


@pytest.mark.parametrize("fmt", [0, 1, 4])
def test_mx_gemm_every_encoding(oracle, fmt):
    """Random finite bytes (subnormals, both zeros, the largest values) and a wide range of scales."""
    from gpu_util import gemm_mx
    a, b, sa, sb = datagen.mx_inputs(256, 256, 512, fmt, dist="bytes", scale_lo=100, scale_hi=150)
    got = gemm_mx(a, b, sa, sb, fmt)
    want = oracle.mx_gemm(a, b, sa, sb, fmt)
    assert rel_err(got, want) <= TOL


def test_mx_gemm_quarter_tile_round(oracle):
    """4096 x 4352: 272 tiles = one full round over 256 compute units plus 16 tiles cut into 128 x 128 quarter tiles."""
    from gpu_util import gemm_mx
    m, n, k = 4096, 4352, 512
    a, b, sa, sb = datagen.mx_inputs(m, n, k, 1, dist="integer")
    got = gemm_mx(a, b, sa, sb, 1)
    rows = np.r_[0:32, m // 2:m // 2 + 32, m - 32:m]
    want = oracle.mx_gemm(a[rows], b, sa[rows], sb, 1)
    assert np.array_equal(got[rows], want)
    # every row: the row sums against (A dequantised) @ (column sums of B dequantised), exact in float64
    tab = datagen.fp8_values(1)
    bd = tab[b] * np.repeat(np.exp2(sb.astype(np.float64) - 127), 32, axis=1)
    ad = tab[a] * np.repeat(np.exp2(sa.astype(np.float64) - 127), 32, axis=1)
    assert np.array_equal(got.astype(np.float64).sum(axis=1), ad @ bd.sum(axis=0))


@pytest.mark.parametrize("fmt,m,n,k", [(1, 300, 700, 1024), (0, 257, 511, 512), (4, 1000, 260, 1024)])
def test_mx_gemm_ragged_m_n(oracle, fmt, m, n, k):
    """m, n that are not multiples of the 256 x 256 tile: the last tile row / column overlaps its neighbour."""
    from gpu_util import gemm_mx
    a, b, sa, sb = datagen.mx_inputs(m, n, k, fmt, dist="integer")
    got = gemm_mx(a, b, sa, sb, fmt)
    assert np.array_equal(got, oracle.mx_gemm(a, b, sa, sb, fmt))
    got16 = gemm_mx(a, b, sa, sb, fmt, c_fp32=False)
    assert np.array_equal(got16, bf16_rne(got))


def _mx_variant(a, b, sa, sb, fmt, variant, c_fp32=True):
    """pto_gemm_mxfp8_variant of the test library: one kernel whatever the public entry point would pick."""
    import torch
    from gpu_util import to_dev
    lib = capi.load_st()
    (m, k), n = a.shape, b.shape[0]
    if fmt == 4:
        k *= 2      # two e2m1 per byte
    ta, tb, tsa, tsb = (to_dev(x) for x in (a, b, sa, sb))
    tc = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0") if c_fp32 else \
        torch.full((m, n), -1, dtype=torch.int16, device="cuda:0")
    rc = lib.pto_gemm_mxfp8_variant(0, tc.data_ptr(), ta.data_ptr(), tb.data_ptr(), tsa.data_ptr(), tsb.data_ptr(), m, n, k, fmt,
                                    int(c_fp32), variant)
    torch.cuda.synchronize()
    out = tc.cpu().numpy()
    return rc, (out if c_fp32 else out.view(np.uint16))


@pytest.mark.parametrize("variant", [5, 6])
@pytest.mark.parametrize("m,n,k", [(256, 192, 512), (256, 512, 1024), (512, 384, 1536), (768, 768, 2048), (300, 260, 512),
                                   (1000, 1100, 1024)])
def test_mx_gemm_four_wave_kernel(oracle, m, n, k, variant):
    """The MXFP8 kernel on four wavefronts (256 x 192 and 256 x 128 tiles; one, two and four groups of four K-steps; m and n
    that the tiles do not divide): integer operands exactly, the generator's distribution to the GEMM tolerance, both fp8
    formats and a mixed pair, the bf16 result = RNE of the fp32 one."""
    for fmt in (0, 1):
        a, b, sa, sb = datagen.mx_inputs(m, n, k, fmt, dist="integer")
        rc, got = _mx_variant(a, b, sa, sb, fmt, variant)
        capi.check(rc, "four-wave MX kernel")
        assert np.array_equal(got, oracle.mx_gemm(a, b, sa, sb, fmt)), (fmt, "integer")
        a, b, sa, sb = datagen.mx_inputs(m, n, k, fmt)
        rc, got = _mx_variant(a, b, sa, sb, fmt, variant)
        assert rc == 0 and np.all(np.isfinite(got)) and rel_err(got, oracle.mx_gemm(a, b, sa, sb, fmt)) <= TOL
        rc, got16 = _mx_variant(a, b, sa, sb, fmt, variant, c_fp32=False)
        assert rc == 0 and np.array_equal(got16, bf16_rne(got))
    a, _, sa, sb = datagen.mx_inputs(m, n, k, 0, dist="bytes")
    _, b, _, _ = datagen.mx_inputs(m, n, k, 1, dist="bytes")
    rc, got = _mx_variant(a, b, sa, sb, 2, variant)
    assert rc == 0 and np.all(np.isfinite(got)) and rel_err(got, oracle.mx_gemm(a, b, sa, sb, 0, 1)) <= TOL
    a3, _, sa3, sb3 = datagen.mx_inputs(m, n, k, 1, dist="bytes")
    _, b3, _, _ = datagen.mx_inputs(m, n, k, 0, dist="bytes")
    rc, got = _mx_variant(a3, b3, sa3, sb3, 3, variant)
    assert rc == 0 and np.all(np.isfinite(got)) and rel_err(got, oracle.mx_gemm(a3, b3, sa3, sb3, 1, 0)) <= TOL


def test_mx_gemm_four_wave_kernel_scale_of_every_block(oracle):
    """Every (row, k block) scale of A and every (column, k block) scale of B reaches its products: operands of ones, scales
    drawn per block from {2^-2 .. 2^3}, so that C[i, j] = 32 sum_b 2^(sa[i, b] + sb[j, b] - 254) exactly."""
    m, n, k = 512, 384, 2048
    rng = np.random.default_rng(77)
    one = 0x38  # 1.0 in e4m3
    a = np.full((m, k), one, dtype=np.uint8)
    b = np.full((n, k), one, dtype=np.uint8)
    sa = rng.integers(125, 131, size=(m, k // 32)).astype(np.uint8)
    sb = rng.integers(125, 131, size=(n, k // 32)).astype(np.uint8)
    want = 32.0 * (np.exp2(sa.astype(np.float64) - 127) @ np.exp2(sb.astype(np.float64) - 127).T)
    for variant in (5, 6):
        rc, got = _mx_variant(a, b, sa, sb, 0, variant)
        assert rc == 0 and np.array_equal(got.astype(np.float64), want), variant
    assert np.array_equal(want, oracle.mx_gemm(a, b, sa, sb, 0).astype(np.float64))


@pytest.mark.parametrize("variant", [5, 6])
@pytest.mark.parametrize("m,n,k", [(256, 192, 1024), (256, 512, 2048), (512, 384, 3072), (300, 260, 1024), (1000, 1100, 2048)])
def test_mxfp4_gemm_four_wave_kernel(oracle, m, n, k, variant):
    """The four-wave kernel with e2m1 operands (two matrix instructions per 16 x 16 block and K-step of 256 k, the 16 scale
    bytes of a row last two steps): the generator's integers exactly, every encoding with a wide range of scales to the GEMM
    tolerance, the bf16 result = RNE of the fp32 one."""
    a, b, sa, sb = datagen.mx_inputs(m, n, k, 4)
    rc, got = _mx_variant(a, b, sa, sb, 4, variant)
    capi.check(rc, "four-wave MX kernel, fp4")
    assert np.array_equal(got, oracle.mx_gemm(a, b, sa, sb, 4))
    a, b, sa, sb = datagen.mx_inputs(m, n, k, 4, dist="bytes", scale_lo=110, scale_hi=140)
    rc, got = _mx_variant(a, b, sa, sb, 4, variant)
    assert rc == 0 and np.all(np.isfinite(got)) and rel_err(got, oracle.mx_gemm(a, b, sa, sb, 4)) <= TOL
    rc, got16 = _mx_variant(a, b, sa, sb, 4, variant, c_fp32=False)
    assert rc == 0 and np.array_equal(got16, bf16_rne(got))


def test_mxfp4_gemm_four_wave_kernel_scale_of_every_block(oracle):
    """As for fp8: operands of ones, scales drawn per block, C[i, j] = 32 sum_b 2^(sa[i, b] + sb[j, b] - 254) exactly."""
    m, n, k = 512, 384, 4096
    rng = np.random.default_rng(78)
    ones = datagen.fp4_pack(np.full((1, k), datagen.fp8_encode(np.ones(1), 4)[0], dtype=np.uint8))
    a, b = np.repeat(ones, m, axis=0), np.repeat(ones, n, axis=0)
    sa = rng.integers(125, 131, size=(m, k // 32)).astype(np.uint8)
    sb = rng.integers(125, 131, size=(n, k // 32)).astype(np.uint8)
    want = 32.0 * (np.exp2(sa.astype(np.float64) - 127) @ np.exp2(sb.astype(np.float64) - 127).T)
    for variant in (5, 6):
        rc, got = _mx_variant(a, b, sa, sb, 4, variant)
        assert rc == 0 and np.array_equal(got.astype(np.float64), want), variant
    assert np.array_equal(want, oracle.mx_gemm(a, b, sa, sb, 4).astype(np.float64))


@pytest.mark.parametrize("fmt", [0, 4])
def test_mx_gemm_public_entry_narrow_n_and_kernel_choice(oracle, fmt):
    """128 <= n < 256 (four-wave kernel only) and shapes on either side of the entry points' choice between the kernels:
    the same exact result on integer data whichever runs."""
    from gpu_util import gemm_mx
    for m, n, k in ((256, 160, 1024), (512, 252, 2048), (1024, 1024, 1024), (2048, 3072, 1024), (512, 258, 1024)):
        a, b, sa, sb = datagen.mx_inputs(m, n, k, fmt, dist="integer")
        assert np.array_equal(gemm_mx(a, b, sa, sb, fmt), oracle.mx_gemm(a, b, sa, sb, fmt)), (m, n, k)


@pytest.mark.parametrize("variant", [5, 6])
@pytest.mark.parametrize("fmt,m,n,k", [(0, 256, 192, 2560), (1, 512, 384, 3584), (0, 256, 256, 4608), (4, 256, 192, 5120),
                                       (4, 512, 384, 7168), (4, 256, 256, 9216)])
def test_mx_gemm_four_wave_kernel_scale_periods(oracle, fmt, m, n, k, variant):
    """K extents that end inside a scale period of the four-wave kernel (64 scale bytes of a row = 16 K-steps of fp8, 8 of
    fp4, loaded at once; K is whole groups of four steps only): scales drawn per block from a wide range with operands of
    ones, so that a scale register taken from the wrong quarter or period shows, then the generator's data exactly."""
    rng = np.random.default_rng(k + fmt)
    one = datagen.fp8_encode(np.ones(1), fmt)[0]
    a, b = np.full((m, k), one, dtype=np.uint8), np.full((n, k), one, dtype=np.uint8)
    if fmt == 4:
        a, b = datagen.fp4_pack(a), datagen.fp4_pack(b)
    sa = rng.integers(124, 131, size=(m, k // 32)).astype(np.uint8)
    sb = rng.integers(124, 131, size=(n, k // 32)).astype(np.uint8)
    want = 32.0 * (np.exp2(sa.astype(np.float64) - 127) @ np.exp2(sb.astype(np.float64) - 127).T)
    rc, got = _mx_variant(a, b, sa, sb, fmt, variant)
    assert rc == 0 and np.array_equal(got.astype(np.float64), want)
    a, b, sa, sb = datagen.mx_inputs(m, n, k, fmt, dist="integer")
    rc, got = _mx_variant(a, b, sa, sb, fmt, variant)
    assert rc == 0 and np.array_equal(got, oracle.mx_gemm(a, b, sa, sb, fmt))


def test_mx_gemm_four_wave_kernel_refuses():
    import torch
    p = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda:0").data_ptr()
    fn = capi.load_st().pto_gemm_mxfp8_variant
    assert fn(0, p, p, p, p, p, 128, 512, 512, 0, 1, 5) == capi.ERR_UNSUPPORTED     # fewer than 256 rows
    assert fn(0, p, p, p, p, p, 256, 160, 512, 0, 1, 5) == capi.ERR_UNSUPPORTED     # narrower than the tile
    assert fn(0, p, p, p, p, p, 256, 258, 512, 0, 1, 6) == capi.ERR_UNSUPPORTED     # rows of C not a multiple of four elements
    assert fn(0, p, p, p, p, p, 256, 256, 640, 0, 1, 6) == capi.ERR_UNSUPPORTED     # k not whole groups of four steps
    assert fn(0, p, p, p, p, p, 256, 256, 1536, 4, 1, 6) == capi.ERR_UNSUPPORTED    # the same for fp4 (a step is 256 k)


def test_mxfp4_gemm_reference_config_2040_8192_8100(oracle):
    """The reference's matmul_mxfp4_performance case: e2m1 operands, m, k, n = 2040, 8192, 8100, bf16 result, its generator's
    integer distribution in [-6, 6) and scales 2^0 .. 2^2: partial sums stay below 2^24, so the fp32 result is exact."""
    from gpu_util import gemm_mx
    m, k, n = 2040, 8192, 8100
    a, b, sa, sb = datagen.mx_inputs(m, n, k, 4)
    got = gemm_mx(a, b, sa, sb, 4)
    rows = np.r_[0:24, 1000:1024, m - 24:m]
    want = oracle.mx_gemm(a[rows], b, sa[rows], sb, 4)
    assert np.array_equal(got[rows], want)
    got16 = gemm_mx(a, b, sa, sb, 4, c_fp32=False)
    assert np.array_equal(got16, bf16_rne(got))
    # every row: row sums against (A dequantised) @ (column sums of B dequantised), exact in float64
    tab = datagen.fp4_values()
    bd = tab[datagen.fp4_unpack(b)] * np.repeat(np.exp2(sb.astype(np.float64) - 127), 32, axis=1)
    ad = tab[datagen.fp4_unpack(a)] * np.repeat(np.exp2(sa.astype(np.float64) - 127), 32, axis=1)
    assert np.array_equal(got.astype(np.float64).sum(axis=1), ad @ bd.sum(axis=0))


def test_mx_gemm_reference_config_6144(oracle):
    """The reference kernel's case: e5m2, 6144^3, bf16 result, its generator's distribution; 96 rows against the oracle and
    the bf16 result against the fp32 one."""
    from gpu_util import gemm_mx
    m = n = k = 6144
    a, b, sa, sb = datagen.mx_inputs(m, n, k, 1)
    got = gemm_mx(a, b, sa, sb, 1)
    rows = np.r_[0:32, 3000:3032, m - 32:m]
    want = oracle.mx_gemm(a[rows], b, sa[rows], sb, 1)
    assert rel_err(got[rows], want) <= TOL
    got16 = gemm_mx(a, b, sa, sb, 1, c_fp32=False)
    assert np.array_equal(got16, bf16_rne(got))
    # bf16 results against the oracle's: never more than one bf16 step apart (a step = a flipped rounding of sums that
    # differ in the last fp32 bits), and few of those
    def ordered(u16):
        v = u16.astype(np.int32)
        return np.where(v & 0x8000, 0x8000 - v, v)
    steps = np.abs(ordered(got16[rows]) - ordered(bf16_rne(want)))
    big = np.abs(want) >= np.max(np.abs(want)) / 256          # (sums that cancel to near zero have no relative accuracy)
    assert steps[big].max() <= 1
    assert np.count_nonzero(steps[big]) <= 0.005 * np.count_nonzero(big)
    # The reference's own check is ResultCmp(golden, out, 0.001) (main.cpp:19-33): an element is bad when it is off by more
    # than 1e-3 both absolutely and relatively, and 0.1 % of the elements may be bad.  The scaled MFMA sums its 64 products
    # and the accumulator with about 20 bits (measured: mean |error| 2e-2 on sums of magnitude 5e3, 1e-5 of the largest),
    # so the sums that cancel to less than about 20 (0.3-0.6 % of the elements with this distribution) are bad by that
    # definition, on the fp32 result as on the bf16 one; the count is recorded here, the bar above is the one asserted.
    ok, max_diff, n_bad = oracle.result_cmp(want, got[rows], 0.001)
    print("ResultCmp(eps 0.001) on the fp32 result: ok", ok, "max diff", max_diff, "bad", n_bad, "of", want.size)
    assert n_bad <= 0.01 * want.size and max_diff <= 1.0


def test_mx_gemm_rejects_bad_arguments():
    import torch
    lib = capi.load()
    t = torch.zeros(16, device="cuda:0")
    p = t.data_ptr()
    assert lib.pto_gemm_mxfp8(0, p, p, p, p, p, 256, 256, 256, 0, 1) == capi.ERR_UNSUPPORTED   # k % 512
    assert lib.pto_gemm_mxfp8(0, p, p, p, p, p, 128, 256, 512, 0, 1) == capi.ERR_UNSUPPORTED   # m < 256
    assert lib.pto_gemm_mxfp8(0, p, p, p, p, p, 256, 256, 512, 4, 1) == capi.ERR_UNSUPPORTED   # fp4 has its own entry point
    assert lib.pto_gemm_mxfp4(0, p, p, p, p, p, 256, 256, 768, 1) == capi.ERR_UNSUPPORTED      # k % 512
    assert lib.pto_gemm_mxfp4(0, p, 0, p, p, p, 256, 256, 512, 1) == capi.ERR_BAD_ARG
    assert lib.pto_gemm_mxfp8(0, p, p, p, p, p, 256, 256, 512, 5, 1) == capi.ERR_UNSUPPORTED   # unknown format
    assert lib.pto_gemm_mxfp8(0, p, p, p, 0, p, 256, 256, 512, 0, 1) == capi.ERR_BAD_ARG
    assert lib.pto_gemm_mxfp8(0, p, p, p, p, p, 256, 0, 512, 0, 1) == capi.ERR_BAD_ARG
