"""Seeded synthetic inputs for the five benchmark/parity workloads.

One documented seed per tensor, drawn from numpy's counter-based Philox generator so that
the same bytes are produced on every host.  Shapes follow the reference's kernels:
A [m,k] fp16 row-major and B stored [n,k] fp16 (a column-major k x n operand) as in
kernels/manual/a2a3/gemm_performance/scripts/gen_data.py:26-38; Q/K/V [B,H,S,D] fp16.
"""
import numpy as np

SEED_GEMM_A = 19          # echoes np.random.seed(19) of the reference's gen_data.py:16
SEED_GEMM_B = 1019
SEED_FA_Q, SEED_FA_K, SEED_FA_V = 7, 1007, 2007   # reference FA golden uses seed 7
SEED_TCVT = 3001
SEED_TCVT_INJECT = 3002
SEED_GATHER_TABLE = 4001
SEED_GATHER_IDX = 4002
SEED_MX_A, SEED_MX_B, SEED_MX_SA, SEED_MX_SB = 19, 2019, 3019, 4019
SEED_TOPK = 5019


def _rng(seed):
    return np.random.Generator(np.random.Philox(key=seed))


def gemm_inputs(m, n, k):
    """A [m,k], B [n,k] fp16, i.i.d. uniform[-1,1] drawn in fp32 then rounded RNE."""
    a = _rng(SEED_GEMM_A).uniform(-1.0, 1.0, size=(m, k)).astype(np.float32).astype(np.float16)
    b = _rng(SEED_GEMM_B).uniform(-1.0, 1.0, size=(n, k)).astype(np.float32).astype(np.float16)
    return a, b


def gemm_inputs_integer(m, n, k):
    """Integer-valued operands in [1,5): fp32 accumulation is exact (tmatmul/gen_data.py:40-41)."""
    a = _rng(SEED_GEMM_A).integers(1, 5, size=(m, k)).astype(np.float16)
    b = _rng(SEED_GEMM_B).integers(1, 5, size=(n, k)).astype(np.float16)
    return a, b


def fa_inputs(batch, heads, seq_q, seq_kv, head_dim, scale=1.0):
    """Q [B,H,Sq,D], K,V [B,H,Skv,D] fp16, N(0,1)*scale."""
    def one(seed, s):
        x = _rng(seed).standard_normal(size=(batch, heads, s, head_dim), dtype=np.float32) * np.float32(scale)
        return x.astype(np.float16)
    return one(SEED_FA_Q, seq_q), one(SEED_FA_K, seq_kv), one(SEED_FA_V, seq_kv)


def tcvt_input(rows, cols, inject=0.001):
    """fp32 N(0,100) with a fraction `inject` of positions overwritten by specials: +-inf, NaN,
    fp32 denormals, values straddling the fp16 overflow threshold (65504/65520) and the fp16
    subnormal range, and exact rounding ties."""
    n = rows * cols
    x = (_rng(SEED_TCVT).standard_normal(size=n, dtype=np.float32) * np.float32(100.0))
    r = _rng(SEED_TCVT_INJECT)
    cnt = int(n * inject)
    if cnt:
        pos = r.integers(0, n, size=cnt)
        specials = np.array([
            0x7f800000, 0xff800000, 0x7fc00000, 0xffc00000, 0x7f800001, 0x7fa12345,  # inf, NaNs (quiet/signalling)
            0x00000001, 0x80000001, 0x007fffff, 0x00400000,                          # fp32 denormals
            0x477fe000, 0x477fefff, 0x477ff000, 0x477ff001, 0xc77ff000, 0x47800000,  # 65504 .. 65520 .. 65536
            0x33000000, 0x33000001, 0x33800000, 0x33c00000, 0x387fc000, 0x387fe000,  # fp16 subnormal edges
            0x38800000, 0x3f801000, 0x3f803000, 0x3f801001, 0x3f802fff,              # ties in the normal range
            0x00000000, 0x80000000, 0x7f7fffff, 0xff7fffff,
        ], dtype=np.uint32)
        xv = x.view(np.uint32)
        xv[pos] = specials[r.integers(0, specials.size, size=cnt)]
        # a slice of fully random bit patterns too
        rnd = r.integers(0, 2**32, size=cnt // 4 + 1, dtype=np.uint64).astype(np.uint32)
        xv[r.integers(0, n, size=rnd.size)] = rnd
    return x.reshape(rows, cols)


def fp8_values(fmt):
    """The 256 values of float8_e4m3fn (fmt 0: 1-4-3, bias 7, no infinities, 0x7f / 0xff NaN) or float8_e5m2
    (fmt 1: 1-5-2, bias 15, IEEE-style infinities and NaNs) as float64, indexed by the byte."""
    v = np.arange(256)
    s = np.where(v & 0x80, -1.0, 1.0)
    if fmt == 0:
        e, f = (v >> 3) & 0xF, (v & 7).astype(np.float64)
        mag = np.where(e == 0, f * 2.0 ** -9, (8 + f) * 2.0 ** (e.astype(np.float64) - 10))
        mag = np.where((e == 0xF) & (f == 7), np.nan, mag)
    else:
        e, f = (v >> 2) & 0x1F, (v & 3).astype(np.float64)
        mag = np.where(e == 0, f * 2.0 ** -16, (4 + f) * 2.0 ** (e.astype(np.float64) - 17))
        mag = np.where(e == 0x1F, np.where(f == 0, np.inf, np.nan), mag)
    return s * mag


def fp4_values():
    """The 16 values of float4_e2m1 (1-2-1, bias 1: 0, 0.5, 1, 1.5, 2, 3, 4, 6 and their negatives) indexed by the nibble."""
    mag = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
    return np.concatenate([mag, -mag])


def fp4_pack(nibbles):
    """[rows, k] nibbles -> [rows, k/2] bytes, element 2i in the low half (pack_two_fp4, tmatmul_mx/gen_data.py:74-84)."""
    nib = np.asarray(nibbles, dtype=np.uint8)
    return (nib[:, 0::2] & 15) | ((nib[:, 1::2] & 15) << 4)


def fp4_unpack(packed):
    p = np.asarray(packed, dtype=np.uint8)
    out = np.empty((p.shape[0], p.shape[1] * 2), dtype=np.uint8)
    out[:, 0::2] = p & 15
    out[:, 1::2] = p >> 4
    return out


def fp8_encode(x, fmt):
    """float array -> fp8 bytes (fmt 0 / 1) or fp4 nibbles (fmt 4), nearest finite value (saturating); a tie takes the
    lower value."""
    tab = fp4_values() if fmt == 4 else fp8_values(fmt)
    finite = np.flatnonzero(np.isfinite(tab) & ~((np.arange(tab.size) == tab.size // 2)))      # one zero: +0
    order = finite[np.argsort(tab[finite], kind="stable")]
    vals = tab[order]
    x = np.asarray(x, dtype=np.float64)
    hi = np.clip(np.searchsorted(vals, x), 1, vals.size - 1)
    lo = hi - 1
    pick = np.where(np.abs(x - vals[lo]) <= np.abs(vals[hi] - x), lo, hi)
    return order[pick].astype(np.uint8)


SEED_QUANT = 20260131


def quant_input(rows, cols, spread=12, specials=True):
    """fp32 [rows, cols] for the MXFP8 quantiser: N(0, 1) with every group of 32 multiplied by its own power of two in
    2^[-spread, spread]; with `specials`, a few groups are made all zero, tiny (below 2^-119, fp32 denormals included),
    huge, or get an infinity, a NaN or a -0."""
    assert cols % 32 == 0
    r = _rng(SEED_QUANT + rows * 131 + cols)
    x = r.standard_normal(size=(rows, cols // 32, 32), dtype=np.float32)
    x *= np.exp2(r.integers(-spread, spread + 1, size=(rows, cols // 32, 1))).astype(np.float32)
    if specials:
        g = x.reshape(-1, 32)
        n = g.shape[0]
        pick = r.permutation(n)[:min(n, 48)]
        for j, gi in enumerate(pick):
            kind = j % 8
            if kind == 0:
                g[gi] = 0.0
            elif kind == 1:
                g[gi] = (r.standard_normal(32) * 1e-40).astype(np.float32)
            elif kind == 2:
                g[gi] = (r.standard_normal(32) * 2.0 ** -122).astype(np.float32)
            elif kind == 3:
                g[gi] = (r.standard_normal(32) * 1e38).clip(-3.4e38, 3.4e38).astype(np.float32)
            elif kind == 4:
                g[gi, r.integers(0, 32)] = np.inf if j % 16 < 8 else -np.inf
            elif kind == 5:
                g[gi, r.integers(0, 32)] = np.nan
                g[gi, r.integers(0, 32)] = -np.inf
            elif kind == 6:
                g[gi, ::3] = -0.0
            else:
                g[gi] = np.float32(448.0) * np.sign(g[gi])          # every element at the top of the range
    return x.reshape(rows, cols)


def mx_inputs(m, n, k, fmt, dist="uniform", scale_lo=127, scale_hi=130):
    """Operands of the MX GEMMs: A [m,k], B [n,k] fp8 bytes (fmt 0 e4m3, 1 e5m2) or [m,k/2], [n,k/2] packed fp4 (fmt 4),
    SA [m,k/32], SB [n,k/32] e8m0 bytes.  For fp4 "uniform" and "integer" draw integers in [-6, 6) as the reference's
    generators do (matmul_mxfp4_performance/scripts/gen_data.py, tmatmul_mx/gen_data.py:108-111).

    dist "uniform": uniform(-5, 5) rounded to fp8 and scales in [127, 130), the distribution of
    kernels/manual/a5/matmul_mxfp8_performance/scripts/gen_data.py:31-38; "integer": integers in [-10, 10) as in
    tests/npu/a5/src/st/testcase/tmatmul_mx/gen_data.py:113-120; "bytes": every finite encoding, subnormals included."""
    ra, rb = _rng(SEED_MX_A), _rng(SEED_MX_B)
    if fmt == 4:
        if dist == "bytes":
            a, b = ra.integers(0, 16, size=(m, k)), rb.integers(0, 16, size=(n, k))
        else:
            a, b = fp8_encode(ra.integers(-6, 6, size=(m, k)), 4), fp8_encode(rb.integers(-6, 6, size=(n, k)), 4)
        a, b = fp4_pack(a), fp4_pack(b)
    elif dist == "uniform":
        a = fp8_encode(ra.uniform(-5.0, 5.0, size=(m, k)), fmt)
        b = fp8_encode(rb.uniform(-5.0, 5.0, size=(n, k)), fmt)
    elif dist == "integer":
        a = fp8_encode(ra.integers(-10, 10, size=(m, k)), fmt)
        b = fp8_encode(rb.integers(-10, 10, size=(n, k)), fmt)
    else:
        finite = np.flatnonzero(np.isfinite(fp8_values(fmt))).astype(np.uint8)
        a = finite[ra.integers(0, finite.size, size=(m, k))]
        b = finite[rb.integers(0, finite.size, size=(n, k))]
    sa = _rng(SEED_MX_SA).integers(scale_lo, scale_hi, size=(m, k // 32)).astype(np.uint8)
    sb = _rng(SEED_MX_SB).integers(scale_lo, scale_hi, size=(n, k // 32)).astype(np.uint8)
    return a, b, sa, sb


def topk_inputs(rows, valid_cols, ld, distinct=0):
    """src [rows, ld] fp32: row i holds uniform(i, i + valid_cols) in its first valid_cols columns and zeros after, as
    kernels/manual/a2a3/topk/scripts/gen_data.py:37-41; distinct > 0: only that many different scores (many ties);
    in_idx = 0 .. valid_cols-1."""
    r = _rng(SEED_TOPK)
    src = np.zeros((rows, ld), dtype=np.float32)
    if distinct:
        src[:, :valid_cols] = r.integers(0, distinct, size=(rows, valid_cols)).astype(np.float32) - distinct // 2
    else:
        src[:, :valid_cols] = (r.uniform(0.0, float(valid_cols), size=(rows, valid_cols)) +
                               np.arange(rows, dtype=np.float64)[:, None]).astype(np.float32)
    return src, np.arange(valid_cols, dtype=np.uint32)


def mla_inputs(batch, heads, x_scale=0.02, w_scale=0.02, seed=20251220):
    """q, k, v [batch, heads, 64, 32] and wq, wk, wv [32, 16], wo [16, 32] fp32 for the multi-latent attention demo:
    normal values times a scale (the reference demo uses 0.02 for everything, which makes the softmax almost uniform;
    x_scale 1, w_scale 0.5 gives scores of a few units and a peaked softmax)."""
    rng = np.random.default_rng(seed)
    q, k, v = ((rng.standard_normal((batch, heads, 64, 32)) * x_scale).astype(np.float32) for _ in range(3))
    wq, wk, wv = ((rng.standard_normal((32, 16)) * w_scale).astype(np.float32) for _ in range(3))
    wo = (rng.standard_normal((16, 32)) * w_scale).astype(np.float32)
    return q, k, v, wq, wk, wv, wo


def gather_inputs(table_rows, cols, n_idx):
    """fp16 table of random bit patterns (NaNs included: the gather is a bit copy) and int32 row indices."""
    table = _rng(SEED_GATHER_TABLE).integers(0, 2**16, size=(table_rows, cols), dtype=np.uint16)
    idx = _rng(SEED_GATHER_IDX).integers(0, table_rows, size=n_idx, dtype=np.int32)
    return table, idx
