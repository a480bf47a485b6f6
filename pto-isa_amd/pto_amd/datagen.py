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


def gather_inputs(table_rows, cols, n_idx):
    """fp16 table of random bit patterns (NaNs included: the gather is a bit copy) and int32 row indices."""
    table = _rng(SEED_GATHER_TABLE).integers(0, 2**16, size=(table_rows, cols), dtype=np.uint16)
    idx = _rng(SEED_GATHER_IDX).integers(0, table_rows, size=n_idx, dtype=np.int32)
    return table, idx
