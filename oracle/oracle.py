"""ctypes loader for the CPU oracle (test infrastructure only).

Loads oracle/libpto_oracle.so (the plain-C restatement of the reference's CPU-simulation ops)
and, when it has been built, oracle/_ref/libpto_ref.so (the reference's own headers compiled
behind a C ABI).  Only tests, the smoke check and the benchmark's CPU-baseline leg import this.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libpto_oracle.so")
_REF = os.path.join(_HERE, "_ref", "libpto_ref.so")

BL_ROW, BL_COL = 0, 1
SL_NONE, SL_ROW, SL_COL = 0, 1, 2


class Layout(C.Structure):
    _fields_ = [("rows", C.c_int32), ("cols", C.c_int32), ("blayout", C.c_int32), ("slayout", C.c_int32),
                ("inner_rows", C.c_int32), ("inner_cols", C.c_int32)]


def build(ref=True):
    """Compile the oracle (and the reference shim when the reference tree is present)."""
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    if ref and os.path.isdir(os.environ.get("PTO_REFERENCE", "/root/reference")):
        subprocess.run(["make", "-s", "-C", _HERE, "ref"], check=True)


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            build(ref=False)
        L = C.CDLL(_LIB)
        L.po_make_layout.restype = Layout
        L.po_make_layout.argtypes = [C.c_int] * 6
        L.po_tile_offset.restype = C.c_size_t
        L.po_tile_offset.argtypes = [C.POINTER(Layout), C.c_size_t, C.c_size_t]
        L.po_f32_to_f16_rne.restype = C.c_uint16
        L.po_f32_to_f16_rne.argtypes = [C.c_uint32]
        L.po_f32_to_f16_rna.restype = C.c_uint16
        L.po_f32_to_f16_rna.argtypes = [C.c_uint32]
        L.po_f32_to_bf16_rne.restype = C.c_uint16
        L.po_f32_to_bf16_rne.argtypes = [C.c_uint32]
        L.po_tgather_mask.restype = C.c_size_t
        L.po_online_cpus.restype = C.c_int
        for name in ("po_tcvt_f32_f16", "po_tcvt_f32_bf16", "po_tcvt_f16_f32"):
            getattr(L, name).argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
            getattr(L, name).restype = None
        L.po_tcvt_f32_s32.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        L.po_gather_rows.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int]
        L.po_gather_rows.restype = None
        L.po_gemm_f16f32.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p] + [C.c_int] * 7
        L.po_gemm_f16f32.restype = None
        L.po_topk_f32.argtypes = [C.c_void_p] * 4 + [C.c_int] * 4
        L.po_topk_f32.restype = None
        L.po_mx_gemm.argtypes = [C.c_void_p] * 5 + [C.c_int] * 6
        L.po_mx_gemm.restype = None
        L.po_f32_to_fp8_e4m3fn.argtypes = [C.c_float]
        L.po_f32_to_fp8_e4m3fn.restype = C.c_uint8
        L.po_quant_mxfp8_e4m3.argtypes = [C.c_void_p] * 5 + [C.c_size_t]
        L.po_quant_mxfp8_e4m3.restype = None
        L.po_fp8_e4m3fn_to_f32.argtypes = [C.c_uint8]
        L.po_fp8_e4m3fn_to_f32.restype = C.c_float
        L.po_fp8_e5m2_to_f32.argtypes = [C.c_uint8]
        L.po_fp8_e5m2_to_f32.restype = C.c_float
        L.po_fp4_e2m1_to_f32.argtypes = [C.c_uint8]
        L.po_fp4_e2m1_to_f32.restype = C.c_float
        L.po_fa_auto_f32.argtypes = [C.c_void_p] * 4 + [C.c_int] * 3
        L.po_fa_auto_f32.restype = None
        L.po_fa_stream_f16.argtypes = [C.c_void_p] * 6 + [C.c_int] * 8
        L.po_fa_stream_f16.restype = None
        L.po_result_cmp_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_float, C.POINTER(C.c_double),
                                        C.POINTER(C.c_size_t)]
        L.po_result_cmp_f32.restype = C.c_int
        L.po_vec_op.argtypes = [C.c_void_p] * 4 + [C.c_float] + [C.c_int] * 4
        L.po_vec_op.restype = None
        L.po_reduce.argtypes = [C.c_void_p, C.c_void_p] + [C.c_int] * 4
        L.po_reduce.restype = None
        L.po_tcmps_packed.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int]
        L.po_tcmps_packed.restype = None
        L.po_tsel_packed.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p] + [C.c_int] * 3
        L.po_tsel_packed.restype = None
        L.po_tfillpad.argtypes = [C.c_void_p, C.c_void_p] + [C.c_int] * 6
        L.po_tfillpad.restype = None
        L.po_tmov_relu.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        L.po_tmov_relu.restype = None
        _lib = L
    return _lib


def ref():
    """The compiled reference, or None when oracle/_ref has not been built."""
    if not os.path.exists(_REF):
        return None
    return C.CDLL(_REF)


def online_cpus():
    return lib().po_online_cpus()


# ------------------------------------------------------------------ layouts
def make_layout(rows, cols, blayout=BL_ROW, slayout=SL_NONE, elem_bytes=2, fractal_bytes=512):
    return lib().po_make_layout(rows, cols, blayout, slayout, elem_bytes, fractal_bytes)


def tile_offset(L, r, c):
    return lib().po_tile_offset(C.byref(L), r, c)


def _i64x5(v):
    return (C.c_int64 * 5)(*[int(x) for x in v])


def tload(L, dtype, gm, shape, stride, valid_row=None, valid_col=None, pad=0):
    """Returns the tile's linear storage after TLOAD (or None where the reference asserts)."""
    gm = np.ascontiguousarray(gm)
    tile = np.zeros(L.rows * L.cols, dtype=dtype)
    padv = np.array([pad], dtype=dtype)
    vr = L.rows if valid_row is None else valid_row
    vc = L.cols if valid_col is None else valid_col
    rc = lib().po_tload(_p(tile), C.byref(L), C.c_int(tile.itemsize), _p(gm), _i64x5(shape), _i64x5(stride),
                        C.c_int(vr), C.c_int(vc), _p(padv))
    return tile if rc == 0 else None


def tstore(out, shape, stride, tile, L, valid_row=None, valid_col=None):
    vr = L.rows if valid_row is None else valid_row
    vc = L.cols if valid_col is None else valid_col
    return lib().po_tstore(_p(out), _i64x5(shape), _i64x5(stride), _p(tile), C.byref(L), C.c_int(tile.itemsize),
                           C.c_int(vr), C.c_int(vc))


def textract(Ld, dvr, dvc, src, Ls, svr, svc, idx_row, idx_col, mode=0):
    dst = np.zeros(Ld.rows * Ld.cols, dtype=src.dtype)
    rc = lib().po_textract(_p(dst), C.byref(Ld), C.c_int(dvr), C.c_int(dvc), _p(src), C.byref(Ls), C.c_int(svr),
                           C.c_int(svc), C.c_int(src.itemsize), C.c_int(idx_row), C.c_int(idx_col), C.c_int(mode))
    return dst if rc == 0 else None


def tmov(Ld, src, Ls, valid_row, valid_col):
    dst = np.zeros(Ld.rows * Ld.cols, dtype=src.dtype)
    lib().po_tmov(_p(dst), C.byref(Ld), _p(src), C.byref(Ls), C.c_int(src.itemsize), C.c_int(valid_row),
                  C.c_int(valid_col))
    return dst


def tmatmul(a, La, b, Lb, Lc, M, N, K, acc=None, bias=None, threads=0):
    """a, b are tile storages (uint16 fp16 bits, float32 or int8); returns the Acc tile storage."""
    L = lib()
    if a.dtype == np.uint16:
        dst = np.zeros(Lc.rows * Lc.cols, dtype=np.float32)
        if bias is not None:
            L.po_tmatmul_bias_f16(_p(dst), C.byref(Lc), _p(a), C.byref(La), _p(b), C.byref(Lb), _p(bias), C.c_int(M),
                                  C.c_int(N), C.c_int(K), C.c_int(threads))
            return dst
        fn = L.po_tmatmul_f16
    elif a.dtype == np.float32:
        dst = np.zeros(Lc.rows * Lc.cols, dtype=np.float32)
        fn = L.po_tmatmul_f32
    else:
        dst = np.zeros(Lc.rows * Lc.cols, dtype=np.int32)
        fn = L.po_tmatmul_s8
    fn(_p(dst), _p(acc) if acc is not None else None, C.byref(Lc), _p(a), C.byref(La), _p(b), C.byref(Lb),
       C.c_int(M), C.c_int(N), C.c_int(K), C.c_int(threads))
    return dst


def gemm_f16f32(A, B, base_k=64, row0=0, row1=0, threads=0):
    """A [m,k] fp16, B [n,k] fp16 (column-major k x n) -> C [m,n] fp32 (rows outside [row0,row1) left 0)."""
    A = np.ascontiguousarray(A).view(np.uint16)
    B = np.ascontiguousarray(B).view(np.uint16)
    m, k = A.shape
    n = B.shape[0]
    Cm = np.zeros((m, n), dtype=np.float32)
    lib().po_gemm_f16f32(_p(Cm), _p(A), _p(B), m, n, k, base_k, row0, row1, threads)
    return Cm


def topk_f32(src, in_idx, valid_cols, topk):
    """src [rows, ld] fp32, in_idx [>= valid_cols] uint32 -> (scores [rows, topk] fp32, indices [rows, topk] uint32)."""
    src = np.ascontiguousarray(src, dtype=np.float32)
    in_idx = np.ascontiguousarray(in_idx, dtype=np.uint32)
    rows, ld = src.shape
    out_s = np.empty((rows, topk), dtype=np.float32)
    out_i = np.empty((rows, topk), dtype=np.uint32)
    lib().po_topk_f32(_p(out_s), _p(out_i), _p(src), _p(in_idx), rows, valid_cols, ld, topk)
    return out_s, out_i


def tgatherb(dst, src, offsets, valid_row, valid_col):
    """TGATHERB (cpu/TGatherB.hpp:21-60): block (r, c) of 32 bytes of dst's valid region = the 32 bytes of src's
    row-major storage from byte offsets[r, c]; source ranges that leave the tile are skipped."""
    dst = np.array(dst, copy=True)
    raw = np.ascontiguousarray(src).view(np.uint8).reshape(-1)
    per = 32 // dst.itemsize
    out = dst.view(np.uint8).reshape(dst.shape[0], -1)
    for r in range(valid_row):
        for c in range(valid_col // per):
            off = int(offsets[r, c])
            if off + 32 <= raw.size:
                out[r, 32 * c:32 * c + 32] = raw[off:off + 32]
    return dst


def tscatter(dst, src, idx, valid_row, valid_col):
    """TSCATTER (cpu/TScatter.hpp:21-44): dst[idx[i, j], j] = src[i, j] for i < valid_row, j < valid_col in row order
    (a later row overwrites an earlier one); rows outside dst are dropped (the reference would write out of bounds)."""
    dst = np.array(dst, copy=True)
    for i in range(valid_row):
        rows = idx[i, :valid_col].astype(np.int64)
        ok = (rows >= 0) & (rows < dst.shape[0])
        cols = np.arange(valid_col)[ok]
        dst[rows[ok], cols] = src[i, cols]
    return dst


def mscatter(mem, src, idx, valid_row, valid_col):
    """MSCATTER (cpu/MGatherScatter.hpp:46-69): mem[idx[i, j]] = src[i, j] in row-major order."""
    mem = np.array(mem, copy=True).reshape(-1)
    for i in range(valid_row):
        mem[idx[i, :valid_col]] = src[i, :valid_col]      # numpy assigns in order: the last of equal indices stays
    return mem


def tci(dst, start, descending, valid_col):
    """TCI (cpu/TCI.hpp:16-35): dst[j] = start -/+ j for j < valid_col, in the tile's integer type (wrap-around)."""
    dst = np.array(dst, copy=True).reshape(-1)
    j = np.arange(valid_col, dtype=np.int64)
    dst[:valid_col] = ((np.int64(start) - j) if descending else (np.int64(start) + j)).astype(dst.dtype)
    return dst


def tpart(dst, a, b, op, dvalid, avalid, bvalid):
    """TPARTADD (op 0) / TPARTMAX (1) / TPARTMIN (2), cpu/TPartOp.hpp:19-45: over dst's valid region [dvr, dvc]: op(a, b)
    where both sources are inside their valid regions, the element of the one that is where only one is, 0 where none
    is; the rest of dst is left as it is."""
    dst = np.array(dst, copy=True)
    (dvr, dvc), (avr, avc), (bvr, bvc) = dvalid, avalid, bvalid
    r, c = np.meshgrid(np.arange(dst.shape[0]), np.arange(dst.shape[1]), indexing="ij")
    in_a, in_b, in_d = (r < avr) & (c < avc), (r < bvr) & (c < bvc), (r < dvr) & (c < dvc)
    both = a + b if op == 0 else np.maximum(a, b) if op == 1 else np.minimum(a, b)
    val = np.where(in_a & in_b, both, np.where(in_a, a, np.where(in_b, b, 0))).astype(dst.dtype)
    dst[in_d] = val[in_d]
    return dst


def tsort32(dst, src, idx, valid_row, valid_col, index_as_value=False):
    """TSORT32 (cpu/TSort32.hpp:44-88): in every row, every group of 32 valid columns is put in descending order of
    score, equal scores in ascending order of index (a stable sort, so equal pairs keep their order), and written as
    8-byte structures: (score, index) for 4-byte elements at columns 2 j, 2 j + 1 of dst, (score, 0, index & 0xffff,
    index >> 16) for 2-byte elements at columns 4 j .. 4 j + 3 (the rest of dst is left as it is).
    The index is stored as its bit pattern (the NPU form: tests/npu/a2a3/src/st/testcase/tsort32/gen_data.py:20-27)
    or, index_as_value, exactly as the CPU simulation does it: the index (its two halves for 2-byte elements) converted
    to the element type by value, and every group of a 2-byte tile starting at column 2 j (cpu/TSort32.hpp:49), so
    that groups after the first overwrite the second half of the one before.  Pure Python: single tiles only."""
    dst = np.array(dst, copy=True)
    per = 8 // dst.dtype.itemsize
    for r in range(valid_row):
        for j in range(0, valid_col, 32):
            n = min(32, valid_col - j)
            order = sorted(range(n), key=lambda t: (-_sort_key(src[r, j + t]), int(idx[r, j + t]), t))
            base = 2 * j if index_as_value else per * j
            for m, t in enumerate(order):
                c = base + per * m
                ix = np.array([idx[r, j + t]], dtype=np.uint32)
                dst[r, c] = src[r, j + t]
                if per == 2:
                    dst[r, c + 1:c + 2] = ix.astype(dst.dtype) if index_as_value else ix.view(dst.dtype)
                else:
                    dst[r, c + 1] = 0
                    with np.errstate(over="ignore"):
                        dst[r, c + 2:c + 4] = (np.array([ix[0], ix[0] >> 16]).astype(dst.dtype) if index_as_value
                                               else ix.view(np.uint16).view(dst.dtype))
    return dst


def _sort_key(x):
    return float(x) if isinstance(x, (np.floating, float)) else int(x)


def _merge(lists, out_max, exhausted):
    """The sequential merge of cpu/TMrgSort.hpp:118-178: take the head with the largest score, the lowest list
    number on ties; stop at out_max structures, when everything is taken, or (exhausted) right after the structure
    that empties a list.  lists: arrays [n_i, elements per structure], the score in column 0.  Returns (merged, taken counts)."""
    pos = [0] * len(lists)
    out = []
    while len(out) < out_max:
        pick = -1
        for b, l in enumerate(lists):
            if pos[b] < len(l) and (pick < 0 or l[pos[b], 0] > lists[pick][pos[pick], 0]):
                pick = b
        if pick < 0:
            break
        out.append(lists[pick][pos[pick]])
        pos[pick] += 1
        if exhausted and any(pos[b] == len(l) for b, l in enumerate(lists)):
            break
    dt = lists[0].dtype
    return (np.array(out, dtype=dt).reshape(-1, lists[0].shape[1]), pos)


def tmrgsort_blocks(dst, src, valid_cols, block_len):
    """TMRGSORT with one source (cpu/TMrgSort.hpp:181-230): every complete group of four blocks of block_len
    elements (8-byte structures: 2 elements of 4 bytes, 4 of 2 bytes, :41-46) inside the first valid_cols columns is
    merged; the rest of dst is left as it is."""
    dst = np.array(dst, copy=True).reshape(-1)
    src = np.asarray(src).reshape(-1)
    per = 8 // dst.dtype.itemsize
    if block_len == 0 or block_len % per:
        return dst
    group = 4 * block_len
    for c in range(0, valid_cols - group + 1, group):
        lists = [src[c + b * block_len:c + (b + 1) * block_len].reshape(-1, per) for b in range(4)]
        merged, _ = _merge(lists, 4 * block_len // per, False)
        dst[c:c + group] = merged.reshape(-1)
    return dst


def tmrgsort_lists(dst, lists, cols, out_cols, exhausted):
    """TMRGSORT with two to four lists (cpu/TMrgSort.hpp:232-297): lists[i][:cols[i]] are 8-byte structures (score first)
    in descending order of score; returns (dst with the merged structures in front, executed counts [4])."""
    dst = np.array(dst, copy=True).reshape(-1)
    per = 8 // dst.dtype.itemsize
    ls = [np.asarray(l).reshape(-1)[:c // per * per].reshape(-1, per) for l, c in zip(lists, cols)]
    merged, pos = _merge(ls, out_cols // per, exhausted)
    dst[:merged.size] = merged.reshape(-1)
    return dst, np.array(pos + [0] * (4 - len(pos)), dtype=np.uint32)


def fp8_table(fmt):
    """All 256 values of float8_e4m3fn (fmt 0) or float8_e5m2 (fmt 1), or the 16 of float4_e2m1 (fmt 4), as float32."""
    if fmt == 4:
        return np.array([lib().po_fp4_e2m1_to_f32(v) for v in range(16)], dtype=np.float32)
    f = lib().po_fp8_e5m2_to_f32 if fmt else lib().po_fp8_e4m3fn_to_f32
    return np.array([f(v) for v in range(256)], dtype=np.float32)


def mx_gemm(A, B, SA, SB, fmt_a=0, fmt_b=None, threads=0):
    """A [m,k] uint8 fp8 (or [m,k/2] packed fp4, fmt 4), B [n,k] likewise, SA [m,k/32], SB [n,k/32] uint8 e8m0
    -> C [m,n] fp32 (float64 accumulation)."""
    A, B, SA, SB = (np.ascontiguousarray(x, dtype=np.uint8) for x in (A, B, SA, SB))
    fmt_b = fmt_a if fmt_b is None else fmt_b
    m, k = A.shape[0], A.shape[1] * (2 if fmt_a == 4 else 1)
    n = B.shape[0]
    assert B.shape[1] * (2 if fmt_b == 4 else 1) == k and k % 32 == 0 and SA.shape == (m, k // 32) and SB.shape == (n, k // 32)
    Cm = np.empty((m, n), dtype=np.float32)
    lib().po_mx_gemm(_p(Cm), _p(A), _p(B), _p(SA), _p(SB), m, n, k, fmt_a, fmt_b, threads)
    return Cm


def quant_mxfp8(x, with_stats=False):
    """x [..., cols] fp32, cols a multiple of 32 -> (q uint8 e4m3 bytes of x's shape, e8m0 uint8 [..., cols/32]); with_stats
    adds the per-group absolute maximum and the factor the group was multiplied by."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.shape[-1] % 32 == 0
    q = np.empty(x.shape, dtype=np.uint8)
    gshape = x.shape[:-1] + (x.shape[-1] // 32,)
    e = np.empty(gshape, dtype=np.uint8)
    amax = np.empty(gshape, dtype=np.float32)
    scale = np.empty(gshape, dtype=np.float32)
    lib().po_quant_mxfp8_e4m3(_p(q), _p(e), _p(amax), _p(scale), _p(x), x.size)
    return (q, e, amax, scale) if with_stats else (q, e)


def fp8_e4m3_encode(x):
    """fp32 array -> e4m3fn bytes, nearest even, saturating, element by element (small arrays)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    f = lib().po_f32_to_fp8_e4m3fn
    return np.array([f(float(v)) for v in x.reshape(-1)], dtype=np.uint8).reshape(x.shape)


# --------------------------------------------------------------- conversion
def tcvt_f32_f16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().po_tcvt_f32_f16(_p(out), _p(x), x.size)
    return out


def tcvt_f32_bf16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().po_tcvt_f32_bf16(_p(out), _p(x), x.size)
    return out


def tcvt_f16_f32(h):
    h = np.ascontiguousarray(h).view(np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib().po_tcvt_f16_f32(_p(out), _p(h), h.size)
    return out


def tcvt_f32_s32(x, round_mode):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.int32)
    lib().po_tcvt_f32_s32(_p(out), _p(x), x.size, round_mode)
    return out


# ------------------------------------------------------------------- gather
def tgather_index(Ld, src0, L0, idx, L1, valid_row, valid_col):
    dst = np.zeros(Ld.rows * Ld.cols, dtype=src0.dtype)
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    lib().po_tgather_index(_p(dst), C.byref(Ld), _p(src0), C.byref(L0), _p(idx), C.byref(L1),
                           C.c_int(src0.itemsize), C.c_int(valid_row), C.c_int(valid_col))
    return dst


def tgather_mask(Ld, src, Ls, valid_row, valid_col, pattern):
    dst = np.zeros(Ld.rows * Ld.cols, dtype=src.dtype)
    n = lib().po_tgather_mask(_p(dst), C.byref(Ld), _p(src), C.byref(Ls), C.c_int(src.itemsize), C.c_int(valid_row),
                              C.c_int(valid_col), C.c_int(pattern))
    return dst, n


def mgather(Ld, gm, idx, Li, valid_row, valid_col):
    dst = np.zeros(Ld.rows * Ld.cols, dtype=gm.dtype)
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    lib().po_mgather(_p(dst), C.byref(Ld), _p(gm), _p(idx), C.byref(Li), C.c_int(gm.itemsize), C.c_int(valid_row),
                     C.c_int(valid_col))
    return dst


def gather_rows(table, idx):
    table = np.ascontiguousarray(table)
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    out = np.empty((idx.size, table.shape[1]), dtype=table.dtype)
    lib().po_gather_rows(_p(out), _p(table), _p(idx), idx.size, table.shape[0], table.shape[1], table.itemsize)
    return out


# ---------------------------------------------------------------- attention
def fa_auto_f32(q, k, v, threads=0):
    q, k, v = (np.ascontiguousarray(t, dtype=np.float32) for t in (q, k, v))
    out = np.empty_like(q)
    lib().po_fa_auto_f32(_p(out), _p(q), _p(k), _p(v), q.shape[0], q.shape[1], threads)
    return out


def mla_attention(q, k, v, wq, wk, wv, wo):
    """Multi-latent attention in float64, the reference's check of its Auto-mode demo
    (demos/cpu/mla_attention_demo/mla_attention_demo.cpp:113-225, mla_reference): per (batch, head)
    Q_lat = Q Wq, K_lat = K Wk, V_lat = V Wv ([S,D] x [D,R]), P = softmax(Q_lat K_lat^T / sqrt(R)) over every row,
    out = (P V_lat) Wo.  q, k, v [B,H,S,D]; wq, wk, wv [D,R]; wo [R,D]; returns float32 [B,H,S,D] (the cast of the
    float64 result, as the demo stores it).  numpy only: the sizes are tiny."""
    q, k, v, wq, wk, wv, wo = (np.asarray(t, dtype=np.float64) for t in (q, k, v, wq, wk, wv, wo))
    R = wq.shape[1]
    out = np.empty(q.shape, dtype=np.float32)
    for b in range(q.shape[0]):
        for h in range(q.shape[1]):
            ql, kl, vl = q[b, h] @ wq, k[b, h] @ wk, v[b, h] @ wv
            sc = (ql @ kl.T) * (1.0 / np.sqrt(float(R)))
            e = np.exp(sc - sc.max(axis=1, keepdims=True))
            denom = e.sum(axis=1, keepdims=True)
            p = e * np.where(denom > 0.0, 1.0 / denom, 0.0)
            out[b, h] = ((p @ vl) @ wo).astype(np.float32)
    return out


def mla_verify_allclose(actual, ref, abs_tol=2e-4, rel_tol=2e-4):
    """The demo's acceptance test (mla_attention_demo.cpp:69-111, 45-47): number of elements with
    |a - r| > abs_tol + rel_tol |r| or a non-finite value."""
    a, r = np.asarray(actual, dtype=np.float32).ravel(), np.asarray(ref, dtype=np.float32).ravel()
    finite = np.isfinite(a) & np.isfinite(r)
    bad = ~finite
    bad[finite] = ~(np.abs(a[finite] - r[finite]) <= np.float32(abs_tol) + np.float32(rel_tol) * np.abs(r[finite]))
    return int(bad.sum())


def fa_stream_f16(q, k, v, tile_s1=128, causal=False, q_offset=0, round_away=True, threads=0):
    """One head: q [S0,D], k,v [S1,D] fp16 -> (o fp32 [S0,D], row_max [S0], row_sum [S0])."""
    q, k, v = (np.ascontiguousarray(t).view(np.uint16) for t in (q, k, v))
    S0, D = q.shape
    S1 = k.shape[0]
    o = np.empty((S0, D), dtype=np.float32)
    rmax = np.empty(S0, dtype=np.float32)
    rsum = np.empty(S0, dtype=np.float32)
    lib().po_fa_stream_f16(_p(o), _p(rmax), _p(rsum), _p(q), _p(k), _p(v), S0, S1, D, tile_s1, int(causal),
                           q_offset, int(round_away), threads)
    return o, rmax, rsum


def result_cmp(expect, actual, eps):
    e = np.ascontiguousarray(expect, dtype=np.float32)
    a = np.ascontiguousarray(actual, dtype=np.float32)
    md = C.c_double()
    nb = C.c_size_t()
    ok = lib().po_result_cmp_f32(_p(e), _p(a), e.size, eps, C.byref(md), C.byref(nb))
    return bool(ok), md.value, nb.value


# ------------------------------------------------- further Vec instructions
VOP = dict(ABS=0, NEG=1, RELU=2, SQRT=3, RSQRT=4, LOG=5, RECIP=6, EXP=7,
           ADD=20, SUB=21, MUL=22, DIV=23, MAX=24, MIN=25, PRELU=26, CMP_EQ=27, CMP_NE=28, CMP_LT=29, CMP_LE=30, CMP_GT=31,
           CMP_GE=32, SELS=33, ADDS=40, SUBS=41, MULS=42, DIVS=43, MAXS=44, MINS=45, LRELU=46,
           ROWEXPAND=60, ROWEXPANDSUB=61, ROWEXPANDMUL=62, ROWEXPANDDIV=63, ROWEXPANDADD=64, ROWEXPANDMAX=65, ROWEXPANDMIN=66,
           ROWEXPANDEXPDIF=67, COLEXPAND=80, COLEXPANDSUB=81, COLEXPANDMUL=82, COLEXPANDDIV=83, COLEXPANDADD=84,
           COLEXPANDMAX=85, COLEXPANDMIN=86, COLEXPANDEXPDIF=87)


def vec_op(op, a, b=None, vec=None, scalar=0.0):
    a = np.ascontiguousarray(a, dtype=np.float32)
    rows, cols = a.shape
    out = np.empty_like(a)
    b = None if b is None else np.ascontiguousarray(b, dtype=np.float32)
    vec = None if vec is None else np.ascontiguousarray(vec, dtype=np.float32)
    lib().po_vec_op(_p(out), _p(a), None if b is None else _p(b), None if vec is None else _p(vec), float(scalar),
                    VOP[op] if isinstance(op, str) else int(op), cols, rows, cols)
    return out


def reduce(op, a):
    """op 0 TROWMAX, 1 TROWMIN, 2 TROWSUM, 3 TCOLMAX, 4 TCOLMIN, 5 TCOLSUM over the whole array."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    rows, cols = a.shape
    out = np.empty(rows if op < 3 else cols, dtype=np.float32)
    lib().po_reduce(_p(out), _p(a), cols, rows, cols, op)
    return out


def tcmps_packed(a, scalar, mode):
    a = np.ascontiguousarray(a, dtype=np.float32)
    rows, cols = a.shape
    out = np.zeros((rows, cols // 8), dtype=np.uint8)
    lib().po_tcmps_packed(_p(out), cols // 8, _p(a), cols, rows, cols, float(scalar), mode)
    return out


def tsel_packed(mask, mask_valid_cols, a, b):
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    mask = np.ascontiguousarray(mask, dtype=np.uint8)
    rows, cols = a.shape
    out = np.empty_like(a)
    lib().po_tsel_packed(_p(out), _p(mask), mask.shape[1], mask_valid_cols, _p(a), _p(b), cols, rows, cols)
    return out


def tfillpad(a, vr, vc, pad_kind):
    a = np.ascontiguousarray(a, dtype=np.float32)
    rows, cols = a.shape
    out = np.empty_like(a)
    lib().po_tfillpad(_p(out), _p(a), cols, rows, cols, vr, vc, pad_kind)
    return out


def tmov_relu(x, relu):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().po_tmov_relu(_p(out), _p(x), x.size, int(relu))
    return out
