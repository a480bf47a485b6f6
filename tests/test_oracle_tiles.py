"""Pins the oracle's layout / data-movement functions (CPU only).

Checks: closed-form Nz/Zn/Zz offsets against an independent brute-force construction
(box-by-box enumeration of storage order), bijectivity, TLOAD/TSTORE round trips, pad fill,
5-D stacking, TEXTRACT (suffix window as the reference CPU simulation; sub-window per the ISA
definition dst[i,j] = src[r0+i, c0+j]) and, when built, bit-for-bit equality with the tile
images produced by the compiled reference headers (oracle/_ref).
"""
import ctypes as C

import numpy as np
import pytest


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def brute_force_order(rows, cols, ir, ic, outer, inner):
    """Enumerate (r,c) in storage order: boxes in `outer` order ('col' = column of boxes first varies slowest
    is the column index), elements inside a box in `inner` order."""
    order = []
    br_n, bc_n = rows // ir, cols // ic
    boxes = [(br, bc) for bc in range(bc_n) for br in range(br_n)] if outer == "col" else \
            [(br, bc) for br in range(br_n) for bc in range(bc_n)]
    for br, bc in boxes:
        cells = [(r, c) for r in range(ir) for c in range(ic)] if inner == "row" else \
                [(r, c) for c in range(ic) for r in range(ir)]
        for r, c in cells:
            order.append((br * ir + r, bc * ic + c))
    return order


@pytest.mark.parametrize("rows,cols,esz", [(32, 48, 2), (64, 32, 4), (16, 16, 2), (128, 64, 2)])
def test_boxed_offsets_match_brute_force(oracle, rows, cols, esz):
    o = oracle
    cases = [
        (o.BL_COL, o.SL_ROW, "col", "row"),   # Nz: boxes column-major, inside row-major
        (o.BL_ROW, o.SL_COL, "row", "col"),   # Zn
        (o.BL_ROW, o.SL_ROW, "row", "row"),   # Zz
    ]
    for bl, sl, outer, inner in cases:
        L = o.make_layout(rows, cols, bl, sl, esz, 512)
        if sl == o.SL_ROW:
            assert (L.inner_rows, L.inner_cols) == (16, 32 // esz)
        else:
            assert (L.inner_rows, L.inner_cols) == (32 // esz, 16)
        if rows % L.inner_rows or cols % L.inner_cols:
            continue
        order = brute_force_order(rows, cols, L.inner_rows, L.inner_cols, outer, inner)
        offs = [o.tile_offset(L, r, c) for r, c in order]
        assert offs == list(range(rows * cols))


def test_acc_fractal_is_16x16(oracle):
    L = oracle.make_layout(32, 32, oracle.BL_COL, oracle.SL_ROW, 4, 1024)
    assert (L.inner_rows, L.inner_cols) == (16, 16)
    order = brute_force_order(32, 32, 16, 16, "col", "row")
    assert [oracle.tile_offset(L, r, c) for r, c in order] == list(range(1024))


def test_plain_offsets(oracle):
    Lr = oracle.make_layout(8, 16, oracle.BL_ROW, oracle.SL_NONE, 4)
    Lc = oracle.make_layout(8, 16, oracle.BL_COL, oracle.SL_NONE, 4)
    for r in range(8):
        for c in range(16):
            assert oracle.tile_offset(Lr, r, c) == r * 16 + c
            assert oracle.tile_offset(Lc, r, c) == c * 8 + r


def test_tload_tstore_round_trip_all_layouts(oracle):
    o = oracle
    rng = np.random.default_rng(1)
    R, Cc = 32, 64
    x = rng.integers(0, 2**16, size=(R, Cc), dtype=np.uint16)
    sh, st_nd, st_dn = [1, 1, 1, R, Cc], [R * Cc] * 3 + [Cc, 1], [R * Cc] * 3 + [1, R]
    xt = np.ascontiguousarray(x.T)      # column-major storage of the same logical matrix
    for bl, sl in [(o.BL_ROW, o.SL_NONE), (o.BL_COL, o.SL_NONE), (o.BL_COL, o.SL_ROW), (o.BL_ROW, o.SL_COL),
                   (o.BL_ROW, o.SL_ROW)]:
        L = o.make_layout(R, Cc, bl, sl, 2)
        for gm, st in ((x, st_nd), (xt, st_dn)):
            tile = o.tload(L, np.uint16, gm, sh, st)
            assert tile is not None
            # logical content: tile(r,c) == x[r,c]
            for r, c in [(0, 0), (5, 7), (31, 63), (16, 15), (17, 48)]:
                assert tile[o.tile_offset(L, r, c)] == x[r, c]
            assert sorted(tile.tolist()) == sorted(x.reshape(-1).tolist())
            out = np.zeros_like(gm)
            assert o.tstore(out, sh, st, tile, L) == 0
            assert np.array_equal(out, gm)


def test_tload_valid_region_and_pad(oracle):
    o = oracle
    L = o.make_layout(16, 32, o.BL_ROW, o.SL_NONE, 4)
    x = np.arange(200, dtype=np.float32).reshape(10, 20)
    tile = o.tload(L, np.float32, x, [1, 1, 1, 10, 20], [200, 200, 200, 20, 1], 10, 20, pad=np.inf)
    img = tile.reshape(16, 32)
    assert np.array_equal(img[:10, :20], x)
    assert np.all(np.isinf(img[10:, :])) and np.all(np.isinf(img[:, 20:]))
    # shape mismatch is where the reference asserts
    assert o.tload(L, np.float32, x, [1, 1, 1, 10, 20], [200, 200, 200, 20, 1], 9, 20) is None


def test_tload_5d_stacks_outer_dims(oracle):
    o = oracle
    L = o.make_layout(24, 8, o.BL_ROW, o.SL_NONE, 4)
    gm = np.arange(2000, dtype=np.float32)
    shape, stride = [1, 2, 3, 4, 8], [1000, 400, 100, 10, 1]
    tile = o.tload(L, np.float32, gm, shape, stride).reshape(24, 8)
    for j in range(2):
        for k in range(3):
            for r in range(4):
                for c in range(8):
                    assert tile[(j * 3 + k) * 4 + r, c] == gm[j * 400 + k * 100 + r * 10 + c]


def test_textract_subwindow_is_a_slice(oracle):
    o = oracle
    Ls = o.make_layout(128, 256, o.BL_COL, o.SL_ROW, 2)       # Mat A (Nz)
    Ld = o.make_layout(128, 64, o.BL_COL, o.SL_ROW, 2)        # Left
    x = np.arange(128 * 256, dtype=np.uint16).reshape(128, 256)
    src = o.tload(Ls, np.uint16, x, [1, 1, 1, 128, 256], [0, 0, 0, 256, 1])
    for kk in range(4):
        # the reference CPU simulation refuses a window that is not the suffix
        got0 = o.textract(Ld, 128, 64, src, Ls, 128, 256, 0, kk * 64, mode=0)
        assert (got0 is None) == (kk != 3)
        got = o.textract(Ld, 128, 64, src, Ls, 128, 256, 0, kk * 64, mode=1)
        out = np.zeros((128, 64), dtype=np.uint16)
        o.tstore(out, [1, 1, 1, 128, 64], [0, 0, 0, 64, 1], got, Ld)
        assert np.array_equal(out, x[:, kk * 64:(kk + 1) * 64])
    # B operand: Zn 256x256 -> Right 64x256 rows window
    Lb = o.make_layout(256, 256, o.BL_ROW, o.SL_COL, 2)
    Lr = o.make_layout(64, 256, o.BL_ROW, o.SL_COL, 2)
    y = (np.arange(256 * 256) % 65521).astype(np.uint16).reshape(256, 256)
    srcb = o.tload(Lb, np.uint16, y, [1, 1, 1, 256, 256], [0, 0, 0, 256, 1])
    got = o.textract(Lr, 64, 256, srcb, Lb, 256, 256, 128, 0, mode=1)
    out = np.zeros((64, 256), dtype=np.uint16)
    o.tstore(out, [1, 1, 1, 64, 256], [0, 0, 0, 256, 1], got, Lr)
    assert np.array_equal(out, y[128:192])
    # out-of-bounds window rejected
    assert o.textract(Lr, 64, 256, srcb, Lb, 256, 256, 224, 0, mode=1) is None


def test_tmov_changes_layout_only(oracle):
    o = oracle
    La = o.make_layout(32, 32, o.BL_COL, o.SL_ROW, 4, 1024)   # Acc
    Lv = o.make_layout(32, 32, o.BL_ROW, o.SL_NONE, 4)
    x = np.random.default_rng(3).standard_normal((32, 32)).astype(np.float32)
    acc = o.tload(La, np.float32, x, [1, 1, 1, 32, 32], [0, 0, 0, 32, 1])
    vec = o.tmov(Lv, acc, La, 32, 32)
    assert np.array_equal(vec.reshape(32, 32), x)


# ------------------------------------------------------------ against the compiled reference
def test_ref_tile_images(oracle, ref):
    o = oracle
    rng = np.random.default_rng(11)
    x = rng.integers(0, 2**16, size=(32, 48), dtype=np.uint16)
    img = np.zeros(32 * 48, dtype=np.uint16)
    ref.ref_image_nz_f16_32x48(_p(img), _p(x))
    L = o.make_layout(32, 48, o.BL_COL, o.SL_ROW, 2)
    assert np.array_equal(img, o.tload(L, np.uint16, x, [1, 1, 1, 32, 48], [0, 0, 0, 48, 1]))

    y = rng.integers(0, 2**16, size=(32, 48), dtype=np.uint16)   # stored [32][48] = column-major 48x32
    ref.ref_image_zn_f16_48x32(_p(img), _p(y))
    L = o.make_layout(48, 32, o.BL_ROW, o.SL_COL, 2)
    assert np.array_equal(img, o.tload(L, np.uint16, y, [1, 1, 1, 48, 32], [0, 0, 0, 1, 48]))

    z = rng.standard_normal((32, 16)).astype(np.float32)
    imgf = np.zeros(32 * 16, dtype=np.float32)
    ref.ref_image_nz_f32_32x16(_p(imgf), _p(z))
    L = o.make_layout(32, 16, o.BL_COL, o.SL_ROW, 4)
    assert np.array_equal(imgf, o.tload(L, np.float32, z, [1, 1, 1, 32, 16], [0, 0, 0, 16, 1]))


def test_ref_pad_and_5d(oracle, ref):
    o = oracle
    x = np.arange(200, dtype=np.float32)
    img = np.zeros(16 * 32, dtype=np.float32)
    ref.ref_image_pad_f32_16x32_valid_10x20(_p(img), _p(x))
    L = o.make_layout(16, 32, o.BL_ROW, o.SL_NONE, 4)
    mine = o.tload(L, np.float32, x, [1, 1, 1, 10, 20], [200, 200, 200, 20, 1], 10, 20, pad=np.inf)
    assert np.array_equal(img, mine)

    gm = np.arange(2000, dtype=np.float32)
    img = np.zeros(24 * 8, dtype=np.float32)
    ref.ref_image_5d_f32_2x3x4x8(_p(img), _p(gm))
    L = o.make_layout(24, 8, o.BL_ROW, o.SL_NONE, 4)
    assert np.array_equal(img, o.tload(L, np.float32, gm, [1, 2, 3, 4, 8], [1000, 400, 100, 10, 1]))


@pytest.mark.parametrize("fn,R,Cc,r0,c0", [("ref_textract_suffix_64x64_16_32", 64, 64, 16, 32),
                                           ("ref_textract_suffix_128x256_0_192", 128, 256, 0, 192)])
def test_ref_textract_suffix(oracle, ref, fn, R, Cc, r0, c0):
    o = oracle
    x = np.arange(R * Cc, dtype=np.uint16).reshape(R, Cc)   # arange as textract/gen_data.py:30
    out = np.zeros((R - r0, Cc - c0), dtype=np.uint16)
    getattr(ref, fn)(_p(out), _p(x))
    assert np.array_equal(out, x[r0:, c0:])                 # golden gm[idx_row:, idx_col:]
    Ls = o.make_layout(R, Cc, o.BL_COL, o.SL_ROW, 2)
    Ld = o.make_layout(R, Cc, o.BL_COL, o.SL_ROW, 2)
    src = o.tload(Ls, np.uint16, x, [1, 1, 1, R, Cc], [0, 0, 0, Cc, 1])
    got = o.textract(Ld, R - r0, Cc - c0, src, Ls, R, Cc, r0, c0, mode=0)
    mine = np.zeros_like(out)
    Lp = o.make_layout(R, Cc, o.BL_ROW, o.SL_NONE, 2)
    plain = o.tmov(Lp, got, Ld, R - r0, Cc - c0)
    o.tstore(mine, [1, 1, 1, R - r0, Cc - c0], [0, 0, 0, Cc - c0, 1], plain, Lp, R - r0, Cc - c0)
    assert np.array_equal(mine, out)
