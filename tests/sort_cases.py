"""Seeded inputs for the TSORT32 / TMRGSORT tests (shared by the oracle tests, the GPU tests and tests/golden/make_golden.py)."""
import numpy as np

SORT32_CASES = [("f32", 8, 128, 0), ("f32", 8, 32, 1), ("f32", 5, 77, 2), ("s32", 7, 32, 3), ("s32", 8, 100, 4), ("f32", 1, 5, 5),
                ("f32", 8, 128, 6)]


def sort32_inputs(dtype, vr, vc, seed):
    """src [8,128], idx [8,128] uint32, out0 [8,256] (what the destination holds before).  Scores are quantised so
    that equal scores are frequent, indices repeat, and signed zeros appear."""
    rng = np.random.default_rng(500 + seed)
    if dtype == "f32":
        src = (rng.integers(-12, 13, size=(8, 128)) * 0.25).astype(np.float32)
        if seed == 6:
            src = rng.standard_normal((8, 128)).astype(np.float32)      # distinct scores
        src[0, 3], src[0, 9] = -0.0, 0.0
        out0 = np.full((8, 256), -777.0, dtype=np.float32)
    else:
        src = rng.integers(-6, 7, size=(8, 128)).astype(np.int32)
        src[1, :4] = [2**31 - 1, -2**31, 0, -1]
        out0 = np.full((8, 256), -777, dtype=np.int32)
    idx = rng.integers(0, 40, size=(8, 128)).astype(np.uint32)
    idx[2, :] = np.arange(128, dtype=np.uint32) + 3000000000           # indices above 2^31 (and above 2^24)
    return src, idx, out0


def sorted_list(rng, n, lo=-8, hi=9, tag=0):
    """n (score, index) structures in descending order of score, with ties; the index records list and position."""
    scores = np.sort(rng.integers(lo, hi, size=n).astype(np.float32) * 0.5)[::-1]
    out = np.empty((n, 2), dtype=np.float32)
    out[:, 0] = scores
    out[:, 1] = (np.arange(n, dtype=np.uint32) + np.uint32(1000 * tag)).view(np.float32)
    return out


BLOCK_CASES = [(1024, 64, 0), (1024, 256, 1), (700, 64, 2), (512, 8, 3), (1000, 128, 4), (100, 64, 5)]


def block_inputs(valid_cols, block_len, seed):
    rng = np.random.default_rng(600 + seed)
    src = np.zeros(1024, dtype=np.float32)
    per = block_len // 2
    for b in range(1024 // block_len):
        src[b * block_len:(b + 1) * block_len] = sorted_list(rng, per, tag=b).reshape(-1)
    return src, np.full(1024, -555.0, dtype=np.float32)


# (structures per list, out structures, exhausted, seed)
LIST_CASES = [((128, 128, 128, 128), 512, 0, 0), ((128, 128, 128, 128), 512, 1, 1), ((100, 7, 64, 33), 204, 0, 2),
              ((100, 7, 64, 33), 204, 1, 3), ((128, 90, 50), 268, 0, 4), ((128, 90, 50), 200, 1, 5), ((64, 128), 192, 0, 6),
              ((64, 128), 100, 0, 7), ((64, 128), 192, 1, 8), ((5, 0, 9, 3), 17, 1, 9), ((5, 0, 9, 3), 17, 0, 10),
              ((0, 0), 4, 1, 11), ((128, 128, 128, 128), 40, 1, 12)]


def list_inputs(counts, seed):
    rng = np.random.default_rng(700 + seed)
    lists = []
    for b, n in enumerate(counts):
        l = np.full(256, 123.0, dtype=np.float32)
        l[:2 * n] = sorted_list(rng, n, tag=b).reshape(-1)
        lists.append(l)
    return lists, np.full(1024, -555.0, dtype=np.float32)


# ---- 2-byte elements: four to a structure (score, 0 / payload, index low, index high) ----
NP16 = {"f16": np.float16, "s16": np.int16, "u16": np.uint16}
DT16 = {"f16": 0, "u16": 1, "s16": 2}          # dtype argument of the 16-bit TMRGSORT programs
SORT32_CASES_16 = [("f16", 8, 32, 20), ("f16", 5, 17, 21), ("s16", 8, 32, 22), ("s16", 3, 16, 23), ("f16", 8, 128, 24),
                   ("s16", 7, 100, 25)]


def sort32_inputs_16(dtype, vr, vc, seed):
    """src [8,128] fp16 / int16, idx [8,128] uint32, out0 [8,512]; ties, repeated indices, signed zeros, indices above 2^16."""
    rng = np.random.default_rng(500 + seed)
    if dtype == "f16":
        src = (rng.integers(-12, 13, size=(8, 128)) * 0.25).astype(np.float16)
        src[0, 3], src[0, 9] = -0.0, 0.0
        src[1, :3] = [65504.0, -65504.0, 6.0e-8]
        out0 = np.full((8, 512), -777.0, dtype=np.float16)
    else:
        src = rng.integers(-6, 7, size=(8, 128)).astype(np.int16)
        src[1, :4] = [32767, -32768, 0, -1]
        out0 = np.full((8, 512), -777, dtype=np.int16)
    idx = rng.integers(0, 40, size=(8, 128)).astype(np.uint32)
    idx[2, :] = np.arange(128, dtype=np.uint32) + 3000000000
    idx[3, :] = np.arange(128, dtype=np.uint32) * 1031 + 70000
    return src, idx, out0


def sorted_list_16(rng, n, dtype, tag=0):
    """n structures [score, payload, position, list tag] of 2-byte elements in descending order of score, with ties."""
    np_t = NP16[dtype]
    if dtype == "f16":
        scores = np.sort((rng.integers(-8, 9, size=n) * 0.5).astype(np.float16))[::-1]
    elif dtype == "u16":
        scores = np.sort(rng.integers(0, 12, size=n).astype(np.uint16) * np.uint16(6000))[::-1]      # values above 32767: unsigned order
    else:
        scores = np.sort(rng.integers(-8, 9, size=n).astype(np.int16) * np.int16(4000))[::-1]
    out = np.empty((n, 4), dtype=np.uint16)
    out[:, 0] = scores.view(np.uint16)
    out[:, 1] = 0xA000 + tag
    out[:, 2] = np.arange(n, dtype=np.uint16)
    out[:, 3] = 100 * tag + 7
    return out.view(np_t)


BLOCK_CASES_16 = [("u16", 2048, 256, 30), ("u16", 1024, 64, 31), ("f16", 2048, 512, 32), ("f16", 1400, 128, 33), ("s16", 2048, 16, 34),
                  ("u16", 100, 64, 35), ("f16", 2048, 6, 36)]


def block_inputs_16(dtype, valid_cols, block_len, seed):
    rng = np.random.default_rng(600 + seed)
    src = np.zeros(2048, dtype=NP16[dtype])
    if block_len % 4 == 0:
        for b in range(2048 // block_len):
            src[b * block_len:(b + 1) * block_len] = sorted_list_16(rng, block_len // 4, dtype, tag=b).reshape(-1)
    return src, np.full(2048, 555, dtype=np.uint16).view(NP16[dtype])


# (dtype, structures per list, out structures, exhausted, seed)
LIST_CASES_16 = [("u16", (128, 128, 128, 128), 512, 0, 40), ("u16", (64, 64, 64), 192, 1, 41), ("f16", (100, 7, 64, 33), 204, 1, 42),
                 ("f16", (64, 128), 100, 0, 43), ("f16", (5, 0, 9, 3), 17, 1, 44), ("u16", (128, 90, 50), 268, 0, 45),
                 ("f16", (128, 128, 128, 128), 512, 1, 46)]


def list_inputs_16(dtype, counts, seed):
    rng = np.random.default_rng(700 + seed)
    lists = []
    for b, n in enumerate(counts):
        l = np.full(512, 123, dtype=np.uint16).view(NP16[dtype])
        l[:4 * n] = sorted_list_16(rng, n, dtype, tag=b).reshape(-1)
        lists.append(l)
    return lists, np.full(2048, 555, dtype=np.uint16).view(NP16[dtype])


# TPARTADD / TPARTMAX / TPARTMIN: (op, dst valid, a valid, b valid)
PART_CASES = [(0, (64, 128), (64, 128), (64, 128)), (0, (64, 128), (40, 128), (64, 70)), (1, (50, 100), (64, 60), (30, 128)),
              (2, (64, 128), (10, 20), (64, 128)), (1, (64, 128), (0, 0), (33, 77)), (2, (20, 30), (64, 128), (5, 128)),
              (0, (64, 128), (17, 33), (40, 9))]


def part_inputs(seed):
    rng = np.random.default_rng(800 + seed)
    a = rng.standard_normal((64, 128)).astype(np.float32)
    b = rng.standard_normal((64, 128)).astype(np.float32)
    return a, b, np.full((64, 128), -999.0, dtype=np.float32)


# TSCATTER / MSCATTER / TCI
SCATTER_CASES = [(64, 128, "perm"), (40, 100, "perm"), (64, 128, "collide"), (17, 5, "collide")]


def scatter_inputs(vr, vc, kind, seed):
    """src [64,128] fp32, idx [64,128] int32 (row numbers: a permutation of the rows per column, or random rows so that
    several source rows send an element to the same place), out0 [64,128]."""
    rng = np.random.default_rng(900 + seed)
    src = rng.standard_normal((64, 128)).astype(np.float32)
    if kind == "perm":
        idx = np.stack([rng.permutation(64) for _ in range(128)], axis=1).astype(np.int32)
    else:
        idx = rng.integers(0, 64, size=(64, 128)).astype(np.int32)
    return src, idx, np.full((64, 128), -321.0, dtype=np.float32)


def mscatter_inputs(vr, vc, seed):
    """distinct memory positions in [0, 8192) for every element"""
    rng = np.random.default_rng(950 + seed)
    src = rng.standard_normal((64, 128)).astype(np.float32)
    idx = rng.permutation(8192).astype(np.int32).reshape(64, 128)
    return src, idx, np.full(8192, -321.0, dtype=np.float32)


CI_CASES = [(0, 0, 1024), (1000, 1, 777), (2**31 - 5, 0, 20), (-7, 1, 1)]


GATHERB_CASES = [(16, 128, "aligned"), (16, 128, "any"), (9, 72, "any"), (16, 128, "edge")]


def gatherb_inputs(kind, seed):
    """src [32,64] fp32 (8192 bytes), offsets [16,16] uint32: block starts (multiples of 32), any byte offsets, or
    offsets around the end of the tile (some source ranges leave it)."""
    rng = np.random.default_rng(990 + seed)
    src = rng.standard_normal((32, 64)).astype(np.float32)
    if kind == "aligned":
        off = (rng.integers(0, 256, size=(16, 16)) * 32).astype(np.uint32)
    elif kind == "any":
        off = rng.integers(0, 8192 - 32 + 1, size=(16, 16)).astype(np.uint32)
    else:
        off = rng.integers(8192 - 64, 8192 + 40, size=(16, 16)).astype(np.uint32)
        off[0, :2] = [8192 - 32, 8192 - 31]      # (offsets near 2^32 make the reference's own range check wrap around)
    return src, off, np.full((16, 128), -42.0, dtype=np.float32)
