"""Oracle vs the committed outputs of the compiled reference (tests/golden/ref_vectors.npz).
Runs wherever the repository is, with or without the reference tree."""
import os

import numpy as np

from pto_amd import datagen

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_vectors.npz"))


def test_gemm_golden(oracle):
    a, b = datagen.gemm_inputs(128, 128, 512)
    mine = oracle.gemm_f16f32(a, b, base_k=64)
    assert np.max(np.abs(mine - G["gemm_128x512x128_ks64"])) <= 1e-5 * np.max(np.abs(mine))
    a, b = datagen.gemm_inputs(128, 256, 64)
    mine = oracle.gemm_f16f32(a, b, base_k=64)
    assert np.max(np.abs(mine - G["gemm_128x64x256_ks64"])) <= 1e-5 * np.max(np.abs(mine))


def test_tcvt_golden(oracle):
    x = datagen.tcvt_input(64, 256, inject=0.05).reshape(-1)
    assert np.array_equal(oracle.tcvt_f32_f16(x), G["tcvt_f32_f16_64x256"])


def test_gather_golden(oracle):
    rng = np.random.default_rng(9)
    src = rng.integers(0, 2**16, size=(16, 1024), dtype=np.uint16)
    idx = rng.integers(-50, 16 * 1024 + 50, size=(16, 128), dtype=np.int32)
    o = oracle
    got = o.tgather_index(o.make_layout(16, 128), src.reshape(-1), o.make_layout(16, 1024), idx.reshape(-1),
                          o.make_layout(16, 128, elem_bytes=4), 16, 128)
    assert np.array_equal(got.reshape(16, 128), G["tgather_index_f16_16x1024_16x128"])


def test_fa_auto_golden(oracle):
    rng = np.random.default_rng(20251220)
    q, k, v = (rng.standard_normal((64, 32), dtype=np.float32) for _ in range(3))
    assert np.max(np.abs(oracle.fa_auto_f32(q, k, v) - G["fa_auto_64x32"])) < 2e-6


def test_textract_golden(oracle):
    x = np.arange(128 * 256, dtype=np.uint16).reshape(128, 256)
    assert np.array_equal(G["textract_suffix_128x256_0_192"], x[:, 192:])
