"""GPU parity of the multi-latent attention program (the reference's Auto-mode demo, demos/cpu/mla_attention_demo)
through the C ABI: against the float64 oracle, against what the reference's CPU simulation produced for the same
instruction sequence (tests/golden/ref_mla.npz), and by the demo's own acceptance test."""
import os

import numpy as np
import pytest
import torch

from pto_amd import capi, datagen

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden", "ref_mla.npz")
TOL = 1e-5   # max |got - want| / max |want|: fp32 matmul chains and an fp32 softmax against float64


def mla_gpu(q, k, v, wq, wk, wv, wo):
    from gpu_util import to_dev, stream
    lib = capi.load()
    t = [to_dev(x) for x in (q, k, v, wq, wk, wv, wo)]
    out = torch.full(q.shape, float("nan"), dtype=torch.float32, device="cuda:0")
    capi.check(lib.pto_mla_attention_f32_s64_d32_r16(stream(), out.data_ptr(), *[x.data_ptr() for x in t], q.shape[0], q.shape[1]),
               "pto_mla_attention_f32_s64_d32_r16")
    torch.cuda.synchronize()
    return out.cpu().numpy()


def rel(got, want):
    return float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))) / np.max(np.abs(want)))


@pytest.mark.parametrize("case,scales", [("demo_scale", (0.02, 0.02)), ("peaked", (1.0, 0.5))])
def test_mla_vs_oracle_and_reference_outputs(oracle, case, scales):
    args = datagen.mla_inputs(1, 2, *scales)
    got = mla_gpu(*args)
    want = oracle.mla_attention(*args)
    assert rel(got, want) <= TOL
    assert oracle.mla_verify_allclose(got, want) == 0            # the demo's acceptance test (abs 2e-4 + rel 2e-4)
    gold = np.load(GOLD)["mla_" + case]                         # the reference's CPU simulation, fp32
    assert rel(got, gold) <= TOL


def test_mla_many_heads_and_limits(oracle):
    args = datagen.mla_inputs(3, 5, 1.0, 0.5, seed=77)
    got = mla_gpu(*args)
    assert rel(got, oracle.mla_attention(*args)) <= TOL
    # heads are independent: head (1, 2) alone gives the same bits
    q, k, v, wq, wk, wv, wo = args
    one = mla_gpu(q[1:2, 2:3].copy(), k[1:2, 2:3].copy(), v[1:2, 2:3].copy(), wq, wk, wv, wo)
    assert np.array_equal(one[0, 0], got[1, 2])
    # a very peaked softmax (scores of +-100): finite and right
    args = datagen.mla_inputs(1, 2, 3.0, 1.0, seed=3)
    got = mla_gpu(*args)
    assert np.all(np.isfinite(got)) and rel(got, oracle.mla_attention(*args)) <= 1e-4


@pytest.mark.parametrize("S,D", [(64, 32), (128, 64)])
def test_attention_auto_vs_oracle_and_reference_output(oracle, S, D):
    """The whole-tile fp32 attention program against the oracle's restatement of the same instruction sequence
    (rounding-level agreement) and, at the demo's size and seed, against the committed output of the reference's CPU
    simulation."""
    from gpu_util import to_dev, stream
    lib = capi.load()
    rng = np.random.default_rng(20251220)
    q, k, v = (rng.standard_normal((S, D), dtype=np.float32) for _ in range(3))   # the inputs of the committed output
    extra = np.random.default_rng(8)
    qs = np.stack([q] + [extra.standard_normal((S, D), dtype=np.float32) * 2 for _ in range(4)]).reshape(1, 5, S, D)
    ks = np.stack([k] + [extra.standard_normal((S, D), dtype=np.float32) * 2 for _ in range(4)]).reshape(1, 5, S, D)
    vs = np.stack([v] + [extra.standard_normal((S, D), dtype=np.float32) for _ in range(4)]).reshape(1, 5, S, D)
    tq, tk, tv = to_dev(qs), to_dev(ks), to_dev(vs)
    out = torch.full((1, 5, S, D), float("nan"), dtype=torch.float32, device="cuda:0")
    capi.check(lib.pto_attention_auto_f32(stream(), out.data_ptr(), tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), 1, 5, S, D), "attention_auto")
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    for h in range(5):
        want = oracle.fa_auto_f32(qs[0, h], ks[0, h], vs[0, h])
        assert rel(got[0, h], want) <= TOL
    if (S, D) == (64, 32):
        gold = np.load(os.path.join(os.path.dirname(GOLD), "ref_vectors.npz"))["fa_auto_64x32"]
        assert rel(got[0, 0], gold) <= TOL
    assert lib.pto_attention_auto_f32(0, out.data_ptr(), tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), 1, 5, 96, 32) == capi.ERR_UNSUPPORTED


def test_mla_rejects_bad_arguments():
    lib = capi.load()
    p = torch.zeros(64 * 32, device="cuda:0").data_ptr()
    assert lib.pto_mla_attention_f32_s64_d32_r16(0, p, p, p, p, p, p, p, p, 0, 1) == capi.ERR_BAD_ARG
    assert lib.pto_mla_attention_f32_s64_d32_r16(0, p, p, 0, p, p, p, p, p, 1, 1) == capi.ERR_BAD_ARG
