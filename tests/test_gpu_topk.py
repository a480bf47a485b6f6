"""GPU parity of the row-wise top-k (kernels/manual/a2a3/topk) through the C ABI: bit-exact scores and indices against
the oracle (the TSORT32 / TMRGSORT comparator applied to the whole row)."""
import numpy as np
import pytest
import torch

from pto_amd import capi, datagen

pytestmark = pytest.mark.gpu


def topk_gpu(src, in_idx, valid_cols, topk):
    from gpu_util import to_dev, stream
    lib = capi.load()
    rows, ld = src.shape
    ts, ti = to_dev(src), to_dev(np.ascontiguousarray(in_idx, dtype=np.uint32))
    os_ = torch.full((rows, topk), float("nan"), dtype=torch.float32, device="cuda:0")
    oi = torch.full((rows, topk), -1, dtype=torch.int32, device="cuda:0")
    capi.check(lib.pto_topk_f32(stream(), os_.data_ptr(), oi.data_ptr(), ts.data_ptr(), ti.data_ptr(), rows, valid_cols, ld, topk),
               "pto_topk_f32")
    torch.cuda.synchronize()
    return os_.cpu().numpy(), oi.cpu().numpy().view(np.uint32)


def same(got, want):
    return np.array_equal(got[0].view(np.uint32), want[0].view(np.uint32)) and np.array_equal(got[1], want[1])


@pytest.mark.parametrize("rows,valid_cols,ld,topk", [(7, 256, 256, 256), (5, 1000, 1024, 37), (3, 1024, 1280, 1000), (4, 777, 800, 777),
                                                     (2, 33, 64, 5), (3, 2048, 2048, 100), (2, 4096, 4096, 4096), (9, 1, 8, 1)])
def test_topk_small_vs_oracle(oracle, rows, valid_cols, ld, topk):
    src, idx = datagen.topk_inputs(rows, valid_cols, ld)
    assert same(topk_gpu(src, idx, valid_cols, topk), oracle.topk_f32(src, idx, valid_cols, topk))


def test_topk_ties_signed_zeros_infinities_and_arbitrary_indices(oracle):
    rows, cols = 6, 1024
    src, _ = datagen.topk_inputs(rows, cols, cols, distinct=7)           # many equal scores: the index decides
    src[0, ::5] = -0.0
    src[1, ::3] = np.inf
    src[2, 1::4] = -np.inf
    src[3] = 0.0
    src[3, ::2] = -0.0                                                   # -0 == +0: pure index order, bit patterns kept
    src[4] = 3.0
    r = np.random.Generator(np.random.Philox(key=11))
    idx = r.permutation(1 << 20)[:cols].astype(np.uint32)                # not monotonic: ties follow the index, not the column
    idx[0] = 0xFFFFFFFF
    for k in (1, 100, cols):
        assert same(topk_gpu(src, idx, cols, k), oracle.topk_f32(src, idx, cols, k))
    # indices that increase with the column (the register-resident network; the rows above went through LDS)
    for mono in (np.arange(cols, dtype=np.uint32), (np.arange(cols, dtype=np.uint32) * 3 + 7) ** 2):
        for k in (1, 100, cols):
            assert same(topk_gpu(src, mono, cols, k), oracle.topk_f32(src, mono, cols, k))
    # and with other row lengths (1, 2, 8 keys per thread; padded rows)
    for c in (200, 512, 1900):
        s2, _ = datagen.topk_inputs(4, c, c + 8, distinct=5)
        s2[1, ::9] = -0.0
        for mono in (np.arange(c, dtype=np.uint32), r.permutation(1 << 16)[:c].astype(np.uint32)):
            assert same(topk_gpu(s2, mono, c, c), oracle.topk_f32(s2, mono, c, c))


def test_topk_reference_config_4800x1024_top1000(oracle):
    """The reference kernel's case: 4800 rows of 1024 valid columns (row stride 1280), top 1000, its generator's data."""
    rows, cols, ld, k = 4800, 1024, 1280, 1000
    src, idx = datagen.topk_inputs(rows, cols, ld)
    got = topk_gpu(src, idx, cols, k)
    assert same(got, oracle.topk_f32(src, idx, cols, k))
    # properties that hold whatever the implementation: sorted, indices distinct and in range, scores = src at the indices
    s, i = got
    assert np.all(s[:, :-1] >= s[:, 1:]) and int(i.max()) < cols
    assert np.array_equal(np.take_along_axis(src[:, :cols], i.astype(np.int64), axis=1), s)
    assert all(np.unique(i[r]).size == k for r in (0, 2399, 4799))


def test_topk_rejects_bad_arguments():
    lib = capi.load()
    t = torch.zeros(16, device="cuda:0")
    p = t.data_ptr()
    assert lib.pto_topk_f32(0, p, p, p, p, 4, 8192, 8192, 4) == capi.ERR_UNSUPPORTED     # more than 4096 columns
    assert lib.pto_topk_f32(0, p, p, p, p, 4, 100, 64, 4) == capi.ERR_UNSUPPORTED        # row stride below the valid columns
    assert lib.pto_topk_f32(0, p, p, p, p, 4, 100, 128, 101) == capi.ERR_UNSUPPORTED     # k above the valid columns
    assert lib.pto_topk_f32(0, p, 0, p, p, 4, 100, 128, 10) == capi.ERR_BAD_ARG
    assert lib.pto_topk_f32(0, p, p, p, p, 0, 100, 128, 10) == capi.ERR_BAD_ARG
