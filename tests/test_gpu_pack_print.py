"""TPREFETCH, TPACK and TPRINT on the GPU through the test library's C ABI.  TPACK keeps the low bits of every element
(npu/a5/TPack.hpp:21-72 of the reference); TPRINT writes the reference's text (npu/a2a3/TPrint.hpp:44-190) to the process's
standard output."""
import numpy as np
import pytest
import torch

from pto_amd import capi

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def run(x, do_print):
    lib = capi.load_st()
    tx = torch.from_numpy(x).to(DEV)
    o16 = torch.zeros((16, 64), dtype=torch.int16, device=DEV)
    o8 = torch.zeros((16, 64), dtype=torch.int8, device=DEV)
    capi.check(lib.pto_st_prefetch_pack_print_s32_16x64(torch.cuda.current_stream().cuda_stream, o16.data_ptr(), o8.data_ptr(), tx.data_ptr(),
                                                        int(do_print)), "pack")
    torch.cuda.synchronize()
    return o16.cpu().numpy(), o8.cpu().numpy()


def test_tprefetch_fills_the_tile_and_tpack_keeps_the_low_bits():
    rng = np.random.default_rng(5)
    x = rng.integers(-2**31, 2**31 - 1, size=(16, 64), dtype=np.int64).astype(np.int32)
    o16, o8 = run(x, False)
    assert np.array_equal(o16, x.astype(np.uint32).astype(np.uint16).view(np.int16))       # low 16 bits
    assert np.array_equal(o8, x.astype(np.uint32).astype(np.uint8).view(np.int8))          # low 8 bits of those


def test_tprint_writes_the_tile_and_the_tensor_as_text(capfd):
    x = (np.arange(16 * 64, dtype=np.int32).reshape(16, 64) - 70)
    run(x, True)
    out = capfd.readouterr().out
    lines = [l for l in out.splitlines() if l.strip()]
    start = lines.index("=== [TPRINT Tile] Data Type: int32, Layout: RowMajor, TileType: Vec ===")
    assert lines[start + 1] == "  Shape: [4, 16], Valid Shape: [3, 10]"
    # one line per row of the tile, `|` after the last valid column, a rule after the last valid row
    row0 = lines[start + 2]
    assert row0.startswith(" ".join("%6d" % v for v in x[0, :10]) + "| ") and len(row0.replace("|", "").split()) == 16      # what follows is padding
    assert lines[start + 4].startswith("%6d %6d" % (x[2, 0], x[2, 1]))
    assert set(lines[start + 5].replace("|", "").split()) == {"------"} and lines[start + 5].count("|") == 1
    assert len(lines[start + 6].replace("|", "").split()) == 16       # the row below the valid region: padding
    g = lines.index("=== [TPRINT GlobalTensor] Data Type: int32, Layout: ND ===")
    assert lines[g + 1] == "  Shape: [1, 1, 1, 2, 4]" and lines[g + 2] == "  Batch [0, 0, 0]:"
    assert lines[g + 3] == " ".join("%6d" % v for v in x[0, :4]) and lines[g + 4] == " ".join("%6d" % v for v in x[1, :4])
