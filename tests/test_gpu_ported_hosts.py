"""The reference's own host programs (the main.cpp beside each manual kernel), compiled where they lie against this
library's runtime shim (include/acl/acl.h -> HIP, include/pto/host/test_common.h) and linked with the ported kernel library
that holds their launcher (pto-isa_amd/build.py: build_ported_hosts; only where the reference tree is mounted, the programs
travel with the tree).  Each runs its whole flow on the GPU -- aclInit ... aclrtMalloc ... ReadFile ... launch ...
WriteFile ... ResultCmp -- on files in its own layout, the golden files written from the native kernels' results (which
the other tests hold against the oracle)."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOSTS = os.path.join(ROOT, "build", "ported", "host")

pytestmark = pytest.mark.gpu


def _program(name):
    path = os.path.join(HOSTS, name)
    if not os.path.exists(path):
        assert os.environ.get("PTO_REQUIRE_PORTED") != "1", "%s is missing and PTO_REQUIRE_PORTED=1" % path
        pytest.skip("%s not built (reference tree absent at build time)" % name)
    return path


def _dirs(tmp_path):
    for d in ("input", "output", "build"):
        os.makedirs(tmp_path / d, exist_ok=True)
    return tmp_path / "input", tmp_path / "output", tmp_path / "build"


def _run(path, cwd):
    print("host program", os.path.basename(path), flush=True)
    return subprocess.run([path], cwd=str(cwd), capture_output=True, text=True, timeout=300)


def test_reference_gemm_host_program(tmp_path):
    """gemm_performance/main.cpp (GemmE2E: m = n = k = 6144, x1_gm.bin, x2_gm.bin stored [n, k] -> output_z.bin against
    golden.bin at eps 1e-3) with the ported gemm_performance_kernel.cpp behind LaunchGEMME2E<uint16_t>; then with a golden
    file that is wrong, which it has to report."""
    import gpu_util as G
    from pto_amd import datagen
    exe = _program("gemm_performance_main")
    inp, out, cwd = _dirs(tmp_path)
    a, b = datagen.gemm_inputs(6144, 6144, 6144)
    a.tofile(inp / "x1_gm.bin")
    b.tofile(inp / "x2_gm.bin")
    golden = G.gemm(a, b)
    golden.tofile(out / "golden.bin")
    r = _run(exe, cwd)
    assert r.returncode == 0 and "test success" in r.stdout, r.stdout + r.stderr
    got = np.fromfile(out / "output_z.bin", dtype=np.float32).reshape(6144, 6144)
    assert np.abs(got - golden).max() <= 2e-3 * np.abs(golden).max()
    (golden + 1000.0).astype(np.float32).tofile(out / "golden.bin")
    r = _run(exe, cwd)
    assert "test failed" in r.stdout, r.stdout + r.stderr


@pytest.mark.parametrize("name,fmt,m,k,n", [("matmul_mxfp8_performance_main", 1, 6144, 6144, 6144),
                                            ("matmul_mxfp4_performance_main", 4, 2040, 8192, 8100)])
def test_reference_mx_matmul_host_programs(tmp_path, name, fmt, m, k, n):
    """matmul_mxfp8_performance/main.cpp and matmul_mxfp4_performance/main.cpp (operands, x1_scale_gm.bin [m, k/32],
    x2_scale_gm.bin stored [n, k/32], bf16 output_z.bin against golden.bin) with their ported kernels."""
    import gpu_util as G
    from pto_amd import datagen
    exe = _program(name)
    inp, out, cwd = _dirs(tmp_path)
    a, b, sa, sb = datagen.mx_inputs(m, n, k, fmt)
    for arr, f in ((a, "x1_gm.bin"), (b, "x2_gm.bin"), (sa, "x1_scale_gm.bin"), (sb, "x2_scale_gm.bin")):
        arr.tofile(inp / f)
    golden = G.gemm_mx(a, b, sa, sb, fmt, c_fp32=False)
    golden.tofile(out / "golden.bin")
    r = _run(exe, cwd)
    assert r.returncode == 0 and "test success" in r.stdout, r.stdout + r.stderr
    got = np.fromfile(out / "output_z.bin", dtype=np.uint16).reshape(m, n)
    assert np.mean(got == golden) > 0.99


def test_reference_topk_host_program(tmp_path):
    """topk/main.cpp (4800 rows of 1024 scores with row stride 1280, top 1000: x1_gm.bin, x1_idx.bin -> output_z.bin /
    index_z.bin against golden_d.bin / golden_i.bin) with the ported topk_kernel.cpp behind launchTopk<float>."""
    import torch
    import gpu_util as G
    from pto_amd import capi, datagen
    exe = _program("topk_main")
    inp, out, cwd = _dirs(tmp_path)
    rows, cols, ld, k = 4800, 1024, 1280, 1000
    src, idx = datagen.topk_inputs(rows, cols, ld)
    src.tofile(inp / "x1_gm.bin")
    np.arange(ld, dtype=np.uint32).tofile(inp / "x1_idx.bin")
    ts, ti = G.to_dev(src), G.to_dev(idx)
    nat_s = torch.zeros((rows, k), dtype=torch.float32, device=G.DEV)
    nat_i = torch.zeros((rows, k), dtype=torch.int32, device=G.DEV)
    capi.check(capi.load().pto_topk_f32(G.stream(), nat_s.data_ptr(), nat_i.data_ptr(), ts.data_ptr(), ti.data_ptr(), rows, cols, ld, k), "topk")
    torch.cuda.synchronize()
    nat_s.cpu().numpy().tofile(out / "golden_d.bin")
    nat_i.cpu().numpy().tofile(out / "golden_i.bin")
    r = _run(exe, cwd)
    assert r.returncode == 0 and "All tests passed!" in r.stdout, r.stdout + r.stderr
    assert np.array_equal(np.fromfile(out / "index_z.bin", dtype=np.int32), nat_i.cpu().numpy().reshape(-1))


@pytest.mark.parametrize("head,s0,s1,causal,tile_s1", [(128, 128, 1024, False, 256), (128, 256, 1024, True, 128)])
def test_reference_flash_attention_host_program(tmp_path, head, s0, s1, causal, tile_s1):
    """flash_atten/main.cpp (run_tfa: the workspace of FIFOs, per-tile sums and maxima, profile and communication buffers
    that it allocates for LaunchTFA; q.bin, kt.bin, v.bin of the case's directory -> o_out.bin against o.bin at eps 1e-3,
    besides the intermediate dumps it always writes) with the ported fa_performance_kernel.cpp, on files written with the
    reference generator's recipe."""
    import sys
    exe = _program("flash_atten_main")
    case = "case_float_H_%d_S0_%d_S1_%d" % (head, s0, s1)
    subprocess.run([sys.executable, os.path.join(ROOT, "pto-isa_amd", "host", "gen_data_fa.py"), str(tmp_path / case), str(head),
                    str(s0), str(s1), str(int(causal)), str(tile_s1)], check=True)
    print("host program flash_atten_main", case, flush=True)
    r = subprocess.run([exe, "--case=" + case], cwd=str(tmp_path), capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "test success" in r.stdout and "test failed" not in r.stdout, r.stdout[-3000:] + r.stderr[-2000:]
    got = np.fromfile(tmp_path / case / "o_out.bin", dtype=np.float32)
    want = np.fromfile(tmp_path / case / "o.bin", dtype=np.float32)
    assert np.abs(got - want).max() <= 2e-3 * np.abs(want).max()
