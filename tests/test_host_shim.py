"""The reference-shaped host boundary: `call_kernel` libraries of the two demos, the GEMM host program with the
reference's file protocol, and its data generator."""
import ctypes as C
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "pto-isa_amd")


def _lib(name):
    path = os.path.join(PKG, name)
    if not os.path.exists(path):
        pytest.fail("%s is not built: run python pto-isa_amd/build.py" % name)
    return C.CDLL(path)


def test_call_kernel_libraries_export_the_entry_point():
    for name in ("libpto_call_gemm.so", "libpto_call_fa.so"):
        assert hasattr(_lib(name), "call_kernel")
    assert os.access(os.path.join(PKG, "host", "gemm_main"), os.X_OK)


def test_gen_data_file_protocol(tmp_path):
    subprocess.run([sys.executable, os.path.join(PKG, "host", "gen_data.py"), str(tmp_path), "128", "64", "256"], check=True)
    a = np.fromfile(tmp_path / "input" / "x1_gm.bin", dtype=np.float16).reshape(128, 64)
    bt = np.fromfile(tmp_path / "input" / "x2_gm.bin", dtype=np.float16).reshape(256, 64)     # stored [n, k]
    g = np.fromfile(tmp_path / "output" / "golden.bin", dtype=np.float32).reshape(128, 256)
    assert np.array_equal(g, a.astype(np.float32) @ bt.astype(np.float32).T)
    assert np.abs(a).max() <= 5 and np.abs(bt).max() <= 5


@pytest.mark.gpu
def test_gemm_main_runs_the_file_protocol(tmp_path):
    subprocess.run([sys.executable, os.path.join(PKG, "host", "gen_data.py"), str(tmp_path), "512", "768", "512"], check=True)
    r = subprocess.run([os.path.join(PKG, "host", "gemm_main"), str(tmp_path), "512", "768", "512"], capture_output=True, text=True, timeout=120)
    assert "test success" in r.stdout, r.stdout + r.stderr
    out = np.fromfile(tmp_path / "output" / "output_z.bin", dtype=np.float32)
    gold = np.fromfile(tmp_path / "output" / "golden.bin", dtype=np.float32)
    assert np.max(np.abs(out - gold) / np.maximum(np.abs(gold), 1.0)) < 2e-3


@pytest.mark.gpu
def test_gemm_main_reports_failure_on_wrong_golden(tmp_path):
    subprocess.run([sys.executable, os.path.join(PKG, "host", "gen_data.py"), str(tmp_path), "256", "256", "256"], check=True)
    g = np.fromfile(tmp_path / "output" / "golden.bin", dtype=np.float32)
    (g + 1000.0).astype(np.float32).tofile(tmp_path / "output" / "golden.bin")
    r = subprocess.run([os.path.join(PKG, "host", "gemm_main"), str(tmp_path), "256", "256", "256"], capture_output=True, text=True, timeout=120)
    assert "test failed" in r.stdout and r.returncode == 1


def test_gen_data_fa_file_protocol(tmp_path):
    """Files and golden of the flash-attention host program: the streamed recipe equals a dense fp64 softmax up to the
    fp16 rounding of the probabilities."""
    subprocess.run([sys.executable, os.path.join(PKG, "host", "gen_data_fa.py"), str(tmp_path), "128", "128", "512"], check=True)
    q = np.fromfile(tmp_path / "q.bin", dtype=np.float16).reshape(128, 128)
    kt = np.fromfile(tmp_path / "kt.bin", dtype=np.float16).reshape(512, 128)                   # stored [s1, head]
    v = np.fromfile(tmp_path / "v.bin", dtype=np.float16).reshape(512, 128)
    o = np.fromfile(tmp_path / "o.bin", dtype=np.float32).reshape(128, 128)
    s = q.astype(np.float64) @ kt.astype(np.float64).T / np.sqrt(128.0)
    p = np.exp(s - s.max(axis=1, keepdims=True))
    want = (p / p.sum(axis=1, keepdims=True)) @ v.astype(np.float64)
    assert np.max(np.abs(o - want)) / np.max(np.abs(want)) < 2e-3
    assert os.access(os.path.join(PKG, "host", "fa_main"), os.X_OK)


@pytest.mark.gpu
@pytest.mark.parametrize("head,s0,s1,causal", [(128, 128, 1024, 0), (128, 512, 512, 1), (64, 256, 768, 0)])
def test_fa_main_runs_the_file_protocol(tmp_path, head, s0, s1, causal):
    subprocess.run([sys.executable, os.path.join(PKG, "host", "gen_data_fa.py"), str(tmp_path), str(head), str(s0), str(s1), str(causal)],
                   check=True)
    r = subprocess.run([os.path.join(PKG, "host", "fa_main"), str(tmp_path), str(head), str(s0), str(s1), str(causal)],
                       capture_output=True, text=True, timeout=120)
    assert "test success" in r.stdout, r.stdout + r.stderr
    out = np.fromfile(tmp_path / "o_out.bin", dtype=np.float32)
    gold = np.fromfile(tmp_path / "o.bin", dtype=np.float32)
    assert np.max(np.abs(out - gold)) / np.max(np.abs(gold)) < 2e-3


@pytest.mark.gpu
def test_fa_main_reports_failure_on_wrong_golden(tmp_path):
    subprocess.run([sys.executable, os.path.join(PKG, "host", "gen_data_fa.py"), str(tmp_path), "128", "128", "256"], check=True)
    g = np.fromfile(tmp_path / "o.bin", dtype=np.float32)
    (g + 10.0).astype(np.float32).tofile(tmp_path / "o.bin")
    r = subprocess.run([os.path.join(PKG, "host", "fa_main"), str(tmp_path), "128", "128", "256"], capture_output=True, text=True, timeout=120)
    assert "test failed" in r.stdout and r.returncode == 1


@pytest.mark.gpu
def test_call_kernel_gemm_6144(oracle):
    import torch
    from pto_amd import datagen
    lib = _lib("libpto_call_gemm.so")
    lib.call_kernel.argtypes = [C.c_uint32] + [C.c_void_p] * 4
    lib.call_kernel.restype = None
    a, b = datagen.gemm_inputs(6144, 6144, 6144)
    ta, tb = torch.from_numpy(a.view(np.int16)).cuda(), torch.from_numpy(b.view(np.int16)).cuda()
    tc = torch.zeros((6144, 6144), dtype=torch.float32, device="cuda")
    lib.call_kernel(24, torch.cuda.current_stream().cuda_stream, tc.data_ptr(), ta.data_ptr(), tb.data_ptr())
    torch.cuda.synchronize()
    rows = [0, 1, 255, 256, 3071, 4097, 6143]
    want = oracle.gemm_f16f32(a, b, base_k=64, row0=0, row1=2)[:2]
    got = tc[:2].cpu().numpy()
    assert np.max(np.abs(got - want)) / np.max(np.abs(want)) < 2e-3
    af, bf = a.view(np.float16).astype(np.float32), b.view(np.float16).astype(np.float32)
    ref = af[rows] @ bf.T
    assert np.max(np.abs(tc[rows].cpu().numpy() - ref)) / np.max(np.abs(ref)) < 2e-3


@pytest.mark.gpu
@pytest.mark.parametrize("causal", [False, True])
def test_call_kernel_flash_attention(causal):
    import torch
    lib = _lib("libpto_call_fa.so")
    lib.call_kernel.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_bool] + [C.c_void_p] * 11
    lib.call_kernel.restype = None
    s0, s1, d = 256, 256 if causal else 512, 128
    rng = np.random.default_rng(7)
    q = (rng.standard_normal((s0, d)) * 1.5).astype(np.float16)
    k = (rng.standard_normal((s1, d)) * 1.2).astype(np.float16)
    v = rng.standard_normal((s1, d)).astype(np.float16)
    tq, tk, tv = (torch.from_numpy(t.view(np.int16)).cuda() for t in (q, k, v))
    o = torch.zeros((s0, d), dtype=torch.float32, device="cuda")
    lib.call_kernel(torch.cuda.current_stream().cuda_stream, d, s0, s1, causal, tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), o.data_ptr(),
                    0, 0, 0, 0, 0, 0, 0)
    torch.cuda.synchronize()
    assert lib.pto_last_status_fa() == 0
    s = q.astype(np.float64) @ k.astype(np.float64).T / np.sqrt(d)
    if causal:
        s = np.where(np.triu(np.ones((s0, s1), dtype=bool), 1), -np.inf, s)
    p = np.exp(s - s.max(axis=1, keepdims=True))
    want = (p / p.sum(axis=1, keepdims=True)) @ v.astype(np.float64)
    assert np.max(np.abs(o.cpu().numpy() - want)) / np.max(np.abs(want)) < 2e-3
    # unsupported head size: nothing is launched and the status says so
    lib.call_kernel(torch.cuda.current_stream().cuda_stream, 64, s0, s1, causal, tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), o.data_ptr(),
                    0, 0, 0, 0, 0, 0, 0)
    assert lib.pto_last_status_fa() != 0


@pytest.mark.gpu
@pytest.mark.parametrize("s0,s1", [(256, 512), (512, 256), (128, 1024)])
def test_call_kernel_flash_attention_causal_rule_of_the_reference(oracle, s0, s1):
    """s1 != s0 with is_causal: key j is visible to query i iff j <= i, with no offset (np.triu(..., 1) in the
    reference's gen_data.py:53; runTFA skips tiles with s1_index > s0_index, fa_performance_kernel.cpp:298-299 and :757).
    Checked against the oracle's streaming recurrence with q_offset = 0 and against a dense float64 softmax."""
    import torch
    lib = _lib("libpto_call_fa.so")
    lib.call_kernel.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_bool] + [C.c_void_p] * 11
    lib.call_kernel.restype = None
    d = 128
    rng = np.random.default_rng(7)
    q = (rng.standard_normal((s0, d)) * 1.5).astype(np.float16)
    k = (rng.standard_normal((s1, d)) * 1.2).astype(np.float16)
    v = rng.standard_normal((s1, d)).astype(np.float16)
    tq, tk, tv = (torch.from_numpy(t.view(np.int16)).cuda() for t in (q, k, v))
    o = torch.full((s0, d), float("nan"), dtype=torch.float32, device="cuda")
    lib.call_kernel(torch.cuda.current_stream().cuda_stream, d, s0, s1, True, tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), o.data_ptr(),
                    0, 0, 0, 0, 0, 0, 0)
    torch.cuda.synchronize()
    assert lib.pto_last_status_fa() == 0
    got = o.cpu().numpy()
    s = q.astype(np.float64) @ k.astype(np.float64).T / np.sqrt(d)
    s = np.where(np.triu(np.ones((s0, s1), dtype=bool), 1), -np.inf, s)
    p = np.exp(s - s.max(axis=1, keepdims=True))
    want = (p / p.sum(axis=1, keepdims=True)) @ v.astype(np.float64)
    assert np.max(np.abs(got - want)) / np.max(np.abs(want)) < 2e-3
    oo, _, _ = oracle.fa_stream_f16(q, k, v, tile_s1=64, causal=True, q_offset=0, round_away=False)
    assert np.max(np.abs(got - oo)) / np.max(np.abs(oo)) < 5e-4


def test_acl_fp16_conversions_match_ieee(tmp_path):
    """aclFloatToFloat16 / aclFloat16ToFloat of the runtime shim (what the reference's flash-attention host program converts
    its fp16 files with): every fp16 pattern to float and back, and float -> fp16 equal to numpy's round-to-nearest-even on
    normals, subnormals, ties, overflow and the specials."""
    src = tmp_path / "cvt.cpp"
    src.write_text("""
#include <acl/acl.h>
#include <cstdio>
#include <vector>
int main(int argc, char **argv)
{
    std::FILE *f = std::fopen(argv[1], "rb");
    std::vector<float> in(1 << 20);
    const size_t n = std::fread(in.data(), sizeof(float), in.size(), f);
    std::fclose(f);
    std::vector<unsigned short> out(n);
    for (size_t i = 0; i < n; ++i)
        out[i] = aclFloatToFloat16(in[i]);
    f = std::fopen(argv[2], "wb");
    std::fwrite(out.data(), 2, n, f);
    std::fclose(f);
    std::vector<float> all(65536);
    for (unsigned h = 0; h < 65536; ++h)
        all[h] = aclFloat16ToFloat((aclFloat16)h);
    f = std::fopen(argv[3], "wb");
    std::fwrite(all.data(), 4, all.size(), f);
    std::fclose(f);
    return 0;
}
""")
    exe = tmp_path / "cvt"
    r = subprocess.run(["g++", "-O2", "-std=c++17", "-I" + os.path.join(ROOT, "include"), "-I/opt/rocm/include", "-D__HIP_PLATFORM_AMD__",
                        str(src), "-o", str(exe), "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    rng = np.random.default_rng(5)
    every = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    finite = every[np.isfinite(every)]
    mids = ((finite[:-1].astype(np.float64) + np.sort(finite)[1:].astype(np.float64)) / 2).astype(np.float32)   # includes exact ties
    x = np.concatenate([rng.normal(size=200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, size=200000).astype(np.float32),
                        every, mids, np.sort(finite)[:-1] + np.float32(0), np.float32([65504, 65519.99, 65520, 1e9, -1e9, 2.0 ** -25,
                                                                                      2.0 ** -25 * 1.0001, 2.0 ** -24, 0.0, -0.0, np.inf, -np.inf])])
    x = x[:1 << 20].astype(np.float32)
    x.tofile(tmp_path / "in.bin")
    subprocess.run([str(exe), str(tmp_path / "in.bin"), str(tmp_path / "out.bin"), str(tmp_path / "all.bin")], check=True)
    got = np.fromfile(tmp_path / "out.bin", dtype=np.uint16)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(got[nan].view(np.float16)))
    back = np.fromfile(tmp_path / "all.bin", dtype=np.float32)
    assert np.array_equal(back.view(np.uint32)[~np.isnan(every)], every.view(np.uint32)[~np.isnan(every)]) and np.all(np.isnan(back[np.isnan(every)]))
