"""Helpers shared by the GPU parity tests: device buffers via torch, calls through the C ABI."""
import numpy as np
import torch

from pto_amd import capi

DEV = "cuda:0"


def to_dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16 or a.dtype == np.float16:
        return torch.from_numpy(a.view(np.int16)).to(DEV)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).to(DEV)
    return torch.from_numpy(a).to(DEV)


def stream():
    return torch.cuda.current_stream().cuda_stream


def gemm(a, b):
    """a [m,k] fp16, b [n,k] fp16 (numpy) -> C [m,n] fp32 (numpy) through pto_gemm_f16f32."""
    lib = capi.load()
    m, k = a.shape
    n = b.shape[0]
    ta, tb = to_dev(a), to_dev(b)
    tc = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV)
    capi.check(lib.pto_gemm_f16f32(stream(), tc.data_ptr(), ta.data_ptr(), tb.data_ptr(), m, n, k), "pto_gemm_f16f32")
    torch.cuda.synchronize()
    return tc.cpu().numpy()


def gemm_mx(a, b, sa, sb, fmt, c_fp32=True):
    """a [m,k], b [n,k] fp8 bytes (fmt 0 / 1) or [m,k/2], [n,k/2] packed fp4 (fmt 4), sa [m,k/32], sb [n,k/32] e8m0 bytes
    -> C [m,n] through pto_gemm_mxfp8 / pto_gemm_mxfp4: fp32 values (c_fp32) or the bf16 bit patterns as uint16."""
    lib = capi.load()
    m, k = a.shape[0], a.shape[1] * (2 if fmt == 4 else 1)
    n = b.shape[0]
    ta, tb, tsa, tsb = (to_dev(x) for x in (a, b, sa, sb))
    if c_fp32:
        tc = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV)
    else:
        tc = torch.full((m, n), -1, dtype=torch.int16, device=DEV)
    if fmt == 4:
        capi.check(lib.pto_gemm_mxfp4(stream(), tc.data_ptr(), ta.data_ptr(), tb.data_ptr(), tsa.data_ptr(), tsb.data_ptr(),
                                      m, n, k, int(c_fp32)), "pto_gemm_mxfp4")
    else:
        capi.check(lib.pto_gemm_mxfp8(stream(), tc.data_ptr(), ta.data_ptr(), tb.data_ptr(), tsa.data_ptr(), tsb.data_ptr(),
                                      m, n, k, fmt, int(c_fp32)), "pto_gemm_mxfp8")
    torch.cuda.synchronize()
    out = tc.cpu().numpy()
    return out if c_fp32 else out.view(np.uint16)


def tcvt(x, kind="f16", mode=capi.CAST_RINT):
    lib = capi.load()
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    tx = to_dev(x)
    th = torch.zeros(max(x.size, 1), dtype=torch.int16, device=DEV)
    fn = lib.pto_tcvt_f32_f16 if kind == "f16" else lib.pto_tcvt_f32_bf16
    capi.check(fn(stream(), th.data_ptr(), tx.data_ptr() if x.size else 0, x.size, mode), "pto_tcvt")
    torch.cuda.synchronize()
    return th.cpu().numpy().view(np.uint16)[:x.size]


def gather_rows(table, idx):
    lib = capi.load()
    tt, ti = to_dev(table), to_dev(np.ascontiguousarray(idx, dtype=np.int32))
    es = table.dtype.itemsize
    out = torch.full((idx.size, table.shape[1]), -1, dtype=torch.int16 if es == 2 else torch.int32, device=DEV)
    capi.check(lib.pto_gather_rows(stream(), out.data_ptr(), tt.data_ptr(), ti.data_ptr(), idx.size, table.shape[0],
                                   table.shape[1], es), "pto_gather_rows")
    torch.cuda.synchronize()
    return out.cpu().numpy().view(table.dtype)
