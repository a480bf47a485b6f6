#!/usr/bin/env python3
"""Benchmark of the PTO tile compute path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only gemm|mx|fa|tcvt|quant|gather|topk]

A step is one pass of the hot path over one batch of synthetic input, resident in HBM before the
timed region: one fp16 -> fp32 GEMM at m=n=k=6144 (the configuration the headline metric is quoted
on).  The other workloads of the metric (flash-attention forward, TCVT, gather) and the MXFP8 GEMM are timed the same
way and reported under "extra".  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "pto-isa_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_FP16_TFLOPS = 2516.6   # MI355X dense fp16 matrix peak (published)
PEAK_FP8_TFLOPS = 5033.2    # dense fp8 matrix peak (published)
PEAK_FP4_TFLOPS = 10066.3   # dense fp4 matrix peak (published)
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E peak (published)
# row gather, 65536 x 1024 fp16 from a 32 MiB table: bytes per launch at the L2 <-> fabric boundary (FETCH_SIZE + WRITE_SIZE
# runs summarised in profiles/cvt_f32_16384x8192_and_gather_rows_65536x1024.md)
GATHER_HBM_SIDE_BYTES = 85.0e6 + 134.3e6

# HBM-side traffic of one 6144^3 GEMM launch, from two rocprofv3 --pmc runs of this script
# (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch of the GEMM kernel), each scaled by what the same
# counter reads for a plain 1 GiB device copy in the same run (--calib-copy): FETCH_SIZE reads
# 524,300 KiB for 1,048,576 KiB actually read (factor 2.0), WRITE_SIZE reads 1,048,576 KiB for
# 1,048,576 KiB written (factor 1.0).
GEMM_6144_FETCH_KIB, GEMM_6144_FETCH_SCALE = 369274.0, 2.0
GEMM_6144_WRITE_KIB, GEMM_6144_WRITE_SCALE = 147458.0, 1.0


SETTLE_S = 0.0   # set from --settle-ms: the workloads under "extra" keep warming up until this much time has passed


GEMM_KERNEL_NOTE = {6144: "GemmF16F32W4<192,4> (256x192 C tile per workgroup of four wavefronts, K-steps of 64; "
                          "768 tiles = three whole rounds on 256 compute units)"}


def time_launches(torch, fn, steps, warmup, settle_s=None):
    """Average duration in ms of fn() over `steps` launches on torch's current stream (HIP events), after `warmup`
    untimed launches and, where settle_s is set, further untimed launches until that much wall time has passed (a
    launch of 0.1 ms repeated 30 times does not bring the GPU out of its idle clocks)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    settle_s = SETTLE_S if settle_s is None else settle_s
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < settle_s:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def prepare_gemm(torch, lib, capi, datagen, size):
    """Operands of one size^3 problem resident in HBM, and the function that launches it."""
    import numpy as np
    a, b = datagen.gemm_inputs(size, size, size)
    ta = torch.from_numpy(a.view(np.int16)).cuda()
    tb = torch.from_numpy(b.view(np.int16)).cuda()
    tc = torch.empty((size, size), dtype=torch.float32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream

    def step():
        capi.check(lib.pto_gemm_f16f32(st, tc.data_ptr(), ta.data_ptr(), tb.data_ptr(), size, size, size), "gemm")
    step.keep = (ta, tb, tc)
    return step


def bench_gemm(torch, lib, capi, datagen, size, steps, warmup, settle_s=None, step=None):
    step = step or prepare_gemm(torch, lib, capi, datagen, size)
    ms = time_launches(torch, step, steps, warmup, settle_s)
    flops = 2.0 * size ** 3
    return {"ms": ms, "tflops": flops / (ms * 1e-3) / 1e12, "flops": flops}


def bench_gemm_mx(torch, lib, capi, datagen, m, n, k, fmt, steps, warmup):
    """MX GEMMs of the reference's matmul_mxfp8_performance (fmt 1: e5m2) and matmul_mxfp4_performance (fmt 4: e2m1)
    cases: e8m0 block scales, bf16 result."""
    a, b, sa, sb = datagen.mx_inputs(m, n, k, fmt)
    ta, tb, tsa, tsb = (torch.from_numpy(x).cuda() for x in (a, b, sa, sb))
    tc = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream

    def step():
        if fmt == 4:
            capi.check(lib.pto_gemm_mxfp4(st, tc.data_ptr(), ta.data_ptr(), tb.data_ptr(), tsa.data_ptr(), tsb.data_ptr(),
                                          m, n, k, 0), "gemm_mxfp4")
        else:
            capi.check(lib.pto_gemm_mxfp8(st, tc.data_ptr(), ta.data_ptr(), tb.data_ptr(), tsa.data_ptr(), tsb.data_ptr(),
                                          m, n, k, fmt, 0), "gemm_mxfp8")
    ms = time_launches(torch, step, steps, warmup)
    flops = 2.0 * m * n * k
    return {"ms": ms, "tflops": flops / (ms * 1e-3) / 1e12, "flops": flops}


def bench_topk(torch, lib, capi, datagen, steps, warmup):
    """Row-wise top-k of the reference's topk kernel: 4800 rows of 1024 scores (row stride 1280), top 1000."""
    import numpy as np
    rows, cols, ld, k = 4800, 1024, 1280, 1000
    src, idx = datagen.topk_inputs(rows, cols, ld)
    ts, ti = torch.from_numpy(src).cuda(), torch.from_numpy(idx.view(np.int32)).cuda()
    out_s = torch.empty((rows, k), dtype=torch.float32, device="cuda")
    out_i = torch.empty((rows, k), dtype=torch.int32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream

    def step():
        capi.check(lib.pto_topk_f32(st, out_s.data_ptr(), out_i.data_ptr(), ts.data_ptr(), ti.data_ptr(), rows, cols, ld, k), "topk")
    ms = time_launches(torch, step, steps, warmup)
    nbytes = rows * cols * 4 + rows * k * 8      # scores read once, scores + indices written
    return {"ms": ms, "gbs": nbytes / (ms * 1e-3) / 1e9, "rows_per_s": rows / (ms * 1e-3)}


def bench_fa(torch, lib, capi, datagen, cfg, steps, warmup):
    import numpy as np
    B, H, S, D, causal = cfg
    scale = 1.0 / np.sqrt(D) if not causal else 1.0
    q, k, v = datagen.fa_inputs(B, H, S, S, D, scale=scale)
    tq, tk, tv = (torch.from_numpy(t.view(np.int16)).cuda() for t in (q, k, v))
    to = torch.empty((B, H, S, D), dtype=torch.int16, device="cuda")
    tl = torch.empty((B, H, S), dtype=torch.float32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream

    def step():
        capi.check(lib.pto_fa_fwd_f16(st, to.data_ptr(), tl.data_ptr(), tq.data_ptr(), tk.data_ptr(), tv.data_ptr(),
                                      B, H, S, S, D, int(causal), 0), "fa")
    ms = time_launches(torch, step, steps, warmup)
    flops = 4.0 * B * H * S * S * D      # the reference's convention (flash_atten/main.cpp:650)
    if causal:
        flops *= 0.5                     # causal counted as half
    return {"ms": ms, "tflops": flops / (ms * 1e-3) / 1e12, "flops": flops,
            "flop_convention": "4*B*H*Sq*Sk*D" + (" / 2 (causal)" if causal else "")}


def bench_tcvt(torch, lib, capi, datagen, steps, warmup, kind):
    rows, cols = 16384, 8192
    n = rows * cols
    # the configuration's data: N(0, 100) with 0.1 % of the positions overwritten by +-inf, NaNs, fp32 denormals, values
    # around the fp16 overflow threshold and rounding ties (the generator the parity tests use); two buffer sets,
    # alternated, so that no launch finds its input in cache
    x0 = torch.from_numpy(datagen.tcvt_input(rows, cols)).reshape(-1).cuda()
    xs = [x0, x0.flip(0).contiguous()]
    outs = [torch.empty(n, dtype=torch.int16, device="cuda") for _ in range(2)]
    fn = lib.pto_tcvt_f32_f16 if kind == "f16" else lib.pto_tcvt_f32_bf16
    st = torch.cuda.current_stream().cuda_stream
    i = [0]

    def step():
        j = i[0] & 1
        i[0] += 1
        capi.check(fn(st, outs[j].data_ptr(), xs[j].data_ptr(), n, capi.CAST_RINT), "tcvt")
    ms = time_launches(torch, step, steps, warmup)
    nbytes = n * 6.0
    return {"ms": ms, "gbs": nbytes / (ms * 1e-3) / 1e9, "bytes": nbytes}


def bench_quant(torch, lib, capi, datagen, steps, warmup):
    """MXFP8 quantisation (the a5 TQUANT) of a 16384 x 8192 fp32 matrix: 4 bytes read, 1 + 1/32 written per element; two
    buffer sets, alternated, so that no launch finds its input in cache."""
    rows, cols = 16384, 8192
    n = rows * cols
    x0 = torch.from_numpy(datagen.quant_input(rows, cols, specials=True)).cuda()
    xs = [x0, x0.flip(0).contiguous()]
    qs = [torch.empty((rows, cols), dtype=torch.uint8, device="cuda") for _ in range(2)]
    ss = [torch.empty((rows, cols // 32), dtype=torch.uint8, device="cuda") for _ in range(2)]
    st = torch.cuda.current_stream().cuda_stream
    i = [0]

    def step():
        j = i[0] & 1
        i[0] += 1
        capi.check(lib.pto_quant_mxfp8_f32(st, qs[j].data_ptr(), ss[j].data_ptr(), xs[j].data_ptr(), rows, cols), "quant")
    ms = time_launches(torch, step, steps, warmup)
    nbytes = n * (4.0 + 1.0 + 1.0 / 32)
    return {"ms": ms, "gbs": nbytes / (ms * 1e-3) / 1e9, "bytes": nbytes}


def bench_gather(torch, lib, capi, datagen, steps, warmup):
    import numpy as np
    table, idx = datagen.gather_inputs(16384, 1024, 65536)
    tt = torch.from_numpy(table.view(np.int16)).cuda()
    ti = torch.from_numpy(idx).cuda()
    outs = [torch.empty((65536, 1024), dtype=torch.int16, device="cuda") for _ in range(2)]
    st = torch.cuda.current_stream().cuda_stream
    i = [0]

    def step():
        j = i[0] & 1
        i[0] += 1
        capi.check(lib.pto_gather_rows(st, outs[j].data_ptr(), tt.data_ptr(), ti.data_ptr(), 65536, 16384, 1024, 2), "gather")
    ms = time_launches(torch, step, steps, warmup)
    nbytes = 65536 * 1024 * 2 * 2 + 65536 * 4.0
    return {"ms": ms, "gbs": nbytes / (ms * 1e-3) / 1e9, "bytes": nbytes}


def cpu_baseline(datagen, size):
    """The reference CPU-simulation arithmetic timed on the host cores, on a bounded sample of the
    6144^3 product (all of it: 5-15 s on 16 cores) through the oracle's port of the tile path
    (TLOAD/TEXTRACT/TMATMUL[_ACC] per K-step of 64), threads over rows as the reference does."""
    from oracle import oracle
    a, b = datagen.gemm_inputs(size, size, size)
    rows = size
    cores = oracle.online_cpus()
    cores = min(cores, 16) if os.environ.get("OMP_NUM_THREADS") is None else min(cores, int(os.environ["OMP_NUM_THREADS"]))
    t0 = time.perf_counter()
    oracle.gemm_f16f32(a, b, base_k=64, row0=0, row1=rows, threads=cores)
    dt = time.perf_counter() - t0
    flops = 2.0 * rows * size * size
    out = {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
           "sample": "the whole m=n=k=%d product (rows 0..%d of C), %.1f s" % (size, rows - 1, dt)}
    ref = oracle.ref()
    if ref is not None:
        import ctypes as C
        import numpy as np
        a1, b1 = datagen.gemm_inputs(1536, 1536, 1536)
        c1 = np.zeros((1536, 1536), dtype=np.float32)
        t0 = time.perf_counter()
        ref.ref_gemm_1536x1536x1536_ks1536(c1.ctypes.data_as(C.c_void_p), a1.ctypes.data_as(C.c_void_p),
                                           b1.ctypes.data_as(C.c_void_p))
        dt1 = time.perf_counter() - t0
        out["reference_1536_single_tile"] = {"seconds": dt1, "tflops": 2.0 * 1536 ** 3 / dt1 / 1e12,
                                             "what": "compiled reference CPU-simulation headers, one TMATMUL 1536^3"}
    return out


def cpu_baselines_extra(datagen, cores):
    """The oracle timed on bounded samples of the other workloads (reported beside the GPU figures, nothing more):
    attention = the first 2048 query rows of one head of each configuration; TCVT = 2^24 elements; gather = 8192 rows;
    top-k = 480 rows; MX GEMMs = a 64 x 2048 x 6144 block."""
    import numpy as np
    from oracle import oracle
    out = {}
    for name, (B, H, S, D, causal) in (("fa_b1_h16_s4096_d128", (1, 16, 4096, 128, False)),
                                       ("fa_causal_b4_h32_s2048_d64", (4, 32, 2048, 64, True))):
        q, k, v = datagen.fa_inputs(1, 1, S, S, D, scale=1.0 / np.sqrt(D) if not causal else 1.0)
        rows = min(S, 2048)
        keys = S if not causal else rows             # causal: the first `rows` queries see the first `rows` keys
        t0 = time.perf_counter()
        oracle.fa_stream_f16(q[0, 0, :rows], k[0, 0, :keys], v[0, 0, :keys], tile_s1=128, causal=causal, threads=cores)
        dt = time.perf_counter() - t0
        flops = 4.0 * rows * keys * D * (0.5 if causal else 1.0)
        out[name] = {"tflops": flops / dt / 1e12, "cores": cores, "kind": "port", "sample": "%d query rows x %d keys of one head, %.2f s" % (rows, keys, dt)}
    x = datagen.tcvt_input(2048, 8192, inject=0.001).reshape(-1)
    t0 = time.perf_counter()
    oracle.tcvt_f32_f16(x)
    dt = time.perf_counter() - t0
    out["tcvt_f32_f16"] = {"gbs": x.size * 6.0 / dt / 1e9, "cores": 1, "kind": "port", "sample": "%d elements, %.2f s" % (x.size, dt)}
    xq = datagen.quant_input(2048, 8192)
    t0 = time.perf_counter()
    oracle.quant_mxfp8(xq)
    dt = time.perf_counter() - t0
    out["quant_mxfp8_f32"] = {"gbs": xq.size * (5.0 + 1.0 / 32) / dt / 1e9, "cores": 1, "kind": "port", "sample": "%d elements, %.2f s" % (xq.size, dt)}
    table, idx = datagen.gather_inputs(16384, 1024, 8192)
    t0 = time.perf_counter()
    oracle.gather_rows(table, idx)
    dt = time.perf_counter() - t0
    out["gather_rows"] = {"gbs": (8192 * 1024 * 2 * 2 + 8192 * 4.0) / dt / 1e9, "cores": 1, "kind": "port", "sample": "8192 rows of 1024 fp16, %.3f s" % dt}
    src, tidx = datagen.topk_inputs(480, 1024, 1280)
    t0 = time.perf_counter()
    oracle.topk_f32(src, tidx, 1024, 1000)
    dt = time.perf_counter() - t0
    out["topk_1024_top1000"] = {"rows_per_s": 480 / dt, "cores": 1, "kind": "port", "sample": "480 rows, %.3f s" % dt}
    for name, fmt in (("gemm_mxfp8_e5m2", 1), ("gemm_mxfp4_e2m1", 4)):
        a, b, sa, sb = datagen.mx_inputs(64, 2048, 6144, fmt)
        t0 = time.perf_counter()
        oracle.mx_gemm(a, b, sa, sb, fmt, threads=cores)
        dt = time.perf_counter() - t0
        out[name] = {"tflops": 2.0 * 64 * 2048 * 6144 / dt / 1e12, "cores": cores, "kind": "port",
                     "sample": "64 x 2048 x 6144 (float64 accumulation), %.2f s" % dt}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--settle-ms", type=float, default=300.0,
                    help="workloads under \"extra\": after the warm-up launches keep launching untimed until this much time has passed")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="gemm | mx | fa | tcvt | quant | gather | topk: time just that workload")
    ap.add_argument("--size", type=int, default=6144)
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run a plain 1 GiB device copy a few times (reference point for FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus %d is not supported (every workload of the metric "
                 "fits one MI355X, and nothing here uses a second device)" % args.gpus)

    import torch
    from pto_amd import capi, datagen
    global SETTLE_S
    SETTLE_S = max(args.settle_ms, 0.0) * 1e-3
    lib = capi.load()
    capi.check(lib.pto_init(), "pto_init")
    torch.cuda.set_device(0)

    extra = {}
    if args.calib_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        ms = time_launches(torch, lambda: dst.copy_(src), 5, 2, settle_s=0.0)
        extra["calib_copy_1GiB"] = {"ms": ms, "gbs": 2.0 * src.numel() * 4 / (ms * 1e-3) / 1e9, "bytes_read": src.numel() * 4,
                                    "bytes_written": src.numel() * 4}
    only = args.only
    gemm = None
    # The headline's operands go to HBM first; its W warm-up and K timed launches come LAST, straight after a settled run
    # of the same kernel, so that they start on a GPU that is already at its working clocks whatever W is (a few
    # launches of 0.4 ms after an idle stretch run at the idle clocks: the same kernel reads 17 % lower then).
    gemm_step = prepare_gemm(torch, lib, capi, datagen, args.size) if only in ("", "gemm") else None
    if gemm_step is not None:
        # the same W warm-up and K timed launches on a GPU that has run nothing yet: the figure a cold start gives, kept
        # beside the headline (which is timed last, on settled clocks)
        r = bench_gemm(torch, lib, capi, datagen, args.size, args.steps, args.warmup, settle_s=0.0, step=gemm_step)
        extra["gemm_%d_cold_w%d" % (args.size, args.warmup)] = {"ms": r["ms"], "tflops": r["tflops"], "frac_fp16_peak": r["tflops"] / PEAK_FP16_TFLOPS,
                                                  "warmup": "exactly %d launches, first GPU work of the process" % args.warmup}
    if only == "":
        for s in (3072, 7680):
            r = bench_gemm(torch, lib, capi, datagen, s, max(args.steps // 2, 1), 2)
            extra["gemm_%d" % s] = {"ms": r["ms"], "tflops": r["tflops"], "frac_fp16_peak": r["tflops"] / PEAK_FP16_TFLOPS}
    if only in ("", "mx"):
        r = bench_gemm_mx(torch, lib, capi, datagen, 6144, 6144, 6144, 1, args.steps, args.warmup)
        extra["gemm_mxfp8_e5m2_bf16_6144"] = {"ms": r["ms"], "tflops": r["tflops"], "frac_fp8_peak": r["tflops"] / PEAK_FP8_TFLOPS}
        r = bench_gemm_mx(torch, lib, capi, datagen, 2040, 8100, 8192, 4, args.steps, args.warmup)
        extra["gemm_mxfp4_e2m1_bf16_m2040_k8192_n8100"] = {"ms": r["ms"], "tflops": r["tflops"],
                                                           "frac_fp4_peak": r["tflops"] / PEAK_FP4_TFLOPS}
        r = bench_gemm_mx(torch, lib, capi, datagen, 6144, 6144, 6144, 4, args.steps, args.warmup)
        extra["gemm_mxfp4_e2m1_bf16_6144"] = {"ms": r["ms"], "tflops": r["tflops"], "frac_fp4_peak": r["tflops"] / PEAK_FP4_TFLOPS}
    if only in ("", "fa") and hasattr(lib, "pto_fa_fwd_f16"):
        for name, cfg in (("fa_b1_h16_s4096_d128", (1, 16, 4096, 128, False)),
                          ("fa_causal_b4_h32_s2048_d64", (4, 32, 2048, 64, True))):
            r = bench_fa(torch, lib, capi, datagen, cfg, args.steps, args.warmup)
            extra[name] = {"ms": r["ms"], "tflops": r["tflops"], "frac_fp16_peak": r["tflops"] / PEAK_FP16_TFLOPS,
                           "flop_convention": r["flop_convention"]}
    if only in ("", "tcvt"):
        for kind in ("f16", "bf16"):
            r = bench_tcvt(torch, lib, capi, datagen, args.steps, args.warmup, kind)
            extra["tcvt_f32_%s_16384x8192" % kind] = {"ms": r["ms"], "gbs": r["gbs"], "frac_hbm_peak": r["gbs"] / PEAK_HBM_GBS}
    if only in ("", "quant") and hasattr(lib, "pto_quant_mxfp8_f32"):
        r = bench_quant(torch, lib, capi, datagen, args.steps, args.warmup)
        extra["quant_mxfp8_f32_16384x8192"] = {"ms": r["ms"], "gbs": r["gbs"], "frac_hbm_peak": r["gbs"] / PEAK_HBM_GBS}
    if only in ("", "topk"):
        r = bench_topk(torch, lib, capi, datagen, args.steps, args.warmup)
        extra["topk_4800x1024_top1000_f32"] = {"ms": r["ms"], "gbs": r["gbs"], "frac_hbm_peak": r["gbs"] / PEAK_HBM_GBS,
                                               "rows_per_s": r["rows_per_s"]}
    if only in ("", "gather"):
        r = bench_gather(torch, lib, capi, datagen, args.steps, args.warmup)
        hbm_side = GATHER_HBM_SIDE_BYTES
        extra["gather_rows_65536x1024_f16"] = {"ms": r["ms"], "gbs_algorithmic": r["gbs"], "cache_resident": True,
                                               "hbm_side_bytes_per_launch": hbm_side,
                                               "gbs_hbm_side": hbm_side / (r["ms"] * 1e-3) / 1e9,
                                               "frac_hbm_peak_hbm_side": hbm_side / (r["ms"] * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                               "note": "cache-resident figure, not an HBM roofline number: gbs_algorithmic counts rows read + "
                                                       "rows written + indices (268.7 MB), but the 32 MiB table is served from cache; the "
                                                       "FETCH_SIZE / WRITE_SIZE counters (profiles/) read 85.0 MB + 134.3 MB per launch at the "
                                                       "L2 <-> fabric boundary, which gbs_hbm_side is computed from"}

    if only in ("", "gemm") and args.size == 6144:
        # the same problem after a settle period (the headline below is timed after exactly W warm-up launches, whatever W
        # is; a few launches of 0.4 ms do not bring the GPU out of its idle or memory-bound clocks)
        r = bench_gemm(torch, lib, capi, datagen, 6144, max(args.steps, 20), 30, settle_s=max(SETTLE_S, 0.3), step=gemm_step)
        extra["gemm_6144_after_settle"] = {"ms": r["ms"], "tflops": r["tflops"], "frac_fp16_peak": r["tflops"] / PEAK_FP16_TFLOPS,
                                           "warmup": "30 launches, then untimed launches until 0.3 s have passed"}
    if gemm_step is not None:
        gemm = bench_gemm(torch, lib, capi, datagen, args.size, args.steps, args.warmup, settle_s=0.0, step=gemm_step)   # exactly W warm-ups
        extra["headline_order"] = "timed last: W warm-up + K timed launches directly after gemm_6144_after_settle (the same kernel, settled clocks)"

    line = {
        "metric": "GEMM TFLOPS & % MFMA peak at m=n=k=6144; flash-attn fwd TFLOPS",
        "value": gemm["tflops"] if gemm else None,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": gemm["ms"] if gemm else None,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp16 x fp16 -> fp32 accumulate",
        "data": "synthetic: A [m,k], B [n,k] i.i.d. uniform[-1,1] fp16 from seed 19 / 1019",
        "config": {"workload": "fp16->fp32 GEMM m=n=k=%d, A row-major, B column-major, full K reduction per output tile "
                               "(256x192 C tile per workgroup at 6144, K-step 64)" % args.size},
        "extra": extra,
    }
    extra["warmup_policy"] = ("headline: exactly %d untimed launches; workloads under extra: %d launches, then untimed launches "
                              "until %.0f ms have passed" % (args.warmup, args.warmup, args.settle_ms))
    traffic = None
    if gemm and args.size == 6144:
        rd = GEMM_6144_FETCH_KIB * GEMM_6144_FETCH_SCALE * 1024.0
        wr = GEMM_6144_WRITE_KIB * GEMM_6144_WRITE_SCALE * 1024.0
        traffic = rd + wr
    if gemm:
        line["roofline"] = {"bound": "mfma", "achieved": gemm["tflops"], "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                            "frac": gemm["tflops"] / PEAK_FP16_TFLOPS, "traffic": traffic,
                            "kernel": GEMM_KERNEL_NOTE.get(args.size, "GemmF16F32W4 (256-row C tiles on four wavefronts; tile width 256 / 192 / 128 by whole rounds)"),
                            "flops_per_launch": gemm["flops"],
                            "traffic_unit": "bytes per launch (read + write at the L2 <-> fabric boundary)",
                            "algorithmic_bytes": 2.0 * 2 * args.size ** 2 + 4.0 * args.size ** 2}
    if not args.no_cpu and only in ("", "gemm"):
        line["cpu_baseline"] = cpu_baseline(datagen, args.size)
        if only == "":
            line["extra"]["cpu_baselines"] = cpu_baselines_extra(datagen, line["cpu_baseline"]["cores"])
    print(json.dumps(line))


if __name__ == "__main__":
    main()
