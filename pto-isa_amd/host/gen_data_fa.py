#!/usr/bin/python3
"""Writes the input and golden files of the flash-attention host program in the reference's layout
(kernels/manual/common/flash_atten/scripts/gen_data.py:32-158): q.bin = Q [s0, head] fp16 (N(0,1) * 1.5), kt.bin = K stored
[s1, head] fp16 (N(0,1) * 1.5), v.bin = V [s1, head] fp16 (N(0,1) * 1.2), o.bin = golden output [s0, head] fp32, numpy
seed 7.  The golden follows the reference's recipe: scores in fp32, softmax streamed over key tiles of `tile_s1` with a
running maximum and sum, the exponentials rounded to fp16 before they multiply V, fp32 accumulation, one division by the
final sum; the causal mask adds -3.40282e38 above the diagonal.

    python gen_data_fa.py <dir> [head s0 s1 [causal [tile_s1]]]
"""
import os
import sys

import numpy as np


def gen(directory, head, s0, s1, causal=False, tile_s1=256):
    np.random.seed(7)
    q = (np.random.randn(s0, head).astype(np.float16) * 1.5).astype(np.float16)
    k = (np.random.randn(head, s1).astype(np.float16) * 1.5).astype(np.float16)        # [head, s1], as the reference draws it
    x = q.astype(np.float32) @ k.astype(np.float32)
    if causal:
        x = x + np.triu(np.full(x.shape, -3.40282e+38, dtype=np.float32), 1)
    scale = np.float32(1.0 / np.sqrt(head))
    v = (np.random.randn(s1, head).astype(np.float16) * 1.2).astype(np.float16)
    tile_s1 = min(tile_s1, s1)
    run_max = run_sum = out = None
    for c0 in range(0, s1, tile_s1):
        tile = x[:, c0:c0 + tile_s1]
        new_max = tile.max(axis=1, keepdims=True)
        if run_max is not None:
            new_max = np.maximum(new_max, run_max)
        p = np.exp((tile - new_max) * scale).astype(np.float32)
        pv = p.astype(np.float16).astype(np.float32) @ v[c0:c0 + tile_s1].astype(np.float32)
        if run_max is None:
            run_sum, out = p.sum(axis=1, keepdims=True), pv
        else:
            rescale = np.exp((run_max - new_max) * scale).astype(np.float32)
            run_sum, out = rescale * run_sum + p.sum(axis=1, keepdims=True), rescale * out + pv
        run_max = new_max
    os.makedirs(directory, exist_ok=True)
    q.tofile(os.path.join(directory, "q.bin"))
    np.ascontiguousarray(k.T).tofile(os.path.join(directory, "kt.bin"))
    v.tofile(os.path.join(directory, "v.bin"))
    (out / run_sum).astype(np.float32).tofile(os.path.join(directory, "o.bin"))


if __name__ == "__main__":
    d = sys.argv[1] if len(sys.argv) > 1 else "."
    a = [int(x) for x in sys.argv[2:]]
    dims = a[:3] if len(a) >= 3 else [128, 128, 1024]
    gen(d, *dims, causal=bool(a[3]) if len(a) > 3 else False, tile_s1=a[4] if len(a) > 4 else 256)
