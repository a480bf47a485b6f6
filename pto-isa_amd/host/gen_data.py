#!/usr/bin/python3
"""Writes the input and golden files of the GEMM host program in the reference's layout
(kernels/manual/a2a3/gemm_performance/scripts/gen_data.py:19-46): input/x1_gm.bin = A [m,k] fp16,
input/x2_gm.bin = B transposed, i.e. stored [n,k] fp16, output/golden.bin = A x B in fp32; values uniform(-5, 5),
numpy seed 19.

    python gen_data.py <dir> [m k n]
"""
import os
import sys

import numpy as np


def gen(directory, m, k, n):
    np.random.seed(19)
    x1 = np.random.uniform(-5, 5, [m, k]).astype(np.float16)
    x2 = np.random.uniform(-5, 5, [k, n]).astype(np.float16)
    golden = np.matmul(x1.astype(np.float32), x2.astype(np.float32)).astype(np.float32)
    os.makedirs(os.path.join(directory, "input"), exist_ok=True)
    os.makedirs(os.path.join(directory, "output"), exist_ok=True)
    x1.tofile(os.path.join(directory, "input", "x1_gm.bin"))
    np.ascontiguousarray(x2.transpose()).tofile(os.path.join(directory, "input", "x2_gm.bin"))
    golden.tofile(os.path.join(directory, "output", "golden.bin"))


if __name__ == "__main__":
    d = sys.argv[1] if len(sys.argv) > 1 else "."
    dims = [int(x) for x in sys.argv[2:5]] if len(sys.argv) > 4 else [6144, 6144, 6144]
    gen(d, *dims)
