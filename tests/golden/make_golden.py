#!/usr/bin/env python3
"""Writes the small fixtures under tests/golden/.

The reference holds no vector for this path and its Python cannot be imported
(its module body loads a closed native library that is not shipped), so these
fixtures are produced by the pinned CPU oracle (oracle/lowbit_oracle.c) on
seeded inputs.  They freeze the oracle's output: a later change of the oracle
or of the HIP kernels that moves a byte shows up against them.

Usage: python tests/golden/make_golden.py   (rewrites lowbit_<qtype>.npz)
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "..", "oracle"))
import lowbit_oracle as orc  # noqa: E402

N, K, M = 16, 256, 3


def main():
    for name, qtype in orc.QTYPES.items():
        r = np.random.default_rng(9000 + qtype)
        w = (r.standard_normal((N, K)) * 0.02).astype(np.float32)
        w[r.random((N, K)) < 0.004] = 0.5
        w[r.random((N, K)) < 0.004] = -0.5
        w[3, :128] = 0.0                                  # zero blocks
        x = r.standard_normal((M, K)).astype(np.float32).astype(np.float16).astype(np.float32)
        blob = orc.quantize(w, qtype)
        np.savez_compressed(os.path.join(HERE, f"lowbit_{name}.npz"),
                            qtype=np.int32(qtype), w=w, x=x, blob=blob,
                            dequant=orc.dequantize(blob, qtype, w.shape),
                            y_exact=orc.mul_mat_exact(blob, x, w.shape, qtype),
                            y_ggml=orc.mul_mat_q(blob, x, w.shape, qtype))
        print(name, blob.size, "bytes")


if __name__ == "__main__":
    main()
