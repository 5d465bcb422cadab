"""Writes the golden vectors of the whole path (inputs and expected outputs) as .npz files
beside this script:

    python tests/golden/make_fixtures.py

The reference ships no golden vectors and cannot be built or run here (nvcc, CUTLASS and a
Blackwell GPU are all absent), so the expected outputs come from the scalar C restatement in
oracle/ref_scalar.c (codes, scales) and from the float64 product of the dequantized operands
(GEMM).  They pin the path against drift: the numpy oracle, the scalar oracle and the HIP
kernels must all keep reproducing these bytes.

Cases: the reference's own example problem (main.py:8-9: K=3584 split 2560/896/128), the
K=4096 split of its benches (bench_reorder.cu:26-28) and the K=14336 down-projection shape,
each with a few token rows and feature rows, absmax-sorted reorder index (main.py:31-33).
"""
from __future__ import annotations

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

CASES = {
    # name: (token rows, feature rows, KN, KS, KO, seed, student_t)
    "k3584": (3, 4, 2560, 896, 128, 11, False),
    "k4096": (4, 4, 2560, 1408, 128, 12, False),
    "k14336": (2, 3, 8960, 4928, 448, 13, True),
}


def main():
    from oracle import mx_oracle as mo
    from oracle import scalar as sc
    from tests import helpers as H

    sc.build()
    for name, (m, n, kn, ks, ko, seed, student) in CASES.items():
        k = kn + ks + ko
        x = H.make_activations(m, k, seed, student_t=student)
        w = H.make_weights(n, k, seed + 100)
        idx = H.absmax_sort_index(x).numpy()
        xb, wb = H.bf16_bits(x), H.bf16_bits(w)
        qx = sc.quantize_x(xb, idx, kn, ks, ko)
        qw = sc.quantize_w(wb, idx, kn, ks, ko)
        out = {"x_bits": xb, "w_bits": wb, "idx": idx, "split": np.array([kn, ks, ko], np.int32)}
        for tag, q, rows in (("x", qx, m), ("w", qw, n)):
            for c in ("qn", "qs", "qo"):
                out[f"{tag}_{c}"] = q[c]
            for s, kseg in zip(("sfn", "sfs", "sfo"), (kn, ks, ko)):
                out[f"{tag}_{s}"] = mo.sf_gather(q[s], rows, kseg)      # logical [rows, kseg/32] E8M0 bytes
        fx = mo.reorder_quantize_x(H.bf16_f32(x), idx, kn, ks, ko)
        fw = mo.reorder_quantize_w(H.bf16_f32(w), idx, kn, ks, ko)
        out["d_f32"] = mo.mixed_matmul(fx, fw).astype(np.float32)           # before the bf16 rounding
        # sum of |a||b| per output: scales the allowance for the order of the fp32 accumulation
        out["d_abs_f32"] = (np.abs(mo.dequantize_x(fx)).astype(np.float64)
                            @ np.abs(mo.dequantize_w(fw)).astype(np.float64).T).astype(np.float32)
        path = os.path.join(HERE, f"path_{name}.npz")
        np.savez_compressed(path, **out)
        print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
