#!/usr/bin/env python3
"""Writes tests/golden/qmm_small.npz: small seeded inputs, their packed blocks and the oracle's outputs.

The reference snapshot holds no vectors for this path, so these are frozen
outputs of the CPU oracle (after it is pinned by tests/test_oracle_*.py): they
guard both the oracle and the GPU kernels against silent drift.
Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle as O  # noqa: E402


def main():
    rng = np.random.Generator(np.random.PCG64(2024))
    n, k, m = 8, 256, 2
    w = (0.02 * rng.standard_normal((n, k), dtype=np.float32)).astype(np.float32)
    a = rng.standard_normal((m, k), dtype=np.float32)
    out = {"w": w.astype(np.float16), "a": a}  # weights kept as fp16 to keep the file small; requantised from that
    w = out["w"].astype(np.float32)
    for name, enc in (("q4_0", O.Q4_0), ("q4_k", O.Q4_K), ("q6_k", O.Q6_K)):
        packed = O.quantize(enc, w)
        out[f"{name}_packed"] = packed
        out[f"{name}_deq_bits"] = O.dequantize(enc, packed, k).view(np.uint32)
        out[f"{name}_out"] = O.matmul_q4_0(a, packed) if enc == O.Q4_0 else O.matmul_f32(enc, a, packed)
    aq = O.quantize_q8_0(a)
    out["a_q8_0"] = aq
    out["q4_0_block_dots"] = O.block_dots_q4_0_q8_0(aq, out["q4_0_packed"], k)
    qw, sc, qz, gi = O.quantize_gptq(w)
    out.update(gptq_qweight=qw, gptq_scales=sc, gptq_qzeros=qz, gptq_g_idx=gi,
               gptq_deq_bits=O.dequantize_gptq(qw, sc, qz).view(np.uint32), gptq_out=O.matmul_gptq(a, qw, sc, qz))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "qmm_small.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
