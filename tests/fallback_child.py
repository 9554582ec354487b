"""Child process of test_gpu_fallback_kernels.py: runs a fixed set of small matmuls through the C ABI with whatever
QMM_DISABLE / QMM_Q4K_TILE / QMM_*_PLANES the parent put into the environment (the library reads them once per process) and checks
every result against the CPU oracle.  Prints one line per case; exits non-zero on the first mismatch."""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import oracle as O  # noqa: E402
from conftest import synth  # noqa: E402
from mojo_amd import QuantizationConfig, QuantizationEncoding as QE, qmatmul  # noqa: E402

CASES = {
    "Q4_K": [(1, 300, 4096, False), (2, 130, 2048, True), (4, 200, 4096, False), (12, 64, 8192, False), (16, 72, 512, True),
             (40, 300, 1024, True), (1, 70, 32768, False), (200, 260, 512, True), (3, 1100, 8192, False), (1030, 8200, 512, True)],
    "Q4_0": [(1, 200, 4096, False), (4, 200, 4096, True), (9, 72, 1056, False), (16, 200, 4096, False), (80, 136, 1024, True), (80, 300, 2560, True)],
    "Q6_K": [(1, 8200, 2048, False), (1, 300, 4096, True), (4, 200, 4096, False), (16, 72, 512, False), (70, 136, 1024, True), (8, 600, 4096, False), (70, 300, 2560, True), (6, 520, 8192, True)],
    "Q5_K": [(2, 300, 4096, False), (6, 200, 4096, True), (16, 72, 1024, False), (1030, 8200, 512, True), (70, 300, 2560, True),
             (12, 520, 6144, False)],
    "GPTQ": [(1, 264, 1024, False), (4, 264, 1024, True), (16, 264, 1024, False), (40, 264, 1024, True), (1030, 8200, 512, True)],
}


def main() -> int:
    dev = "cuda:0"
    seed = 70
    for name, cases in CASES.items():
        for m, n, k, bf16 in cases:
            seed += 1
            w, a = synth(seed, n, k, m)
            if bf16:
                a = O.bf16_to_f32(O.f32_to_bf16(a))
            lhs = torch.from_numpy(a).to(dev)
            if bf16:
                lhs = lhs.to(torch.bfloat16)
            if name == "GPTQ":
                qw, sc, qz, gi = O.quantize_gptq(w)
                want = O.matmul_gptq(a, qw, sc, qz)
                got = qmatmul(QE.GPTQ, QuantizationConfig(), lhs, torch.from_numpy(qw).to(dev),
                              torch.from_numpy(sc.view(np.float16)).to(dev), torch.from_numpy(qz).to(dev))
            else:
                enc, oenc = {"Q4_K": (QE.Q4_K, O.Q4_K), "Q4_0": (QE.Q4_0, O.Q4_0), "Q6_K": (QE.Q6_K, O.Q6_K),
                             "Q5_K": (QE.Q5_K, O.Q5_K)}[name]
                wq = O.quantize(oenc, w)
                want = O.matmul_q4_0(a, wq) if name == "Q4_0" else O.matmul_f32(oenc, a, wq)
                got = qmatmul(enc, None, lhs, torch.from_numpy(wq).to(dev))
            ok = O.isclose(got.cpu().numpy(), want, 1e-3, 1e-4)
            print(f"{name} m={m} n={n} k={k} bf16={bf16}: {'ok' if ok.all() else 'MISMATCH %d of %d' % ((~ok).sum(), ok.size)}", flush=True)
            if not ok.all():
                return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
