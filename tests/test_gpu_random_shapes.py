"""Seeded random shapes through qmatmul, every encoding: a net under the shape-by-shape cases of test_gpu_parity.py.

The dispatch picks a kernel from (encoding, lhs type, M, N, K) by thresholds and fitted costs; a draw of shapes that
nobody chose lands on both sides of most of them.  Each case is checked against the oracle's fp64 product of the
operands the path defines (Q4_0: the Q8_0 round trip of the lhs), within the bar of the reference's isclose scaled by
the size of a row's outputs (sums of thousands of terms may cancel to far below their terms' rounding).
"""
import numpy as np
import pytest
import torch

import oracle as O
from conftest import synth
from mojo_amd import QuantizationConfig, QuantizationEncoding as QE, qmatmul

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
ENC = {QE.Q4_0: O.Q4_0, QE.Q4_K: O.Q4_K, QE.Q6_K: O.Q6_K, QE.Q5_K: O.Q5_K}
INDEX = {QE.Q4_0: 0, QE.Q4_K: 1, QE.Q6_K: 2, QE.Q5_K: 4}
ROWS = (1, 2, 3, 4, 5, 7, 8, 9, 12, 16, 17, 24, 31, 32, 33, 40, 48, 63, 64, 65, 80, 96, 100, 128, 129, 200, 256, 257, 300, 520)
KS = (256, 512, 768, 1024, 1280, 2048, 2304, 2816, 4096, 4608, 5120, 6144, 8192, 11008, 12288, 14336)


def _cases(enc_index: int, count: int):
    rng = np.random.Generator(np.random.PCG64(1000 + enc_index))
    out = []
    for _ in range(count):
        m = int(rng.choice(ROWS))
        k = int(rng.choice(KS))
        # wide enough for several tiles now and then, small enough for the oracle's fp64 product
        n = int(rng.integers(1, 40)) * 8 if rng.random() < 0.5 else int(rng.integers(300, 2400)) // 8 * 8
        while m * n * k > 3.0e9:
            n = max(8, n // 2 // 8 * 8)
        out.append((m, n, k, bool(rng.random() < 0.5)))
    return out


def _close(got, truth, what):
    got = got.detach().cpu().numpy()
    scale = np.abs(truth).max(axis=1, keepdims=True)
    ok = np.abs(got - truth) <= 1e-4 + 1e-4 * scale + 1e-3 * np.abs(truth)
    assert ok.all(), f"{what}: {np.count_nonzero(~ok)} of {ok.size} outputs off; worst {np.abs(got - truth).max()} (row scale {scale.max()})"


@pytest.mark.parametrize("enc", [QE.Q4_K, QE.Q5_K, QE.Q6_K, QE.Q4_0])
def test_random_shapes_block_encodings(enc):
    for i, (m, n, k, bf16) in enumerate(_cases(INDEX[enc], 60)):
        w, a = synth(2000 + 37 * INDEX[enc] + i, n, k, m)
        if bf16:
            a = O.bf16_to_f32(O.f32_to_bf16(a))
        wq = O.quantize(ENC[enc], w)
        truth = O.matmul_q4_0(a, wq) if enc == QE.Q4_0 else O.matmul_f64(ENC[enc], a, wq)
        lhs = torch.from_numpy(a).to(DEV)
        got = qmatmul(enc, None, lhs.to(torch.bfloat16) if bf16 else lhs, torch.from_numpy(wq).to(DEV))
        _close(got, truth, f"{enc.name} {m}x{n}x{k} bf16={bf16}")


def test_random_shapes_gptq():
    for i, (m, n, k, bf16) in enumerate(_cases(9, 60)):
        group = (64, 128, 128, 256)[i % 4]
        if k % group:
            continue
        w, a = synth(3000 + i, n, k, m)
        if bf16:
            a = O.bf16_to_f32(O.f32_to_bf16(a))
        qw, sc, qz, gi = O.quantize_gptq(w, group)
        truth = O.matmul_gptq(a, qw, sc, qz, group=group, f64=True)
        lhs = torch.from_numpy(a).to(DEV)
        got = qmatmul(QE.GPTQ, QuantizationConfig(group_size=group), lhs.to(torch.bfloat16) if bf16 else lhs,
                      torch.from_numpy(qw).to(DEV), torch.from_numpy(sc.view(np.float16)).to(DEV), torch.from_numpy(qz).to(DEV),
                      torch.from_numpy(gi).to(DEV))
        _close(got, truth, f"GPTQ g{group} {m}x{n}x{k} bf16={bf16}")
