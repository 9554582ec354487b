"""Frozen vectors (tests/golden/qmm_small.npz): the oracle on CPU, the kernels on the GPU."""
import os

import numpy as np
import pytest

import oracle as O

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "qmm_small.npz"))
K = 256
ENC = (("q4_0", O.Q4_0), ("q4_k", O.Q4_K), ("q6_k", O.Q6_K))


def test_oracle_reproduces_golden_vectors():
    w, a = G["w"].astype(np.float32), G["a"]
    for name, enc in ENC:
        packed = O.quantize(enc, w)
        assert np.array_equal(packed, G[f"{name}_packed"])
        assert np.array_equal(O.dequantize(enc, packed, K).view(np.uint32), G[f"{name}_deq_bits"])
        out = O.matmul_q4_0(a, packed) if enc == O.Q4_0 else O.matmul_f32(enc, a, packed)
        assert np.array_equal(out, G[f"{name}_out"])
    assert np.array_equal(O.quantize_q8_0(a), G["a_q8_0"])
    assert np.array_equal(O.block_dots_q4_0_q8_0(G["a_q8_0"], G["q4_0_packed"], K), G["q4_0_block_dots"])
    qw, sc, qz, gi = O.quantize_gptq(w)
    assert np.array_equal(qw, G["gptq_qweight"]) and np.array_equal(sc, G["gptq_scales"])
    assert np.array_equal(O.dequantize_gptq(qw, sc, qz).view(np.uint32), G["gptq_deq_bits"])


@pytest.mark.gpu
def test_gpu_reproduces_golden_vectors():
    import torch

    from mojo_amd import QuantizationConfig, QuantizationEncoding as QE
    from mojo_amd import block_dots_q4_0, dequantize, qmatmul, quantize, quantize_gptq

    dev = "cuda:0"
    t = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(dev)
    w, a = t(G["w"].astype(np.float32)), t(G["a"])
    for (name, _), enc in zip(ENC, (QE.Q4_0, QE.Q4_K, QE.Q6_K)):
        packed = quantize(enc, w)
        assert np.array_equal(packed.cpu().numpy(), G[f"{name}_packed"])
        deq = dequantize(enc, packed).cpu().numpy().view(np.uint32)
        assert np.array_equal(deq, G[f"{name}_deq_bits"])
        out = qmatmul(enc, None, a, packed).cpu().numpy()
        assert O.isclose(out, G[f"{name}_out"], 1e-3, 1e-4).all()
    assert np.array_equal(quantize(QE.Q8_0, a).cpu().numpy(), G["a_q8_0"])
    dots = block_dots_q4_0(t(G["a_q8_0"]), t(G["q4_0_packed"])).cpu().numpy()
    assert np.array_equal(dots, G["q4_0_block_dots"])
    qw, sc, qz, gi = quantize_gptq(w)
    assert np.array_equal(qw.cpu().numpy(), G["gptq_qweight"])
    assert np.array_equal(sc.cpu().numpy().view(np.uint16), G["gptq_scales"])
    cfg = QuantizationConfig()
    deq = dequantize(QE.GPTQ, qw, sc, qz, gi, config=cfg).cpu().numpy().view(np.uint32)
    assert np.array_equal(deq, G["gptq_deq_bits"])
    out = qmatmul(QE.GPTQ, cfg, a, qw, sc, qz, gi).cpu().numpy()
    assert O.isclose(out, G["gptq_out"], 1e-3, 1e-4).all()
