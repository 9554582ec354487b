"""Pins of the oracle's quantisers, integer block dots and matmuls (no GPU)."""
import numpy as np
import pytest

import np_formats as NF
import oracle as O
from conftest import synth


# ------------------------------------------------------------------ Q4_0 / Q8_0 quantisers: closed-form properties
def test_q4_0_quantiser_properties():
    w, _ = synth(0, 64, 1024, 1)
    packed = O.quantize(O.Q4_0, w)
    assert np.array_equal(packed, NF.quantize_q4_0(w))  # independent vectorised restatement
    back = O.dequantize(O.Q4_0, packed, 1024)
    blocks = w.reshape(64, 32, 32)
    d = O.f16_to_f32(packed.reshape(64, 32, 18)[:, :, 0:2].copy().view(np.uint16)[..., 0])
    codes = packed.reshape(64, 32, 18)[:, :, 2:]
    q = np.concatenate([codes & 15, codes >> 4], axis=2).astype(np.int32)
    idx = np.argmax(np.abs(blocks), axis=2)
    # the element of largest magnitude maps to code 0, i.e. to -8*d
    assert np.all(np.take_along_axis(q, idx[..., None], axis=2) == 0)
    # d = max / -8 rounded to fp16
    mx = np.take_along_axis(blocks, idx[..., None], axis=2)[..., 0]
    assert np.array_equal(d, (mx / np.float32(-8)).astype(np.float16).astype(np.float32))
    # error bound: half a step except at the +8 clamp (code 15 stands for values up to 8*d)
    err = np.abs(back.reshape(64, 32, 32) - blocks)
    step = np.abs(mx / -8)[..., None]
    assert np.all(err <= step * (0.5 + 2.0**-9) + 1e-9) or np.all(err[q < 15] <= (step * np.ones_like(err))[q < 15] * 0.51)
    assert np.all(err <= step * 1.01)


def test_q4_0_quantiser_edge_blocks():
    x = np.zeros((3, 32), np.float32)
    x[1, :] = 0.25          # all equal: the first element wins, every code 0 (= -8 * d with d = -1/32)
    x[2, 5] = -3.0
    x[2, 9] = 3.0           # tie in magnitude: the first (negative) one decides the sign of d
    packed = O.quantize(O.Q4_0, x)
    assert np.array_equal(packed, NF.quantize_q4_0(x))
    d = O.f16_to_f32(packed[:, 0:2].copy().view(np.uint16)[:, 0])
    assert d[0] == 0 and np.all(packed[0, 2:] == 0x88)  # zero block: d = 0, codes 8
    assert d[1] == np.float32(-0.03125) and np.all(packed[1, 2:] == 0x00)
    assert d[2] == np.float32(0.375)  # -3 / -8
    back = O.dequantize(O.Q4_0, packed, 32)
    assert back[2, 5] == -3.0 and back[2, 9] == np.float32(7 * 0.375)  # +3 clamps to code 15 = 7*d


def test_q8_0_quantiser_properties_and_ties():
    _, a = synth(1, 8, 4096, 8)
    packed = O.quantize_q8_0(a)
    assert np.array_equal(packed, NF.quantize_q8_0(a))
    blocks = packed.reshape(8, 128, 34)
    q = blocks[:, :, 2:].view(np.int8).astype(np.int32)
    assert q.min() >= -127 and q.max() <= 127
    idx = np.argmax(np.abs(a.reshape(8, 128, 32)), axis=2)
    assert np.all(np.abs(np.take_along_axis(q, idx[..., None], axis=2)) == 127)
    # explicit ties: amax = 127 -> d = 1 -> x/d lands exactly on .5; round half away from zero
    x = np.zeros((1, 32), np.float32)
    x[0, :9] = [127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5]
    got = O.quantize_q8_0(x)[0, 2:11].view(np.int8)
    assert got.tolist() == [127, 1, 2, 3, -1, -2, -3, 127, -127]
    assert np.all(O.quantize_q8_0(np.zeros((1, 32), np.float32)) == 0)


# ------------------------------------------------------------------ K-quant / GPTQ packers: valid blocks, bounded error
@pytest.mark.parametrize("enc,bits", [(O.Q4_K, 4), (O.Q6_K, 6)])
def test_kquant_packers_round_trip_error(enc, bits):
    w, _ = synth(2, 32, 2048, 1)
    w[3, 256:512] = 0.0
    w[4, :] = 0.0
    packed = O.quantize(enc, w)
    back = O.dequantize(enc, packed, 2048)
    assert np.isfinite(back).all()
    assert np.all(back[4] == 0) and np.all(back[3, 256:512] == 0)
    rng_per_sub = np.ptp(w.reshape(32, -1, 32 if enc == O.Q4_K else 16), axis=2).max()
    # error below ~one quantisation step of the widest sub-block (scales are themselves quantised)
    assert np.abs(back - w).max() <= 1.6 * rng_per_sub / (2**bits - 1)
    assert np.sqrt(np.mean((back - w) ** 2)) < {4: 2.0e-3, 6: 5.0e-4}[bits]


def test_gptq_packer_round_trip_error():
    w, _ = synth(3, 64, 1024, 1)
    qw, sc, qz, gi = O.quantize_gptq(w)
    back = O.dequantize_gptq(qw, sc, qz)
    amax = np.abs(w.reshape(64, 8, 128)).max(axis=2)
    step = (2 * amax / 15)[:, :, None]
    assert np.all(np.abs(back.reshape(64, 8, 128) - w.reshape(64, 8, 128)) <= 0.51 * step + 1e-3 * step + 1e-7)


# ------------------------------------------------------------------ integer block dots
def test_block_dots_against_int64_and_extremes():
    w, a = synth(0, 48, 512, 3)
    wq, aq = O.quantize(O.Q4_0, w), O.quantize_q8_0(a)
    got = O.block_dots_q4_0_q8_0(aq, wq, 512)
    wc = wq.reshape(48, 16, 18)[:, :, 2:].astype(np.int64)
    w_int = np.concatenate([wc & 15, wc >> 4], axis=2) - 8
    a_int = aq.reshape(3, 16, 34)[:, :, 2:].view(np.int8).astype(np.int64)
    want = np.einsum("mbk,nbk->mnb", a_int, w_int)
    assert np.array_equal(got.astype(np.int64), want)
    ext_w = np.zeros((2, 18), np.uint8); ext_w[1, 2:] = 0xFF
    ext_a = np.zeros((2, 34), np.uint8); ext_a[0, 2:] = np.int8(-127).view(np.uint8); ext_a[1, 2:] = 127
    got = O.block_dots_q4_0_q8_0(ext_a, ext_w, 32)[:, :, 0]
    assert got.tolist() == [[32 * 8 * 127, -32 * 7 * 127], [-32 * 8 * 127, 32 * 7 * 127]]


def test_q4_0_matmul_is_scaled_sum_of_block_dots():
    w, a = synth(0, 40, 1024, 2)
    wq, aq = O.quantize(O.Q4_0, w), O.quantize_q8_0(a)
    dots = O.block_dots_q4_0_q8_0(aq, wq, 1024).astype(np.float64)
    dw = O.f16_to_f32(wq.reshape(40, 32, 18)[:, :, 0:2].copy().view(np.uint16)[..., 0]).astype(np.float64)
    da = O.f16_to_f32(aq.reshape(2, 32, 34)[:, :, 0:2].copy().view(np.uint16)[..., 0]).astype(np.float64)
    truth = np.einsum("mnb,nb,mb->mn", dots, dw, da)
    got = O.matmul_q4_0(a, wq)
    assert O.isclose(got, truth, 1e-5, 1e-6).all()
    assert np.array_equal(got, O.matmul_q4_0_q8_0(aq, wq, 1024))


# ------------------------------------------------------------------ fp32 matmuls: fp64 truth and closed forms
@pytest.mark.parametrize("enc", [O.Q4_0, O.Q4_K, O.Q6_K])
def test_matmul_f32_against_fp64_numpy(enc):
    w, a = synth(4, 96, 2048, 3)
    wq = O.quantize(enc, w)
    deq = O.dequantize(enc, wq, 2048).astype(np.float64)
    truth = a.astype(np.float64) @ deq.T
    assert np.abs(O.matmul_f64(enc, a, wq) - truth).max() < 1e-12
    assert O.isclose(O.matmul_f32(enc, a, wq), truth, 1e-5, 2e-6).all()
    # bf16-rounded weights mode
    deq_bf = O.bf16_to_f32(O.f32_to_bf16(O.dequantize(enc, wq, 2048))).astype(np.float64)
    assert np.abs(O.matmul_f64(enc, a, wq, w_bf16=True) - a.astype(np.float64) @ deq_bf.T).max() < 1e-12


def test_matmul_gptq_against_fp64_numpy():
    w, a = synth(5, 64, 512, 3)
    qw, sc, qz, _ = O.quantize_gptq(w)
    truth = a.astype(np.float64) @ O.dequantize_gptq(qw, sc, qz).astype(np.float64).T
    assert np.abs(O.matmul_gptq(a, qw, sc, qz, f64=True) - truth).max() < 1e-12
    assert O.isclose(O.matmul_gptq(a, qw, sc, qz), truth, 1e-5, 2e-6).all()


def test_matmul_special_cases():
    # one-hot activation picks out one dequantised weight column
    w, _ = synth(6, 16, 512, 1)
    for enc in (O.Q4_K, O.Q6_K):
        wq = O.quantize(enc, w)
        deq = O.dequantize(enc, wq, 512)
        a = np.zeros((1, 512), np.float32)
        a[0, 301] = 2.0
        assert np.array_equal(O.matmul_f32(enc, a, wq)[0], 2.0 * deq[:, 301])
    # constant codes: Q4_K block with all codes 5, scales 3, mins 2 -> w = 15 d - 2 dmin everywhere
    blk = np.zeros((1, 144), np.uint8)
    blk[0, 0:4] = [0x00, 0x3C, 0x00, 0x38]  # d = 1, dmin = 0.5
    blk[0, 4:16] = O.pack_scales_q4_k(np.full(8, 3, np.uint8), np.full(8, 2, np.uint8))
    blk[0, 16:] = 0x55
    a = np.arange(256, dtype=np.float32)[None, :] / 16
    assert O.matmul_f32(O.Q4_K, a, blk)[0, 0] == np.float32(14.0 * a.sum())
    # batch rows are independent, and permuting weight rows permutes outputs
    w, a = synth(7, 32, 256, 4)
    wq = O.quantize(O.Q4_K, w)
    full = O.matmul_f32(O.Q4_K, a, wq)
    for i in range(4):
        assert np.array_equal(full[i], O.matmul_f32(O.Q4_K, a[i:i + 1], wq)[0])
    perm = np.random.default_rng(0).permutation(32)
    assert np.array_equal(O.matmul_f32(O.Q4_K, a, wq[perm]), full[:, perm])


def test_isclose_is_the_reference_rule():
    # stdlib/src/math/math.mojo:1023-1030: symmetric, atol OR rtol*max(|a|,|b|), equal infinities close, nan never
    assert O.isclose(1.0, 1.0009, 1e-3, 1e-4) and not O.isclose(1.0, 1.0011, 1e-3, 1e-4)
    assert O.isclose(0.0, 9e-5, 1e-3, 1e-4) and not O.isclose(0.0, 2e-4, 1e-3, 1e-4)
    assert O.isclose(np.inf, np.inf) and not O.isclose(np.inf, -np.inf) and not O.isclose(np.nan, np.nan)
    assert O.isclose(1000.0, 1000.9, 1e-3, 1e-4) == O.isclose(1000.9, 1000.0, 1e-3, 1e-4)


def test_swiglu_closed_forms():
    """silu(x) * u: zero at zero, x for large x, the reflection identity silu(x) - silu(-x) = x, the slope 1/2 at the
    origin, the minimum -0.27846 at x = -1.27846, and no overflow at either end of the fp32 range."""
    x = np.array([0.0, 1.0, -1.0, 30.0, -30.0, 1e30, -1e30], np.float32)
    one = np.ones_like(x)
    s = O.swiglu(x, one)
    assert s[0] == 0.0 and abs(s[1] - 1.0 / (1.0 + np.exp(-1.0))) < 1e-15
    assert np.allclose(O.swiglu(x, one) - O.swiglu(-x, one), x.astype(np.float64), rtol=1e-12)
    assert abs(s[3] - 30.0) < 1e-11 and abs(s[4]) < 1e-11 and s[5] == np.float64(np.float32(1e30)) and s[6] == 0.0
    assert abs(O.swiglu(np.float32(1e-6), 1.0) / 1e-6 - 0.5) < 1e-6
    xm = -1.2784645
    assert abs(O.swiglu(xm, 1.0) + 0.2784645) < 1e-6 and O.swiglu(xm - 0.01, 1.0) > O.swiglu(xm, 1.0) < O.swiglu(xm + 0.01, 1.0)
    assert np.array_equal(O.swiglu(x, 3.0 * one), 3.0 * s)



def test_rmsnorm_closed_forms_and_restatement():
    """qo_rmsnorm: a constant row c gives gamma * c / sqrt(c^2 + eps); with eps = 0 the squares of y / gamma sum to K and
    scaling x changes nothing; an independent fp64 restatement agrees to fp32 rounding; to_bf16 is the bf16 narrowing of
    the fp32 result."""
    rng = np.random.default_rng(91)
    k = 768
    gamma = rng.uniform(0.5, 1.5, k).astype(np.float32)
    c = np.float32(-3.25)
    y = O.rmsnorm(np.full((2, k), c, np.float32), gamma, 1e-5)
    assert np.allclose(y, gamma.astype(np.float64) * c / np.sqrt(float(c) ** 2 + 1e-5), rtol=3e-7)
    x = (rng.standard_normal((5, k)) * np.logspace(-3, 3, 5)[:, None]).astype(np.float32)
    y0 = O.rmsnorm(x, gamma, 0.0)
    assert np.allclose(((y0.astype(np.float64) / gamma) ** 2).sum(axis=1), k, rtol=1e-6)
    assert np.allclose(O.rmsnorm(4.0 * x, gamma, 0.0), y0, rtol=3e-7)  # (a power of two: exact up to the one rounding of rs)
    eps = 1e-3
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + eps) * gamma
    assert np.allclose(O.rmsnorm(x, gamma, eps), want, rtol=4e-7, atol=0)
    assert np.array_equal(O.rmsnorm(x, gamma, eps, to_bf16=True), O.bf16_to_f32(O.f32_to_bf16(O.rmsnorm(x, gamma, eps))))
    # a larger eps can only shrink the result
    assert np.all(np.abs(O.rmsnorm(x, gamma, 1.0)) <= np.abs(y0))


def test_timed_cpu_baseline_kernel_agrees_with_the_checker():
    """The hand-vectorised Q4_K kernel that the benchmark times sums in another order than matmul_f32: it is held to the
    matmul tolerance (rtol 1e-3, atol 1e-4, symmetric) against it and against the fp64 truth, never used as a checker."""
    rng = np.random.default_rng(11)
    for m, n, k in ((1, 70, 4096), (3, 33, 14336), (2, 9, 256)):
        w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
        wq = O.quantize(O.Q4_K, w)
        a = rng.standard_normal((m, k)).astype(np.float32)
        got = O.baseline_matmul_q4_k(a, wq)
        if got is None:
            pytest.skip("host without AVX2")
        for want in (O.matmul_f32(O.Q4_K, a, wq), O.matmul_f64(O.Q4_K, a, wq).astype(np.float32)):
            tol = np.maximum(1e-3 * np.maximum(np.abs(got), np.abs(want)), 1e-4)
            assert (np.abs(got - want) <= tol).all()
