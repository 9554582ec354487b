"""Pins of the oracle's integer-activation K-quant paths (activations -> Q8_K blocks, integer sub-block dots)."""
import numpy as np
import pytest

import oracle as O
from conftest import synth
from np_formats import dequant_q5_k, dequant_q6_k, f16, unpack_scales_q4_k


def _fields(q8k: np.ndarray, k: int):
    """(d f32 [rows, nb], qs int8 [rows, nb, 256], bsums int16 [rows, nb, 16]) of Q8_K bytes."""
    rows, nb = q8k.shape[0], k // 256
    b = q8k.reshape(rows, nb, 292)
    d = b[:, :, :4].copy().view(np.float32)[:, :, 0]
    qs = b[:, :, 4:260].copy().view(np.int8)
    bs = b[:, :, 260:].copy().view(np.int16)
    return d, qs, bs


def test_q8_k_quantiser_properties_and_independent_restatement():
    rng = np.random.default_rng(7)
    k = 1024
    x = (rng.standard_normal((6, k)) * rng.uniform(1e-3, 50.0, (6, 1))).astype(np.float32)
    x[2, 256:512] = 0.0                       # an all-zero block
    x[3, 5], x[3, 9] = 77.0, -77.0            # two elements of the same largest magnitude: the first one decides
    x[3, :256] = np.clip(x[3, :256], -77, 77)
    d, qs, bs = _fields(O.quantize_q8_k(x), k)
    xb = x.reshape(6, k // 256, 256)
    # independent restatement: first index of the largest magnitude, iscale = -127 / that element, ties to even
    idx = np.abs(xb).argmax(axis=2)
    mx = np.take_along_axis(xb, idx[:, :, None], 2)[:, :, 0]
    with np.errstate(divide="ignore", invalid="ignore"):
        iscale = np.where(mx != 0, np.float32(-127.0) / mx, np.float32(0)).astype(np.float32)
        want_q = np.minimum(127, np.rint((iscale[:, :, None] * xb).astype(np.float32))).astype(np.int8)
        want_d = np.where(mx != 0, np.float32(1.0) / iscale, np.float32(0)).astype(np.float32)
    np.testing.assert_array_equal(qs, want_q)
    np.testing.assert_array_equal(d.view(np.uint32), want_d.view(np.uint32))
    np.testing.assert_array_equal(bs, qs.reshape(6, k // 256, 16, 16).astype(np.int32).sum(axis=3).astype(np.int16))
    # properties: the deciding element maps to -127, codes within +-127, error bound, zero block
    assert (np.take_along_axis(qs, idx[:, :, None], 2)[:, :, 0][mx != 0] == -127).all()
    assert qs.min() >= -127 and qs.max() <= 127
    assert (np.abs(qs * d[:, :, None] - xb) <= np.abs(d)[:, :, None] * 0.5000001 + 1e-12).all()
    assert d[2, 1] == 0 and not qs[2, 1].any() and not bs[2, 1].any()
    assert qs[3, 0, 5] == -127 and qs[3, 0, 9] == 127 and d[3, 0] == np.float32(1.0) / (np.float32(-127.0) / np.float32(77.0))


def test_q8_k_rounds_half_to_even():
    x = np.zeros((1, 256), np.float32)
    x[0, 0] = 127.0                            # iscale = -1 exactly
    x[0, 1:7] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5]
    _, qs, _ = _fields(O.quantize_q8_k(x), 256)
    assert qs[0, 0, :7].tolist() == [-127, 0, -2, -2, 0, 2, 2]


def test_q4_k_q8_k_block_sums_against_int64_brute_force():
    n, k, m = 5, 768, 3
    w, a = synth(41, n, k, m)
    wq, aq = O.quantize(O.Q4_K, w), O.quantize_q8_k(a)
    isum, msum = O.block_sums_q4_k_q8_k(aq, wq, k)
    _, q8, bs = _fields(aq, k)
    wb = wq.reshape(n, k // 256, 144)
    for j in range(n):
        for b in range(k // 256):
            sc, mn = unpack_scales_q4_k(wb[j, b, 4:16])
            qs = wb[j, b, 16:].astype(np.int64)
            codes = np.empty(256, np.int64)        # element order of the block
            for c in range(4):
                codes[64 * c:64 * c + 32] = qs[32 * c:32 * c + 32] & 15
                codes[64 * c + 32:64 * c + 64] = qs[32 * c:32 * c + 32] >> 4
            for i in range(m):
                prod = (codes * q8[i, b].astype(np.int64)).reshape(8, 32).sum(axis=1)
                assert isum[i, j, b] == int((prod * sc.astype(np.int64)).sum())
                sub = bs[i, b].astype(np.int64).reshape(8, 2).sum(axis=1)
                assert msum[i, j, b] == int((sub * mn.astype(np.int64)).sum())
                assert (sub == q8[i, b].astype(np.int64).reshape(8, 32).sum(axis=1)).all()


def test_integer_path_equals_fp_path_on_exactly_representable_activations():
    """Integer activations with largest magnitude 127 in every block quantise to themselves (d = -+1), so the
    integer path must give the fp64 truth of the fp32-activation path up to fp32 summation."""
    n, k, m = 33, 1024, 4
    w, _ = synth(42, n, k, m)
    rng = np.random.default_rng(3)
    a = rng.integers(-126, 127, (m, k)).astype(np.float32)
    a[:, ::256] = np.array([127.0, -127.0, 127.0, -127.0])[:, None]
    wq = O.quantize(O.Q4_K, w)
    d, qs, _ = _fields(O.quantize_q8_k(a), k)
    np.testing.assert_array_equal(qs.reshape(m, k).astype(np.float32) * np.repeat(d, 256, axis=1), a)
    got = O.matmul_q4_k_act_q8_k(a, wq)
    truth = O.matmul_f64(O.Q4_K, a, wq)
    assert np.abs(got - truth).max() <= 2e-6 * np.abs(truth).max() + 1e-6 * np.abs(a).max()


def test_integer_path_is_a_quantisation_of_the_fp_path():
    """On N(0,1) activations the two treatments differ by the Q8_K rounding (about 0.4 % per element), far more
    than the parity tolerance: a kernel cannot pass for one while computing the other."""
    n, k, m = 64, 4096, 2
    w, a = synth(43, n, k, m)
    wq = O.quantize(O.Q4_K, w)
    ip, fp = O.matmul_q4_k_act_q8_k(a, wq), O.matmul_f32(O.Q4_K, a, wq)
    rel = np.abs(ip - fp) / np.abs(fp).max()
    assert 1e-4 < rel.max() < 3e-2
    assert not O.isclose(ip, fp, 1e-3, 1e-4).all()


@pytest.mark.parametrize("enc,bpb,d_at,dmin_at", [(O.Q5_K, 176, 0, 2), (O.Q6_K, 210, 208, None)])
def test_q5_k_q6_k_block_sums_against_int64_brute_force(enc, bpb, d_at, dmin_at):
    """Blocks of random bytes (every code, fifth-bit / high-bit and scale pattern) with d = 1 and dmin = 0 dequantise, in
    the independent NumPy restatement, to the integers sc * q: their int64 dot with the Q8_K codes is isum.  With d = 0
    and dmin = 1 the same restatement gives -mn per weight, and the dot is -msum."""
    n, k, m = 6, 768, 3
    rng = np.random.default_rng(51)
    one = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    a = rng.standard_normal((m, k)).astype(np.float32)
    aq = O.quantize_q8_k(a)
    _, q8, _ = _fields(aq, k)
    blocks = rng.integers(0, 256, (n, k // 256, bpb), dtype=np.uint8)
    deq = dequant_q5_k if enc == O.Q5_K else dequant_q6_k
    blocks[:, :, d_at:d_at + 2] = one
    if dmin_at is not None:
        blocks[:, :, dmin_at:dmin_at + 2] = 0
    wq = blocks.reshape(n, -1)
    isum, msum = O.block_sums_kquant_q8_k(enc, aq, wq, k)
    ints = deq(wq, k).astype(np.float64)
    assert np.array_equal(ints, np.rint(ints))
    want = np.einsum("nbk,mbk->mnb", ints.reshape(n, -1, 256).astype(np.int64), q8.astype(np.int64))
    assert np.array_equal(isum.astype(np.int64), want)
    if dmin_at is None:
        assert not msum.any()
        return
    blocks[:, :, d_at:d_at + 2] = 0
    blocks[:, :, dmin_at:dmin_at + 2] = one
    wq = blocks.reshape(n, -1)
    _, msum = O.block_sums_kquant_q8_k(enc, aq, wq, k)
    mins = deq(wq, k).astype(np.float64)
    want = -np.einsum("nbk,mbk->mnb", mins.reshape(n, -1, 256).astype(np.int64), q8.astype(np.int64))
    assert np.array_equal(msum.astype(np.int64), want)


def test_generic_q8_k_functions_equal_the_q4_k_ones():
    n, k, m = 9, 1024, 3
    w, a = synth(52, n, k, m)
    wq, aq = O.quantize(O.Q4_K, w), O.quantize_q8_k(a)
    for x, y in zip(O.block_sums_kquant_q8_k(O.Q4_K, aq, wq, k), O.block_sums_q4_k_q8_k(aq, wq, k)):
        assert np.array_equal(x, y)
    assert np.array_equal(O.matmul_kquant_act_q8_k(O.Q4_K, a, wq), O.matmul_q4_k_act_q8_k(a, wq))


@pytest.mark.parametrize("enc", [O.Q5_K, O.Q6_K])
def test_q5_k_q6_k_integer_path_equals_fp_path_on_exactly_representable_activations(enc):
    n, k, m = 33, 1024, 4
    w, _ = synth(53, n, k, m)
    rng = np.random.default_rng(5)
    a = rng.integers(-126, 127, (m, k)).astype(np.float32)
    a[:, ::256] = np.array([127.0, -127.0, 127.0, -127.0])[:, None]
    wq = O.quantize(enc, w)
    got = O.matmul_kquant_act_q8_k(enc, a, wq)
    truth = O.matmul_f64(enc, a, wq)
    assert np.abs(got - truth).max() <= 2e-6 * np.abs(truth).max() + 1e-6 * np.abs(a).max()
    # and on ordinary activations it is a different (quantised) treatment
    _, a2 = synth(54, n, k, m)
    ip, fp = O.matmul_kquant_act_q8_k(enc, a2, wq), O.matmul_f32(enc, a2, wq)
    assert not O.isclose(ip, fp, 1e-3, 1e-4).all()
