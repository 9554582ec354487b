"""Pins of the oracle's integer-activation Q4_K path (activations -> Q8_K blocks, integer sub-block dots)."""
import numpy as np

import oracle as O
from conftest import synth
from np_formats import f16, unpack_scales_q4_k


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
