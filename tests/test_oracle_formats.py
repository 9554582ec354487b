"""Pins of the CPU oracle's conversions, block layouts and dequantisers (no GPU).

The reference snapshot holds no fixture for this path, so each function is pinned
by what the published formats and arithmetic fix: IEEE binary16 exhaustively,
hand-worked known-answer blocks, pack/unpack round trips over every field value,
the exactness lemma by brute force, and an independent vectorised restatement.
"""
import numpy as np
import pytest
import torch

import np_formats as NF
import oracle as O
from conftest import synth


# ------------------------------------------------------------------ fp16 / bf16
def test_f16_to_f32_exhaustive():
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    assert np.array_equal(O.f16_to_f32(h).view(np.uint32), want.view(np.uint32))


def test_f32_to_f16_round_trip_midpoints_and_random():
    h = np.arange(65536, dtype=np.uint16)
    vals = h.view(np.float16).astype(np.float32)
    fin = np.isfinite(vals)
    assert np.array_equal(O.f32_to_f16(vals[fin]), h[fin])  # every finite half survives
    pos = np.sort(vals[fin & (vals >= 0)])
    mids = ((pos[:-1].astype(np.float64) + pos[1:].astype(np.float64)) / 2).astype(np.float32)
    for delta in (-1, 0, 1):  # exact ties and their neighbours, both signs
        m = (mids.view(np.int32) + delta).view(np.float32)
        for x in (m, -m):
            assert np.array_equal(O.f32_to_f16(x), x.astype(np.float16).view(np.uint16))
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(2_000_000) * np.exp(rng.uniform(-25, 13, 2_000_000))).astype(np.float32)
    with np.errstate(over="ignore"):
        assert np.array_equal(O.f32_to_f16(x), x.astype(np.float16).view(np.uint16))
    edge = np.array([65504.0, 65519.9, 65520.0, 1e9, np.inf, -np.inf, 2.0**-24, 2.0**-25, 2.0**-25 * 1.0001, 0.0, -0.0],
                    np.float32)
    with np.errstate(over="ignore"):
        assert np.array_equal(O.f32_to_f16(edge), edge.astype(np.float16).view(np.uint16))
    assert np.isnan(O.f16_to_f32(O.f32_to_f16(np.array([np.nan], np.float32))))[0]


def test_reference_kats_for_half_types():
    # stdlib/test/builtin/test_simd.mojo:59-69: 33.0 survives bf16 and fp16 round trips
    x = np.array([33.0], np.float32)
    assert O.bf16_to_f32(O.f32_to_bf16(x))[0] == 33.0
    assert O.f16_to_f32(O.f32_to_f16(x))[0] == 33.0


def test_bf16_rule_matches_torch_and_reference_formula():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(1_000_000) * np.exp(rng.uniform(-30, 30, 1_000_000))).astype(np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.f32_to_bf16(x), want)
    # stdlib/src/builtin/simd.mojo:3287-3300 restated on integers
    bits = x.view(np.uint32).astype(np.uint64)
    ref = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(O.f32_to_bf16(x), ref)
    # every upper half with the tie / just-below / just-above lower halves
    hi = np.arange(65536, dtype=np.uint32) << 16
    for lo in (0x7FFF, 0x8000, 0x8001, 0x0000, 0xFFFF):
        v = (hi | lo).view(np.float32)
        ok = ~np.isnan(v)
        want = torch.from_numpy(v.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(O.f32_to_bf16(v)[ok], want[ok])
    assert O.f32_to_bf16(np.array([np.nan], np.float32))[0] & 0x7FC0 == 0x7FC0


# ------------------------------------------------------------------ block parameters
def test_block_sizes_and_bits_per_weight():
    assert O.BLOCK == {O.Q4_0: (32, 18), O.Q4_K: (256, 144), O.Q6_K: (256, 210), O.Q5_K: (256, 176)}
    assert [8 * b / e for e, b in O.BLOCK.values()] == [4.5, 4.5, 6.5625, 5.5]
    assert O.quantize_q8_0(np.zeros((1, 32), np.float32)).shape == (1, 34)


# ------------------------------------------------------------------ known-answer blocks worked by hand
def test_q4_0_known_block():
    # d = 0.5 (0x3800); byte j = j | ((15 - j) << 4): element j -> j-8, element j+16 -> 7-j
    blk = np.zeros(18, np.uint8)
    blk[0:2] = [0x00, 0x38]
    blk[2:] = [j | ((15 - j) << 4) for j in range(16)]
    got = O.dequantize(O.Q4_0, blk[None, :], 32)[0]
    want = np.array([(j - 8) * 0.5 for j in range(16)] + [(7 - j) * 0.5 for j in range(16)], np.float32)
    assert np.array_equal(got, want)


def test_q4_k_known_block():
    # d = 2.0 (0x4000), dmin = 0.25 (0x3400); scales/mins chosen to use every bit field
    sc = np.array([1, 63, 32, 5, 17, 48, 63, 33], np.uint8)
    mn = np.array([0, 2, 63, 31, 16, 63, 1, 47], np.uint8)
    s = np.zeros(12, np.uint8)
    s[0:4] = (sc[0:4] & 63) | ((sc[4:8] >> 4) << 6)
    s[4:8] = (mn[0:4] & 63) | ((mn[4:8] >> 4) << 6)
    s[8:12] = (sc[4:8] & 15) | ((mn[4:8] & 15) << 4)
    assert np.array_equal(O.pack_scales_q4_k(sc, mn), s)
    usc, umn = O.unpack_scales_q4_k(s)
    assert np.array_equal(usc, sc) and np.array_equal(umn, mn)
    blk = np.zeros(144, np.uint8)
    blk[0:4] = [0x00, 0x40, 0x00, 0x34]
    blk[4:16] = s
    # chunk c, byte l: low nibble (sub-block 2c) = (l + c) % 16, high nibble (sub-block 2c+1) = (3*l + c) % 16
    for c in range(4):
        for l in range(32):
            blk[16 + 32 * c + l] = ((l + c) % 16) | (((3 * l + c) % 16) << 4)
    got = O.dequantize(O.Q4_K, blk[None, :], 256)[0]
    want = np.empty(256, np.float32)
    for c in range(4):
        for l in range(32):
            want[64 * c + l] = 2.0 * sc[2 * c] * ((l + c) % 16) - 0.25 * mn[2 * c]
            want[64 * c + 32 + l] = 2.0 * sc[2 * c + 1] * ((3 * l + c) % 16) - 0.25 * mn[2 * c + 1]
    assert np.array_equal(got, want)


def test_q5_k_known_block():
    # d = 2.0, dmin = 0.25, the scale / min fields of the Q4_K block above; code of (sub-block j, position l) =
    # (5 l + 3 j) % 32: low four bits in the nibble planes, fifth bit in bit j of qh[l]
    sc = np.array([1, 63, 32, 5, 17, 48, 63, 33], np.uint8)
    mn = np.array([0, 2, 63, 31, 16, 63, 1, 47], np.uint8)
    blk = np.zeros(176, np.uint8)
    blk[0:4] = [0x00, 0x40, 0x00, 0x34]
    blk[4:16] = O.pack_scales_q4_k(sc, mn)
    code = lambda j, l: (5 * l + 3 * j) % 32
    for l in range(32):
        blk[16 + l] = sum(((code(j, l) >> 4) & 1) << j for j in range(8))
    for c in range(4):
        for l in range(32):
            blk[48 + 32 * c + l] = (code(2 * c, l) & 15) | ((code(2 * c + 1, l) & 15) << 4)
    got = O.dequantize(O.Q5_K, blk[None, :], 256)[0]
    want = np.array([2.0 * sc[j] * code(j, l) - 0.25 * mn[j] for j in range(8) for l in range(32)], np.float32)
    assert np.array_equal(got, want)
    assert {code(j, l) for j in range(8) for l in range(32)} == set(range(32))  # every code value occurs


def test_q5_k_single_rounding_and_packer():
    """d * sc * q is exact for 5-bit codes as well (11 + 6 + 5 bits); the packer's blocks decode to within half
    a step of the input and use the fifth bit."""
    rng = np.random.default_rng(14)
    d = rng.integers(0x0400, 0x5000, 40).astype(np.uint16).view(np.float16).astype(np.float64)
    dlq = d[:, None, None] * np.arange(64)[None, :, None] * np.arange(32)[None, None, :]
    assert np.array_equal(dlq.astype(np.float32).astype(np.float64), dlq)
    w, _ = synth(15, 16, 1024, 1)
    packed = O.quantize(O.Q5_K, w)
    assert packed.shape == (16, 4 * 176)
    back = O.dequantize(O.Q5_K, packed, 1024)
    b = packed.reshape(16, 4, 176)
    dsc = NF.f16(b[:, :, 0:2])[:, :, None] * NF.unpack_scales_q4_k(b[:, :, 4:16])[0]        # step of every sub-block
    dmn = NF.f16(b[:, :, 2:4])[:, :, None] * NF.unpack_scales_q4_k(b[:, :, 4:16])[1]
    err = np.abs(back - w).reshape(16, 4, 8, 32)
    # a code is the nearest one to (x + min) / step, so the error is half a step unless the 6-bit min or scale
    # clipped the range; allow those the rounding of the two 6-bit fields
    lim = 0.5 * dsc + np.abs(dmn - (-np.minimum(w.reshape(16, 4, 8, 32).min(axis=3), 0))) + 31 * np.abs(
        dsc - (w.reshape(16, 4, 8, 32).max(axis=3).clip(0) - w.reshape(16, 4, 8, 32).min(axis=3).clip(None, 0)) / 31)
    assert (err <= lim[..., None] + 1e-7).all()
    rms = lambda e: float(np.sqrt(np.mean(e.astype(np.float64) ** 2)))
    assert rms(back - w) < 0.75 * rms(O.dequantize(O.Q4_K, O.quantize(O.Q4_K, w), 1024) - w)  # one more bit of code
    assert b[:, :, 16:48].any() and (b[:, :, 16:48] != 0xFF).any()


def test_q6_k_known_block():
    # d = 0.125 (0x3000); scale j = j - 8 (int8); code of weight e = (5*e + 3) % 64
    codes = np.array([(5 * e + 3) % 64 for e in range(256)], np.int32)
    blk = np.zeros(210, np.uint8)
    for h in range(2):
        for l in range(32):
            q = [codes[128 * h + l + 32 * t] for t in range(4)]
            blk[64 * h + l] = (q[0] & 15) | ((q[2] & 15) << 4)
            blk[64 * h + 32 + l] = (q[1] & 15) | ((q[3] & 15) << 4)
            blk[128 + 32 * h + l] = (q[0] >> 4) | ((q[1] >> 4) << 2) | ((q[2] >> 4) << 4) | ((q[3] >> 4) << 6)
    blk[192:208] = np.arange(-8, 8, dtype=np.int8).view(np.uint8)
    blk[208:210] = [0x00, 0x30]
    got = O.dequantize(O.Q6_K, blk[None, :], 256)[0]
    want = np.array([0.125 * (e // 16 - 8) * (codes[e] - 32) for e in range(256)], np.float32)
    assert np.array_equal(got, want)


def test_gptq_known_tensor():
    # K = 128 (one group), N = 8; weight (k, n) code = (k + 2n) % 16, scale_n = 2^-n, stored zero 7
    k, n = 128, 8
    q = (np.arange(k)[:, None] + 2 * np.arange(n)[None, :]) % 16
    qweight = np.zeros((k // 8, n), np.uint32)
    for kk in range(k):
        qweight[kk // 8] |= (q[kk].astype(np.uint32) << (4 * (kk % 8)))
    scales = (2.0 ** -np.arange(n)).astype(np.float16)[None, :].view(np.uint16)
    qzeros = np.array([[0x77777777]], np.uint32).view(np.int32)
    got = O.dequantize_gptq(qweight.view(np.int32), scales, qzeros)
    want = ((q - 8) * (2.0 ** -np.arange(n))[None, :]).T.astype(np.float32)
    assert np.array_equal(got, want)


# ------------------------------------------------------------------ round trips over every field value
def test_q4_k_scale_pack_unpack_all_values():
    for j in range(8):
        for a in range(64):
            sc = np.full(8, 21, np.uint8)
            mn = np.full(8, 42, np.uint8)
            sc[j] = a
            mn[j] = 63 - a
            usc, umn = O.unpack_scales_q4_k(O.pack_scales_q4_k(sc, mn))
            assert np.array_equal(usc, sc) and np.array_equal(umn, mn)
    rng = np.random.default_rng(2)
    for _ in range(500):
        sc, mn = rng.integers(0, 64, 8).astype(np.uint8), rng.integers(0, 64, 8).astype(np.uint8)
        s = O.pack_scales_q4_k(sc, mn)
        nsc, nmn = NF.unpack_scales_q4_k(s)
        assert np.array_equal(nsc, sc) and np.array_equal(nmn, mn)


def test_q6_k_every_code_in_every_position():
    """Quantiser packs and dequantiser unpacks the 4+2 bit planes consistently for all 64 codes."""
    for code in range(64):
        x = np.zeros((1, 256), np.float32)
        # super-block whose sub-block scale is exactly 1: max magnitude -32 -> scale 1, d = 1/128*128...
        x[0, :] = code - 32
        x[0, 0] = -32.0  # fixes scale = 1 for sub-block 0; other sub-blocks get scale (code-32)/-32 or similar
        packed = O.quantize(O.Q6_K, x)
        back = O.dequantize(O.Q6_K, packed, 256)
        assert np.abs(back - x).max() <= 0.51 * max(1.0, abs(code - 32)) / 31 + 1e-6


# ------------------------------------------------------------------ exactness lemma, brute force
def test_q4_0_q6_k_gptq_products_are_exact():
    """f16 d (11 bits) x small integers stays within 24 bits: fp32 evaluation order cannot matter."""
    rng = np.random.default_rng(3)
    d = np.concatenate([rng.integers(0x0400, 0x7BFF, 2000).astype(np.uint16).view(np.float16).astype(np.float64),
                        np.array([6.1e-5, 65504.0, 1.0, 1 / 3], np.float16).astype(np.float64)])
    for q in range(-8, 8):
        assert np.array_equal((d * q).astype(np.float32).astype(np.float64), d * q)
    sc = np.arange(-128, 128)
    q6 = np.arange(-32, 32)
    prod = d[:200, None, None] * sc[None, :, None] * q6[None, None, :]
    with np.errstate(over="ignore"):
        as32 = prod.astype(np.float32)
    fin = np.isfinite(as32)
    assert np.array_equal(as32[fin].astype(np.float64), prod[fin])
    step1 = (d[:200, None].astype(np.float32) * sc[None, :].astype(np.float32))  # d*sc first, as the oracle does
    assert np.array_equal(step1.astype(np.float64), d[:200, None] * sc[None, :])


def test_q4_k_single_rounding():
    """(d*sc)*q and dmin*m are exact; only the subtraction rounds, so fused and unfused agree."""
    rng = np.random.default_rng(4)
    d = rng.integers(0x0400, 0x5000, 40).astype(np.uint16).view(np.float16).astype(np.float64)
    dm = rng.integers(0x0400, 0x5000, 40).astype(np.uint16).view(np.float16).astype(np.float64)
    sc, m, q = np.arange(64), np.arange(64), np.arange(16)
    dl = d[:, None] * sc[None, :]
    assert np.array_equal(dl.astype(np.float32).astype(np.float64), dl)
    dlq = dl[:, :, None] * q[None, None, :]
    assert np.array_equal(dlq.astype(np.float32).astype(np.float64), dlq)
    ml = dm[:, None] * m[None, :]
    assert np.array_equal(ml.astype(np.float32).astype(np.float64), ml)
    # oracle value == correctly rounded exact difference, for a sample of all (sc, m, q)
    blk = np.zeros((1, 144), np.uint8)
    for trial in range(20):
        scv, mnv = rng.integers(0, 64, 8).astype(np.uint8), rng.integers(0, 64, 8).astype(np.uint8)
        blk[0, 0:2] = np.frombuffer(np.float16(d[trial]).tobytes(), np.uint8)
        blk[0, 2:4] = np.frombuffer(np.float16(dm[trial]).tobytes(), np.uint8)
        blk[0, 4:16] = O.pack_scales_q4_k(scv, mnv)
        blk[0, 16:] = rng.integers(0, 256, 128).astype(np.uint8)
        got = O.dequantize(O.Q4_K, blk, 256)[0]
        qs = blk[0, 16:].reshape(4, 32).astype(np.int64)
        qq = np.stack([qs & 15, qs >> 4], axis=1).reshape(8, 32)
        exact = d[trial] * scv.astype(np.float64)[:, None] * qq - dm[trial] * mnv.astype(np.float64)[:, None]
        assert np.array_equal(got, exact.reshape(256).astype(np.float32))


# ------------------------------------------------------------------ independent restatement on random bytes
@pytest.mark.parametrize("enc,fn", [(O.Q4_0, NF.dequant_q4_0), (O.Q4_K, NF.dequant_q4_k), (O.Q6_K, NF.dequant_q6_k),
                                    (O.Q5_K, NF.dequant_q5_k)])
def test_dequant_matches_vectorised_restatement(enc, fn):
    w, _ = synth(20 + enc, 32, 1024, 1)
    packed = O.quantize(enc, w)
    rng = np.random.default_rng(5)
    epb, bpb = O.BLOCK[enc]
    blocks = packed.reshape(-1, bpb)
    keep = {O.Q4_0: slice(0, 2), O.Q4_K: slice(0, 4), O.Q6_K: slice(208, 210), O.Q5_K: slice(0, 4)}[enc]
    rnd = rng.integers(0, 256, blocks.shape, dtype=np.uint8)
    rnd[:, keep] = blocks[:, keep]
    blocks[blocks.shape[0] // 2:] = rnd[blocks.shape[0] // 2:]  # half quantised data, half arbitrary bit patterns
    a, b = O.dequantize(enc, packed, 1024), fn(packed, 1024)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_dequant_gptq_matches_vectorised_restatement():
    w, _ = synth(30, 64, 512, 1)
    qw, sc, qz, gi = O.quantize_gptq(w)
    assert np.array_equal(gi, np.arange(512) // 128)
    assert np.all(qz.view(np.uint32) == 0x77777777)
    rng = np.random.default_rng(6)
    qw = rng.integers(-2**31, 2**31, qw.shape, dtype=np.int64).astype(np.int32)
    assert np.array_equal(O.dequantize_gptq(qw, sc, qz), NF.dequant_gptq(qw, sc, qz))


def test_gptq_act_order_group_index():
    """g_idx: (1) the plain index k // group changes nothing; (2) an act-order checkpoint dequantises to the
    sorted-order weight with its columns put back (an independent route: pack in sorted order, then permute
    the dequantised columns); (3) the vectorised restatement agrees on arbitrary bits and arbitrary group indices."""
    n, k, group = 24, 512, 64
    w, _ = synth(31, n, k, 1)
    rng = np.random.default_rng(32)
    perm = rng.permutation(k)
    qs, sc, qz, gi0 = O.quantize_gptq(np.ascontiguousarray(w[:, perm]), group)
    qz = rng.integers(-2**31, 2**31, qz.shape, dtype=np.int64).astype(np.int32)  # every zero point 1..16
    assert np.array_equal(O.dequantize_gptq(qs, sc, qz, group, g_idx=gi0), O.dequantize_gptq(qs, sc, qz, group))
    qw, gi = NF.gptq_act_order(qs, perm, group)
    assert np.array_equal(np.bincount(gi, minlength=k // group), np.full(k // group, group))
    sorted_w = O.dequantize_gptq(qs, sc, qz, group)          # [N, K] in sorted order
    want = np.empty_like(sorted_w)
    want[:, perm] = sorted_w
    got = O.dequantize_gptq(qw, sc, qz, group, g_idx=gi)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert not np.array_equal(got, O.dequantize_gptq(qw, sc, qz, group))  # the index matters
    anyg = rng.integers(0, k // group, k).astype(np.int32)
    qr = rng.integers(-2**31, 2**31, qw.shape, dtype=np.int64).astype(np.int32)
    assert np.array_equal(O.dequantize_gptq(qr, sc, qz, group, g_idx=anyg), NF.dequant_gptq(qr, sc, qz, group, g_idx=anyg))
    # matmul: fp64 sums over the dequantised weight
    a = rng.standard_normal((3, k)).astype(np.float32)
    truth = a.astype(np.float64) @ got.astype(np.float64).T
    assert np.abs(O.matmul_gptq(a, qw, sc, qz, group, f64=True, g_idx=gi) - truth).max() < 1e-12
    assert O.isclose(O.matmul_gptq(a, qw, sc, qz, group, g_idx=gi), truth, 1e-5, 2e-6).all()


def test_non_finite_and_zero_scales_propagate():
    blk = np.zeros((1, 18), np.uint8)
    blk[0, 2:] = 0x5A
    for bits, check in ((0x7C00, np.isinf), (0x7E00, np.isnan), (0x0001, np.isfinite), (0x0000, lambda v: v == 0)):
        blk[0, 0:2] = [bits & 0xFF, bits >> 8]
        out = O.dequantize(O.Q4_0, blk, 32)
        assert check(out).all()
