"""GPU parity: every kernel behind the C ABI against the CPU oracle on the same seeded inputs.

Bars: packed bytes, dequantised weights and int8 block dots bit-exact; fp32
matmul outputs within rtol 1e-3 / atol 1e-4 under the reference's symmetric
isclose (stdlib/src/math/math.mojo:1023-1030).
"""
import numpy as np
import pytest
import torch

import oracle as O
from conftest import synth
from mojo_amd import QuantizationConfig, QuantizationEncoding as QE
from mojo_amd import block_dots_q4_0, dequantize, qmatmul, qmatmul_grouped, qmatmul_rmsnorm, qmatmul_swiglu, quantize, quantize_gptq

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-3, 1e-4
ENC = {QE.Q4_0: O.Q4_0, QE.Q4_K: O.Q4_K, QE.Q6_K: O.Q6_K, QE.Q5_K: O.Q5_K}
DEV = "cuda:0"


def gpu(x):
    return torch.from_numpy(np.ascontiguousarray(x)).to(DEV)


def assert_close(got, want, what):
    got = got.detach().cpu().numpy() if isinstance(got, torch.Tensor) else got
    ok = O.isclose(got, want, RTOL, ATOL)
    if not ok.all():
        bad = np.argwhere(~ok)
        i = tuple(bad[0])
        raise AssertionError(
            f"{what}: {len(bad)}/{ok.size} outside rtol={RTOL} atol={ATOL}; first {i}: got {got[i]} want {want[i]}; "
            f"max abs err {np.abs(got - want).max()}")


def bits(x):
    return x.detach().cpu().contiguous().view(torch.uint8).numpy()


# ------------------------------------------------------------------ quantisers
@pytest.mark.parametrize("enc", [QE.Q4_0, QE.Q4_K, QE.Q6_K, QE.Q5_K])
def test_quantize_bytes_match_oracle(enc):
    w, _ = synth(3, 96, 1024, 1)
    w[5, 256:512] = 0.0  # an all-zero super-block
    w[7, :32] = 0.0
    w[9, 0:32] = -w[9, 0:32].max()  # ties in the max search
    got = quantize(enc, gpu(w)).cpu().numpy()
    want = O.quantize(ENC[enc], w)
    assert np.array_equal(got, want)


def test_quantize_q8_0_bytes_match_oracle():
    _, a = synth(4, 8, 2048, 16)
    a[3, 64:96] = 0.0
    a[2, 0:8] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.0]  # x/d lands on .5 ties when amax = 127
    got = quantize(QE.Q8_0, gpu(a)).cpu().numpy()
    assert np.array_equal(got, O.quantize_q8_0(a))


def test_quantize_gptq_matches_oracle():
    w, _ = synth(5, 64, 512, 1)
    qw, sc, qz, gi = [t.cpu().numpy() for t in quantize_gptq(gpu(w))]
    oqw, osc, oqz, ogi = O.quantize_gptq(w)
    assert np.array_equal(qw, oqw) and np.array_equal(sc.view(np.uint16), osc)
    assert np.array_equal(qz, oqz) and np.array_equal(gi, ogi)


# ------------------------------------------------------------------ dequantisers (bit-exact)
@pytest.mark.parametrize("enc", [QE.Q4_0, QE.Q4_K, QE.Q6_K, QE.Q5_K])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dequantize_bit_exact(enc, dtype):
    w, _ = synth(6, 128, 2048, 1)
    packed = O.quantize(ENC[enc], w)
    # random bytes in the code/scale fields exercise every bit pattern, fp16 fields stay finite
    rng = np.random.default_rng(1)
    noisy = packed.copy()
    epb, bpb = O.BLOCK[ENC[enc]]
    blocks = noisy.reshape(-1, bpb)
    keep = {O.Q4_0: slice(0, 2), O.Q4_K: slice(0, 4), O.Q6_K: slice(208, 210), O.Q5_K: slice(0, 4)}[ENC[enc]]
    rnd = rng.integers(0, 256, blocks.shape, dtype=np.uint8)
    rnd[:, keep] = blocks[:, keep]
    blocks[64:] = rnd[64:]
    want = O.dequantize(ENC[enc], noisy, 2048)
    got = dequantize(enc, gpu(noisy), dtype=dtype)
    if dtype == torch.float32:
        assert np.array_equal(bits(got), want.view(np.uint8).reshape(128, -1))
    else:
        assert np.array_equal(bits(got).view(np.uint16), O.f32_to_bf16(want))


def test_dequantize_gptq_bit_exact():
    w, _ = synth(7, 128, 1024, 1)
    qw, sc, qz, gi = O.quantize_gptq(w)
    want = O.dequantize_gptq(qw, sc, qz)
    cfg = QuantizationConfig()
    got = dequantize(QE.GPTQ, gpu(qw), gpu(sc.view(np.float16)), gpu(qz), gpu(gi), config=cfg)
    assert np.array_equal(bits(got), want.view(np.uint8).reshape(128, -1))
    got = dequantize(QE.GPTQ, gpu(qw), gpu(sc.view(np.float16)), gpu(qz), config=cfg)
    assert np.array_equal(bits(got), want.view(np.uint8).reshape(128, -1))


def test_dequantize_gptq_rejects_tensors_that_do_not_fit_the_config():
    """A group size smaller than the checkpoint's would index scales / qzeros past their end: refused on the host."""
    w, _ = synth(8, 64, 512, 1)
    qw, sc, qz, gi = O.quantize_gptq(w, 128)
    t = [gpu(qw), gpu(sc.view(np.float16)), gpu(qz)]
    with pytest.raises(ValueError, match="scales/qzeros"):
        dequantize(QE.GPTQ, *t, config=QuantizationConfig(group_size=64))
    with pytest.raises(TypeError, match="scales"):
        dequantize(QE.GPTQ, t[0], gpu(sc.view(np.int16)), t[2], config=QuantizationConfig())


@pytest.mark.parametrize("m", [1, 4, 64])
def test_gptq_asymmetric_checkpoint(m):
    """sym=False: zero points other than 8 in qzeros (stored value + 1), through dequantize and every matmul kernel."""
    n, k, group = 128, 1024, 128
    w, a = synth(25, n, k, m)
    a = O.bf16_to_f32(O.f32_to_bf16(a))
    qw, sc, qz, gi = O.quantize_gptq(w, group)
    rng = np.random.Generator(np.random.PCG64(26))
    qz = rng.integers(0, 2**32, size=qz.shape, dtype=np.uint64).astype(np.uint32).view(np.int32)
    cfg = QuantizationConfig(group_size=group, sym=False)
    want_w = O.dequantize_gptq(qw, sc, qz, group)
    got_w = dequantize(QE.GPTQ, gpu(qw), gpu(sc.view(np.float16)), gpu(qz), config=cfg)
    assert np.array_equal(bits(got_w), want_w.view(np.uint8).reshape(n, -1))
    truth = O.matmul_gptq(a, qw, sc, qz, group, f64=True)
    got = qmatmul(QE.GPTQ, cfg, gpu(a), gpu(qw), gpu(sc.view(np.float16)), gpu(qz), gpu(gi))
    assert_close(got, truth, f"asymmetric GPTQ m={m}")


@pytest.mark.parametrize("m,n,k,group,bf16", [(1, 200, 1024, 128, False), (3, 72, 512, 64, True), (5, 136, 1024, 128, False),
                                               (20, 64, 512, 32, False), (2, 72, 4096, 32, False)])
def test_gptq_act_order_checkpoint(m, n, k, group, bf16):
    """desc_act=True: g_idx names the group of every k in no particular order; through dequantize (bit-exact) and
    the matmul (the last shape has too many groups for the kernel's LDS table and reads scales from memory)."""
    import np_formats as NF

    w, a = synth(27, n, k, m)
    if bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    rng = np.random.Generator(np.random.PCG64(28))
    perm = rng.permutation(k)
    qs, sc, qz, _ = O.quantize_gptq(np.ascontiguousarray(w[:, perm]), group)
    qz = rng.integers(0, 2**32, size=qz.shape, dtype=np.uint64).astype(np.uint32).view(np.int32)
    qw, gi = NF.gptq_act_order(qs, perm, group)
    cfg = QuantizationConfig(group_size=group, desc_act=True, sym=False)
    want_w = O.dequantize_gptq(qw, sc, qz, group, g_idx=gi)
    got_w = dequantize(QE.GPTQ, gpu(qw), gpu(sc.view(np.float16)), gpu(qz), gpu(gi), config=cfg)
    assert np.array_equal(bits(got_w), want_w.view(np.uint8).reshape(n, -1))
    truth = O.matmul_gptq(a, qw, sc, qz, group, f64=True, g_idx=gi)
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    got = qmatmul(QE.GPTQ, cfg, lhs, gpu(qw), gpu(sc.view(np.float16)), gpu(qz), gpu(gi))
    assert_close(got, truth, f"act-order GPTQ m={m} n={n} k={k} group={group}")
    assert_close(got, O.matmul_gptq(a, qw, sc, qz, group, g_idx=gi), "act-order GPTQ against the fp32 oracle")
    with pytest.raises(TypeError):
        qmatmul(QE.GPTQ, cfg, lhs, gpu(qw), gpu(sc.view(np.float16)), gpu(qz))


# ------------------------------------------------------------------ Q4_0: integer dots and matmul
def test_block_dots_bit_exact():
    w, a = synth(0, 256, 1024, 4)
    wq, aq = O.quantize(O.Q4_0, w), O.quantize_q8_0(a)
    got = block_dots_q4_0(gpu(aq), gpu(wq)).cpu().numpy()
    assert np.array_equal(got, O.block_dots_q4_0_q8_0(aq, wq, 1024))


def test_block_dots_extremes():
    # all codes 0 (-8) against all -127 / +127, and all codes 15 (+7)
    wq = np.zeros((2, 18), np.uint8)
    wq[:, :2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    wq[1, 2:] = 0xFF
    aq = np.zeros((2, 34), np.uint8)
    aq[0, 2:] = np.int8(-127).view(np.uint8)
    aq[1, 2:] = 127
    got = block_dots_q4_0(gpu(aq), gpu(wq)).cpu().numpy()[:, :, 0]
    assert got.tolist() == [[32 * 8 * 127, -32 * 7 * 127], [-32 * 8 * 127, 32 * 7 * 127]]


def _integer_dot_case(m, n, k, one_hot, bf16, seed):
    """Inputs on which the fp32 output of the Q4_0 path IS the integer block dot: weight blocks with scale 1.0 (fp16
    0x3C00; with one_hot only block (7 row + 3) % nblocks of a row has it, the others 0.0), random nibbles; lhs
    values integers or .5 ties of magnitude <= 127 with one +-127 per 32-block, so that the Q8_0 scale is exactly 1
    and a code is round-half-away of its value.  Every partial sum is an integer below 2^24, so fp32 adds them
    exactly in any order: out[i, j] == sum_b scale[j, b] * isum[i, j, b] bit for bit."""
    rng = np.random.Generator(np.random.PCG64(seed))
    nb = k // 32
    blocks = rng.integers(0, 256, (n, nb, 18), dtype=np.uint8)
    hot = np.ones((n, nb), bool)
    if one_hot:
        hot[:] = False
        hot[np.arange(n), (7 * np.arange(n) + 3) % nb] = True
    blocks[:, :, 0] = 0
    blocks[:, :, 1] = np.where(hot, 0x3C, 0)
    wq = np.ascontiguousarray(blocks.reshape(n, nb * 18))
    a = rng.integers(-127, 128, (m, nb, 32)).astype(np.float32)
    ties = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5], np.float32)  # (all exact in bf16)
    a[:, ::3, 8:16] = ties  # x / d lands on a .5 tie in every third block
    a[:, 1::5, 16:24] = 0.0
    peak = rng.integers(0, 8, (m, nb))
    sign = rng.choice(np.array([-127.0, 127.0], np.float32), (m, nb))
    np.put_along_axis(a, peak[:, :, None], sign[:, :, None], axis=2)
    a = np.ascontiguousarray(a.reshape(m, k))
    aq = O.quantize_q8_0(a)
    assert (aq.reshape(m, nb, 34)[:, :, :2] == np.array([0x00, 0x3C], np.uint8)).all()  # every activation scale is 1.0
    isum = O.block_dots_q4_0_q8_0(aq, wq, k).astype(np.int64)
    want = (isum * hot[None, :, :]).sum(axis=2)
    assert np.abs(want).max() < 2**24
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    return lhs, gpu(wq), want.astype(np.float32)


# (m, n, k) -> kernel: 1, 4: the decode kernel that quantises the lhs itself; K = 8224: the first-version decode kernel
# behind the stand-alone quantiser; 5, 16: small-batch int8 matrix-core kernel, which also serves 33, 64 and 65 rows in
# passes of 16 (a last pass of one row) and 3 rows on a K past 8192; 9 and 40 with K % 256 != 0: the 16-row-tile kernel
# (1, 3 tiles per group); 256: the plane GEMM on the fp16 matrix cores
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("one_hot", [True, False])
@pytest.mark.parametrize("m,n,k", [(1, 200, 4096), (4, 200, 4096), (2, 70, 8224), (5, 200, 4096), (16, 200, 4096),
                                   (9, 72, 1056), (33, 200, 1024), (64, 72, 4096), (65, 200, 1024), (256, 136, 4096),
                                   (3, 72, 16384), (40, 72, 1056), (1, 200, 14336)])
def test_q4_0_production_kernels_give_the_integer_block_dots(m, n, k, one_hot, bf16):
    """The int8 block dots of every Q4_0 matmul kernel, read off its fp32 output, equal the oracle's bit for bit
    (Q8_0 codes with .5 ties included)."""
    lhs, wq, want = _integer_dot_case(m, n, k, one_hot, bf16, seed=31 + m)
    got = qmatmul(QE.Q4_0, None, lhs, wq).cpu().numpy()
    assert np.array_equal(got, want), f"{(got != want).sum()} of {got.size} outputs differ from the integer dots"


@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (16, 1024, 4096), (5, 130, 64), (3, 7, 32), (33, 64, 256)])
def test_q4_0_matmul(m, n, k):
    w, a = synth(0, n, k, m)
    wq = O.quantize(O.Q4_0, w)
    want = O.matmul_q4_0(a, wq)
    got = qmatmul(QE.Q4_0, None, gpu(a), gpu(wq))
    assert_close(got, want, f"Q4_0 {m}x{n}x{k}")


@pytest.mark.parametrize("m,n,k,lhs_bf16", [(2, 1000, 8192, False), (4, 300, 4096, True), (1, 5001, 2048, False),
                                            (1, 70000, 256, False), (3, 9, 4128, False), (2, 64, 8224, True),
                                            (4, 33, 8192, False), (1, 4099, 14336, False), (1, 300, 11008, True),
                                            (1, 70, 14528, False), (1, 130, 14560, True), (1, 9, 8224, False)])
def test_q4_0_decode_shapes(m, n, k, lhs_bf16):
    """Q4_0 decode: rows at every 2-byte alignment, K up to 8192 in the kernel that quantises the lhs itself
    (more rows on a longer K through the Q8_0 planes), many rows per wavefront, bf16 lhs.  One lhs row: that kernel up to
    K = 14528 with six or eight blocks per lane (8224, 11008 / 14336, 14528; 14560 is past it)."""
    w, a = synth(52, n, k, m)
    if lhs_bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q4_0, w)
    want = O.matmul_q4_0(a, wq)
    got = qmatmul(QE.Q4_0, None, gpu(a).to(torch.bfloat16) if lhs_bf16 else gpu(a), gpu(wq))
    assert_close(got, want, f"Q4_0 decode {m}x{n}x{k} bf16={lhs_bf16}")


@pytest.mark.parametrize("m,n,k,lhs_bf16", [(16, 5000, 4096, False), (9, 300, 512, False), (12, 64, 14336, True),
                                            (5, 4100, 256, False), (16, 16400, 2048, True), (37, 300, 1024, False),
                                            (64, 5000, 4096, True), (81, 4100, 2048, False), (3, 200, 14336, False),
                                            (2, 130, 16384, True), (3, 200, 5120, False), (4, 130, 8192, True)])
def test_q4_0_small_batch(m, n, k, lhs_bf16):
    """5..16 lhs rows, K a multiple of 256: several 16-row tiles per workgroup, ragged last tile, groups of K in
    which only some wavefronts have a share.  More rows go through the same kernel in passes of 16 while that beats making
    the planes (37: a last pass of five rows; 81: of one), and so do 2..4 rows on a K past 8192 and 3, 4 rows on one past 4096."""
    w, a = synth(53, n, k, m)
    if lhs_bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q4_0, w)
    want = O.matmul_q4_0(a, wq)
    got = qmatmul(QE.Q4_0, None, gpu(a).to(torch.bfloat16) if lhs_bf16 else gpu(a), gpu(wq))
    assert_close(got, want, f"Q4_0 small batch {m}x{n}x{k} bf16={lhs_bf16}")


# ------------------------------------------------------------------ Q4_K / Q6_K with fp32 activations
@pytest.mark.parametrize("enc", [QE.Q4_K, QE.Q6_K, QE.Q5_K])
@pytest.mark.parametrize("m,n,k", [(1, 1024, 4096), (4, 512, 4096), (16, 256, 2048), (3, 5, 256), (2, 66, 14336),
                                   (20, 64, 512)])
def test_kquant_matmul_f32(enc, m, n, k):
    w, a = synth(3, n, k, m)
    wq = O.quantize(ENC[enc], w)
    want = O.matmul_f32(ENC[enc], a, wq)
    truth = O.matmul_f64(ENC[enc], a, wq)
    got = qmatmul(enc, None, gpu(a), gpu(wq))
    assert_close(got, want, f"{enc.name} {m}x{n}x{k} vs fp32 oracle")
    assert_close(got, truth, f"{enc.name} {m}x{n}x{k} vs fp64 truth")


@pytest.mark.parametrize("enc", [QE.Q4_K, QE.Q6_K, QE.Q5_K])
def test_kquant_matmul_bf16_lhs(enc):
    w, a = synth(5, 256, 1024, 4)
    a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(ENC[enc], w)
    want = O.matmul_f32(ENC[enc], a, wq)
    got = qmatmul(enc, None, gpu(a).to(torch.bfloat16), gpu(wq))
    assert_close(got, want, f"{enc.name} bf16 lhs")


@pytest.mark.parametrize("m,n,k,bf16", [(1, 4099, 4096, False), (1, 1030, 4096, True), (3, 777, 14336, False), (1, 130, 32768, False),
                                        (4, 2050, 1280, True), (7, 300, 8192, False), (1, 2100, 28672, False)])
def test_q5_k_decode_shapes(m, n, k, bf16):
    """Q5_K through its kernel's variants: activations in registers (one row, K <= 4096), from the LDS copy,
    several groups of 16 super-blocks with a partial last one, row counts that leave wavefronts unequal work,
    and the random bit patterns of the dequantiser test (every fifth-bit / nibble combination)."""
    w, a = synth(41, n, k, m)
    if bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q5_K, w)
    rng = np.random.default_rng(42)
    blocks = wq.reshape(-1, 176)
    rnd = rng.integers(0, 256, blocks.shape, dtype=np.uint8)
    rnd[:, 0:4] = blocks[:, 0:4]
    blocks[::3] = rnd[::3]
    truth = O.matmul_f64(O.Q5_K, a, wq)
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    got = qmatmul(QE.Q5_K, None, lhs, gpu(wq))
    assert_close(got, truth, f"Q5_K {m}x{n}x{k} bf16={bf16}")


@pytest.mark.parametrize("m,n,k,bf16", [(5, 16, 4096, False), (8, 1000, 4096, True), (16, 4099, 4096, False), (16, 530, 4096, True),
                                        (12, 9000, 512, False), (7, 300, 8192, False), (16, 77, 14336, True), (9, 40, 32768, False),
                                        (20, 130, 4608, True), (32, 72, 1024, False), (4, 4200, 14336, False), (2, 2100, 14336, False),
                                        (20, 1100, 8192, False)])
def test_q5_k_small_batch_matrix_core_kernel(m, n, k, bf16):
    """Q5_K with 5..32 lhs rows, K a multiple of 512: weight rows decoded once for the lhs rows of a pass (codes as exact fp16
    integers, one matrix-core instruction per 32-weight sub-block, the min term through the lhs sub-block sums); 8-row passes
    (fp32) and 16-row passes (bf16: no residual rows), tiles that end past the matrix, more tiles than workgroups, K in
    rounds of 4096 columns, side by side in the grid and added by a launch of their own (4200 weight rows: several tiles per
    workgroup and round), with a last round in which only some wavefronts have a share; a third of the blocks carry random
    bytes (every fifth-bit / nibble / scale combination); rows of very different magnitude share a pass."""
    w, a = synth(44, n, k, m)
    a[m - 1] *= 10.0  # (not more: the random blocks make large weights, and fp32 sums of 1e4 carry 1e-3 of noise)
    a[0] *= 1e-4
    a[1, :512] *= 1e-3
    if bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q5_K, w)
    rng = np.random.default_rng(45)
    blocks = wq.reshape(-1, 176)
    rnd = rng.integers(0, 256, blocks.shape, dtype=np.uint8)
    rnd[:, 0:4] = blocks[:, 0:4]
    blocks[::3] = rnd[::3]
    truth = O.matmul_f64(O.Q5_K, a, wq)
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    got = qmatmul(QE.Q5_K, None, lhs, gpu(wq))
    assert_close(got, truth, f"Q5_K {m}x{n}x{k} bf16={bf16} vs fp64 truth")
    # (against the fp32 oracle only where cancellation leaves something to compare: both are fp32 sums in different orders)
    want = O.matmul_f32(O.Q5_K, a, wq)
    big = np.abs(truth) > 1e-3 * np.abs(truth).max(axis=1, keepdims=True)
    assert O.isclose(got.cpu().numpy()[big], want[big], RTOL, ATOL).all()


@pytest.mark.parametrize("m,n,k", [(1, 256, 1024), (4, 520, 512), (16, 64, 4096), (18, 64, 256), (1, 14336, 4096), (3, 200, 14336),
                                   (1, 4096, 14336), (2, 1000, 8192), (1, 8, 4096), (2, 4104, 1024)])
def test_gptq_matmul(m, n, k):
    w, a = synth(5, n, k, m)
    qw, sc, qz, gi = O.quantize_gptq(w)
    want = O.matmul_gptq(a, qw, sc, qz)
    got = qmatmul(QE.GPTQ, QuantizationConfig(), gpu(a), gpu(qw), gpu(sc.view(np.float16)), gpu(qz), gpu(gi))
    assert_close(got, want, f"GPTQ {m}x{n}x{k}")


@pytest.mark.parametrize("enc", [QE.Q4_0, QE.Q4_K, QE.Q5_K, QE.Q6_K])
@pytest.mark.parametrize("m", [1, 4, 8, 40])
def test_non_finite_lhs_values_stay_in_their_row(enc, m):
    """A NaN in the lhs gives the oracle's outputs, NaN for NaN (Q4_0: the Q8_0 quantiser's maximum search drops it on
    both sides).  An infinity makes its whole output row non-finite on both sides; the kind may differ: the K-quant
    kernels add the offset / min terms as separate sums, so they report NaN (inf - inf) where the element-wise
    oracle reports +-inf.  Rows without such a value are not touched by it."""
    w, a = synth(5, 64, 2048, m)
    wq = O.quantize(ENC[enc], w)
    for val in (np.nan, np.inf, -np.inf):
        a2 = a.copy()
        a2[0, 300] = val
        want = O.matmul_q4_0(a2, wq) if enc == QE.Q4_0 else O.matmul_f32(ENC[enc], a2, wq)
        got = qmatmul(enc, None, gpu(a2), gpu(wq)).cpu().numpy()
        assert np.array_equal(np.isfinite(got[0]), np.isfinite(want[0])), f"{enc.name} m={m} {val}: finiteness of the row differs"
        if np.isnan(val):
            assert np.array_equal(np.isnan(got[0]), np.isnan(want[0]))
        fin = np.isfinite(want[0])
        assert O.isclose(got[0][fin], want[0][fin], RTOL, ATOL).all()
        if m > 1:
            assert_close(got[1:], want[1:], f"{enc.name} m={m}: rows next to a non-finite one")


@pytest.mark.parametrize("m,n,k,group,bf16", [
    (2, 72, 256, 128, False), (5, 1000, 1024, 128, False), (8, 8, 4096, 64, False), (13, 136, 4096, 256, True),
    (16, 520, 8192, 128, False), (16, 200, 14336, 128, True), (7, 264, 4352, 64, False), (3, 2048, 2048, 256, True),
    (33, 96, 4096, 128, False), (1, 264, 14336, 128, True), (1, 200, 8448, 64, False), (2, 136, 12288, 128, False)])
def test_gptq_small_batch(m, n, k, group, bf16):
    """2 to 16 lhs rows (and 33 as passes) through the matrix-core small-batch kernel: one to sixteen wavefronts of
    256 k each, K beyond 4096 as launches that add to the output (8192 = 2 x 16, 14336 = 3 x 16 + 8, 4352 = 16 + 1
    wavefronts), ragged N, N of eight columns, arbitrary zero points, lhs rows of very different magnitude.  On a K
    past 8192 the kernel also serves one row and two fp32 rows (the column kernel walks such a K with one workgroup
    per 64 columns)."""
    w, a = synth(81, n, k, m)
    a[0] *= 1e-6
    a[m - 1] *= 3e4
    if m > 2:
        a[1, : k // 2] = 0.0
    if bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    qw, sc, qz, gi = O.quantize_gptq(w, group)
    rng = np.random.Generator(np.random.PCG64(82))
    qz = rng.integers(0, 2**32, size=qz.shape, dtype=np.uint64).astype(np.uint32).view(np.int32)
    truth = O.matmul_gptq(a, qw, sc, qz, group, f64=True)
    cfg = QuantizationConfig(group_size=group, sym=False)
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    got = qmatmul(QE.GPTQ, cfg, lhs, gpu(qw), gpu(sc.view(np.float16)), gpu(qz), gpu(gi))
    assert_close(got, truth, f"GPTQ small batch {m}x{n}x{k} group={group} bf16={bf16}")


@pytest.mark.parametrize("m,n,k,bf16", [(13, 64, 14336, False), (16, 520, 8192, True), (9, 33, 4352, False), (12, 1, 4608, True),
                                        (16, 100, 28672, False), (5, 72, 8192, True)])
def test_q4_k_small_batch_k_chunks(m, n, k, bf16):
    """9 to 16 lhs rows (from 5 with a bf16 lhs), at most 4096 weight rows and K beyond 4096: the small-batch kernel that cuts K across
    workgroups (2 x 16, 4 x 14, 2 x 9 with an idle wavefront, 2 x 9 and 7 x 16 super-blocks), partial sums through the
    workspace; a third of the rows carry arbitrary bit patterns, lhs rows of very different magnitude."""
    w, a = synth(95, n, k, m)
    a[0] *= 1e-5
    a[m - 1] *= 1e4
    if bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    blocks = O.quantize(O.Q4_K, w).reshape(n, k // 256, 144)
    rng = np.random.Generator(np.random.PCG64(96))
    blocks[::3] = rng.integers(0, 256, size=blocks[::3].shape, dtype=np.uint8)
    blocks[::3, :, 0:2] = np.frombuffer(np.float16(0.001).tobytes(), dtype=np.uint8)
    blocks[::3, :, 2:4] = np.frombuffer(np.float16(0.0007).tobytes(), dtype=np.uint8)
    wq = np.ascontiguousarray(blocks.reshape(n, -1))
    truth = O.matmul_f64(O.Q4_K, a, wq)
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    got = qmatmul(QE.Q4_K, None, lhs, gpu(wq))
    assert_close(got, truth, f"Q4_K small batch, K chunks {m}x{n}x{k} bf16={bf16}")


@pytest.mark.parametrize("m,n,k,bf16", [(4, 4090, 14336, False), (8, 2048, 16384, True), (3, 1000, 14336, False), (8, 4096, 8192, False),
                                        (2, 1360, 12288, True)])
def test_q4_k_small_batch_groups_of_k_over_the_grid(m, n, k, bf16):
    """2 to 8 lhs rows, few 16-row tiles and a K beyond 4096, where one workgroup per (share of the tiles, group of 4096
    columns) fills the part: every workgroup converts the lhs of its group once, the groups' results go through the
    workspace and a launch of their own adds them in group order (64 x 4 workgroups of 4 tiles with a ragged last tile, 64 x 4
    of 2, 63 x 4 of 1, 128 x 2 with eight fp32 rows, 85 x 3); lhs rows of very different magnitude."""
    w, a = synth(97, n, k, m)
    a[0] *= 1e-4
    a[m - 1] *= 8.0  # (not more: of thousands of fp32 sums over 14336 terms some cancel to where the bar is the terms' rounding)
    if bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q4_K, w)
    want = O.matmul_f32(O.Q4_K, a, wq)
    truth = O.matmul_f64(O.Q4_K, a, wq)
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    got = qmatmul(QE.Q4_K, None, lhs, gpu(wq))
    assert_close(got, want, f"Q4_K small batch, groups of K {m}x{n}x{k} bf16={bf16} vs fp32 oracle")
    assert_close(got, truth, f"Q4_K small batch, groups of K {m}x{n}x{k} bf16={bf16} vs fp64 truth")


@pytest.mark.parametrize("m", [4, 16, 64])
def test_q4_k_unit_sub_block_scales_long_k(m):
    """Q4_K rows whose 6-bit scales and mins are all 1, K = 14336, fp32 lhs, through the matrix-core kernels: the
    operand sc * q is then at most 15, and held as the fp16 subnormal sc * q * 2^-24 the matrix cores dropped low
    product bits towards minus infinity (mean error -2e-5 to -5e-5 here).  Held as sc * q * 2^-18 there is none."""
    n, k = 64, 14336
    rng = np.random.Generator(np.random.PCG64(93))
    blocks = rng.integers(0, 256, size=(n, k // 256, 144), dtype=np.uint8)
    blocks[:, :, 4:12] = 1      # scales and mins of sub-blocks 0..3 (and zero top bits for 4..7)
    blocks[:, :, 12:16] = 0x11  # low nibbles of the scales and mins of sub-blocks 4..7
    d = np.full((n, k // 256, 1), 0.02 / 7.5, dtype=np.float16)
    blocks[:, :, 0:2] = d.view(np.uint8)
    blocks[:, :, 2:4] = d.view(np.uint8)
    wq = blocks.reshape(n, -1)
    a = rng.standard_normal((m, k), dtype=np.float32)
    truth = O.matmul_f64(O.Q4_K, a, wq)
    got = qmatmul(QE.Q4_K, None, gpu(a), gpu(wq)).cpu().numpy()
    assert_close(got, truth, f"Q4_K unit scales {m}x{n}x{k}")
    assert abs(float((got - truth).mean())) < 3e-6


@pytest.mark.parametrize("m,bf16,bound", [(5, False, 5e-6), (5, True, 5e-6), (16, True, 5e-6), (64, True, 3e-5), (1024, True, 3e-5), (1024, False, 1.5e-5)])
def test_gptq_long_k_mean_error(m, bf16, bound):
    """K = 14336 with unit-size activations: the mean of (result - fp64 truth) over all outputs stays small.  The matrix
    cores cut the low bits of products of fp16 subnormals towards minus infinity; with the non-negative GPTQ codes held
    as q * 2^-24 that was a bias of 6e-5 (small-batch kernel) to 2e-4 (GEMM, fp32 lhs) at this K, more than the absolute
    tolerance.  The small-batch kernel now holds the codes at the top of the subnormal's mantissa: no measurable bias.
    The GEMM keeps them low for a bf16 lhs (short products: 1.5e-5) and, for an fp32 lhs, moves them two bits up and
    runs the residual plane as a launch of its own (6e-6).  (With N = 64 the GEMM, cut into K shares, is taken from 33 rows on.)"""
    n, k = 64, 14336
    w, a = synth(91, n, k, m)
    if bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    qw, sc, qz, gi = O.quantize_gptq(w)
    truth = O.matmul_gptq(a, qw, sc, qz, f64=True)
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    got = qmatmul(QE.GPTQ, QuantizationConfig(), lhs, gpu(qw), gpu(sc.view(np.float16)), gpu(qz), gpu(gi)).cpu().numpy()
    assert_close(got, truth, f"GPTQ {m}x{n}x{k} bf16={bf16}")
    assert abs(float((got - truth).mean())) < bound


@pytest.mark.parametrize("m,n,k,group,bf16", [(1, 264, 1024, 32, False), (2, 72, 2048, 64, True), (4, 136, 4096, 256, False),
                                               (1, 64, 28672, 128, False), (3, 8, 512, 128, False), (1, 128, 480, 96, False)])
def test_gptq_decode_group_sizes(m, n, k, group, bf16):
    """Group sizes 32, 64, 96, 128 and 256 through the decode kernel (4 or 16 packed rows per inner step), a long K,
    N of eight columns, arbitrary zero points."""
    w, a = synth(71, n, k, m)
    if bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    qw, sc, qz, gi = O.quantize_gptq(w, group)
    rng = np.random.Generator(np.random.PCG64(72))
    qz = rng.integers(0, 2**32, size=qz.shape, dtype=np.uint64).astype(np.uint32).view(np.int32)  # any zero point
    truth = O.matmul_gptq(a, qw, sc, qz, group, f64=True)
    cfg = QuantizationConfig(group_size=group, sym=False)
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    got = qmatmul(QE.GPTQ, cfg, lhs, gpu(qw), gpu(sc.view(np.float16)), gpu(qz), gpu(gi))
    assert_close(got, truth, f"GPTQ decode {m}x{n}x{k} group={group}")


def test_leading_dims_broadcast():
    w, a = synth(8, 64, 512, 6)
    wq = O.quantize(O.Q4_K, w)
    want = O.matmul_f32(O.Q4_K, a, wq).reshape(2, 3, 64)
    got = qmatmul(QE.Q4_K, None, gpu(a).reshape(2, 3, 512), gpu(wq))
    assert got.shape == (2, 3, 64)
    assert_close(got, want, "leading dims")


# ------------------------------------------------------------------ Q4_K decode (one lhs row)
@pytest.mark.parametrize("n,k,lhs_bf16", [(1, 256, False), (7, 512, True), (70000, 256, False), (129, 4096, False),
                                          (300, 4352, True), (50, 8192, False), (33, 9984, False), (40, 16384, True),
                                          (12, 16640, False), (5000, 3840, False), (600, 18944, False), (70, 24576, True),
                                          (9, 33024, False)])
def test_q4_k_decode_shapes(n, k, lhs_bf16):
    """One lhs row: rows cut into 1, 2, 4 or 8 parts (K up to about 28000, as long as the staged lhs fits the LDS; longer
    rows take the streaming kernel), parts that do not fill a wavefront, fewer rows than wavefronts, many rows per wavefront."""
    w, a = synth(23, n, k, 1)
    if lhs_bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q4_K, w)
    want = O.matmul_f32(O.Q4_K, a, wq)
    truth = O.matmul_f64(O.Q4_K, a, wq)
    got = qmatmul(QE.Q4_K, None, gpu(a).to(torch.bfloat16) if lhs_bf16 else gpu(a), gpu(wq))
    assert_close(got, want, f"Q4_K decode 1x{n}x{k} vs fp32 oracle")
    assert_close(got, truth, f"Q4_K decode 1x{n}x{k} vs fp64 truth")


# ------------------------------------------------------------------ Q4_K small batch (2..16 lhs rows)
@pytest.mark.parametrize("m,n,k,lhs_bf16", [(2, 9000, 1024, False), (4, 8200, 4608, False), (7, 4100, 2048, True),
                                            (8, 6000, 4608, False), (5, 300, 256, False), (12, 5000, 1280, True),
                                            (12, 5000, 1280, False), (16, 4500, 4608, False)])
def test_q4_k_small_batch_many_tiles(m, n, k, lhs_bf16):
    """Several 16-row tiles per workgroup, ragged last tile, groups of K with one or two super-blocks per wavefront."""
    w, a = synth(21, n, k, m)
    if lhs_bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q4_K, w)
    want = O.matmul_f32(O.Q4_K, a, wq)
    truth = O.matmul_f64(O.Q4_K, a, wq)
    lhs = gpu(a).to(torch.bfloat16) if lhs_bf16 else gpu(a)
    got = qmatmul(QE.Q4_K, None, lhs, gpu(wq))
    assert_close(got, want, f"Q4_K small batch {m}x{n}x{k} vs fp32 oracle")
    assert_close(got, truth, f"Q4_K small batch {m}x{n}x{k} vs fp64 truth")


@pytest.mark.parametrize("m", [3, 8])
def test_q4_k_small_batch_wide_range_lhs(m):
    """Rows and 256-column blocks of very different magnitude: the power-of-two scaling per row and block keeps the
    fp16 operands in range, and what each block contributes keeps its relative precision."""
    n, k = 200, 2048
    w, a = synth(22, n, k, m)
    a *= np.logspace(-5, 4, m, dtype=np.float32)[:, None]
    a *= np.repeat(np.logspace(-3, 3, k // 256, dtype=np.float32), 256)[None, :]
    wq = O.quantize(O.Q4_K, w)
    truth = O.matmul_f64(O.Q4_K, a, wq)
    got = qmatmul(QE.Q4_K, None, gpu(a), gpu(wq)).cpu().numpy()
    scale = np.abs(truth).max(axis=1, keepdims=True)
    assert np.all(np.abs(got - truth) <= 1e-4 * scale + 1e-3 * np.abs(truth))


# ------------------------------------------------------------------ Q4_K with Q8_K-quantised activations
def test_quantize_q8_k_bytes_match_oracle():
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((9, 1024)) * rng.uniform(1e-3, 40.0, (9, 1))).astype(np.float32)
    x[1, 256:512] = 0.0
    x[2, 3], x[2, 200] = -55.0, 55.0
    x[2, :256] = np.clip(x[2, :256], -55, 55)
    x[3, 0], x[3, 1:7] = 127.0, [0.5, 1.5, 2.5, -0.5, -1.5, -2.5]
    x[3, 7:256] = np.clip(x[3, 7:256], -100, 100)
    assert np.array_equal(bits(quantize(QE.Q8_K, gpu(x))), O.quantize_q8_k(x))


@pytest.mark.parametrize("m,n,k,lhs_bf16", [(1, 1000, 4096, False), (4, 300, 4096, False), (2, 129, 14336, True),
                                            (3, 5000, 512, False), (1, 70, 16384, False), (7, 64, 1024, False),
                                            (4, 40, 8192, True), (1, 3, 256, False)])
def test_q4_k_matmul_with_q8_k_activations(m, n, k, lhs_bf16):
    """The integer-activation treatment against its own oracle, at a tolerance ten times tighter than the parity bar
    (only fp32 summation order differs); and it is not the floating-point treatment."""
    w, a = synth(71, n, k, m)
    if lhs_bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q4_K, w)
    want = O.matmul_q4_k_act_q8_k(a, wq)
    lhs = gpu(a).to(torch.bfloat16) if lhs_bf16 else gpu(a)
    got = qmatmul(QE.Q4_K, None, lhs, gpu(wq), act_q8k=True).cpu().numpy()
    assert O.isclose(got, want, 1e-4, 1e-5).all(), f"max abs err {np.abs(got - want).max()}"
    if n * m >= 64 and k >= 1024:
        assert not O.isclose(got, O.matmul_f32(O.Q4_K, a, wq), 1e-4, 1e-5).all()


@pytest.mark.parametrize("enc,m,n,k,lhs_bf16", [
    (QE.Q6_K, 1, 1000, 4096, False), (QE.Q6_K, 4, 130, 2048, True), (QE.Q6_K, 16, 64, 14336, False), (QE.Q6_K, 100, 257, 1024, False),
    (QE.Q5_K, 1, 515, 4096, False), (QE.Q5_K, 3, 70, 8192, True), (QE.Q5_K, 48, 130, 768, False),
    (QE.Q4_K, 5, 300, 4096, False), (QE.Q4_K, 16, 96, 14336, True), (QE.Q4_K, 300, 520, 1024, False), (QE.Q4_K, 2, 40, 20480, False)])
def test_kquant_matmul_with_q8_k_activations(enc, m, n, k, lhs_bf16):
    """Q8_K activations for every K-quant and row count: where no kernel takes the integer sub-block dots itself, the
    quantised activations go through the floating-point kernels as d8 * code, which differs from the integer treatment
    (the oracle's) only by fp32 summation; and the result is not the unquantised-activation one."""
    w, a = synth(73, n, k, m)
    if lhs_bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(ENC[enc], w)
    want = O.matmul_kquant_act_q8_k(ENC[enc], a, wq)
    lhs = gpu(a).to(torch.bfloat16) if lhs_bf16 else gpu(a)
    got = qmatmul(enc, None, lhs, gpu(wq), act_q8k=True).cpu().numpy()
    assert O.isclose(got, want, 1e-4, 1e-5).all(), f"max abs err {np.abs(got - want).max()}"
    if n * m >= 64 and k >= 1024:
        assert not O.isclose(got, O.matmul_f32(ENC[enc], a, wq), 1e-4, 1e-5).all()


def _kquant_integer_case(enc, m, n, k, bf16, seed):
    """Inputs on which the fp32 output of the Q8_K-activation path IS a sum of the integer block sums: weight blocks of random
    bytes with d = 1.0 (and dmin = 1.0; fp16 0x3C00), scale fields kept small (6-bit scales and mins below 16, Q6_K's int8
    scales in [-8, 7]); lhs values small integers with one +-127 per 256-block, so that every Q8_K scale is +-1 and a code is
    its value (or minus it).  Then out[i, j] == sum_b d8[i, b] * (isum[i, j, b] - msum[i, j, b]), every term and partial sum an
    integer below 2^24, which fp32 adds exactly in any order."""
    rng = np.random.Generator(np.random.PCG64(seed))
    nb = k // 256
    bpb = {QE.Q4_K: 144, QE.Q5_K: 176, QE.Q6_K: 210}[enc]
    blocks = rng.integers(0, 256, (n, nb, bpb), dtype=np.uint8)
    one = np.array([0x00, 0x3C], np.uint8)
    if enc == QE.Q6_K:
        blocks[:, :, 192:208] = rng.integers(-8, 8, (n, nb, 16)).astype(np.int8).view(np.uint8)
        blocks[:, :, 208:210] = one
    else:
        blocks[:, :, 0:2] = one
        blocks[:, :, 2:4] = one
        blocks[:, :, 4:16] &= 0x0F  # scales / mins of sub-blocks 0..3 below 16; 4..7 keep their low four bits only
    wq = np.ascontiguousarray(blocks.reshape(n, nb * bpb))
    a = rng.integers(-7, 8, (m, nb, 256)).astype(np.float32)
    a[:, 1::3, 40:80] = 0.0
    peak = rng.integers(0, 256, (m, nb))
    sign = rng.choice(np.array([-127.0, 127.0], np.float32), (m, nb))
    np.put_along_axis(a, peak[:, :, None], sign[:, :, None], axis=2)
    a = np.ascontiguousarray(a.reshape(m, k))
    aq = O.quantize_q8_k(a)
    d8 = aq.reshape(m, nb, 292)[:, :, :4].copy().view(np.float32).reshape(m, nb)
    assert (np.abs(d8) == 1.0).all()
    isum, msum = O.block_sums_kquant_q8_k(ENC[enc], aq, wq, k)
    terms = d8[:, None, :].astype(np.int64) * (isum.astype(np.int64) - msum.astype(np.int64))
    assert np.abs(np.cumsum(np.abs(terms), axis=2)).max() < 2**24
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    return lhs, gpu(wq), terms.sum(axis=2).astype(np.float32)


# rows 1..4: one pass of the integer kernels (Q4_K quantises its lhs in the kernel, Q5_K / Q6_K read Q8_K planes made once
# per call); 7, 16: passes of four; K = 256: a single block; 2304 / 1280: ragged groups of 16 / 4 super-blocks
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("enc,m,n,k", [(QE.Q6_K, 1, 200, 1024), (QE.Q6_K, 4, 130, 256), (QE.Q6_K, 7, 64, 1280), (QE.Q6_K, 16, 33, 512),
                                       (QE.Q5_K, 1, 200, 1024), (QE.Q5_K, 3, 130, 256), (QE.Q5_K, 7, 64, 2304), (QE.Q5_K, 16, 33, 512),
                                       (QE.Q4_K, 2, 200, 1024), (QE.Q4_K, 7, 64, 2304), (QE.Q4_K, 16, 33, 256)])
def test_kquant_production_kernels_give_the_integer_block_sums(enc, m, n, k, bf16):
    """The integer sub-block sums of the Q8_K-activation kernels (QMM_FLAG_ACT_Q8K, up to 16 lhs rows), read off the fp32 output,
    equal the oracle's block by block sums bit for bit."""
    lhs, wq, want = _kquant_integer_case(enc, m, n, k, bf16, seed=51 + m)
    got = qmatmul(enc, None, lhs, wq, act_q8k=True).cpu().numpy()
    assert np.array_equal(got, want), f"{(got != want).sum()} of {got.size} outputs differ from the integer sums"


@pytest.mark.parametrize("enc,m", [(QE.Q6_K, 8), (QE.Q4_K, 8), (QE.Q5_K, 3), (QE.Q4_K, 2)])
def test_q8_k_activations_with_bf16_output(enc, m):
    """Both flags in one call: the bf16 result is the rounding of the fp32 result of the same call (the Q4_K integer kernel
    for up to four rows, the fp32 round trip of the lhs otherwise), also through the static scratch."""
    n, k = 300, 2048
    w, a = synth(74, n, k, m)
    wq = O.quantize(ENC[enc], w)
    f32 = qmatmul(enc, None, gpu(a), gpu(wq), act_q8k=True)
    want = O.f32_to_bf16(f32.cpu().numpy())
    for static in (False, True):
        got = qmatmul(enc, None, gpu(a), gpu(wq), act_q8k=True, out_dtype=torch.bfloat16, static_scratch=static)
        assert got.dtype == torch.bfloat16
        assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), want), (enc, m, static)


def test_q8_k_activations_only_for_k_quants():
    w, a = synth(72, 8, 256, 1)
    with pytest.raises(NotImplementedError):
        qmatmul(QE.Q4_0, None, gpu(a), gpu(O.quantize(O.Q4_0, w)), act_q8k=True)


# ------------------------------------------------------------------ matrices that share their lhs
@pytest.mark.parametrize("enc,m,k,ns,lhs_bf16", [(QE.Q4_K, 1, 4096, (512, 130, 130), False), (QE.Q4_K, 1, 14336, (300, 77), True),
                                                 (QE.Q4_K, 1, 512, (9000, 1, 17, 4100), False),
                                                 (QE.Q4_K, 3, 1024, (64, 200), False), (QE.Q4_K, 4, 4096, (4100, 130, 130), False),
                                                 (QE.Q4_K, 4, 14336, (300, 77), False), (QE.Q4_K, 2, 8192, (1024, 1500, 40), True),
                                                 (QE.Q4_K, 8, 2304, (20, 33, 7, 50), True), (QE.Q4_K, 12, 512, (300, 17), False),
                                                 (QE.Q6_K, 1, 1024, (96, 40), False),
                                                 (QE.Q4_0, 2, 256, (33, 64, 5), False), (QE.Q4_K, 1, 256, (8, 8, 8, 8, 8), False)])
def test_grouped_matmul_equals_separate_calls(enc, m, k, ns, lhs_bf16):
    """q | k | v and gate | up style groups: the one-launch paths (Q4_K, up to four matrices, 1..16 lhs rows) and the
    per-matrix path give what qmatmul gives on each matrix, bit for bit, and agree with the oracle.  One exception: a separate
    call with 2..8 rows on a matrix of few tiles and a K beyond 4096 (here 2 x 1500 x 8192) cuts K over the grid and adds the
    parts in another order than the grouped launch, which walks K inside each workgroup: equal to fp32 rounding there."""
    ws, a = [], None
    for j, n in enumerate(ns):
        w, a = synth(60 + j, n, k, m)
        ws.append(O.quantize(ENC[enc], w))
    if lhs_bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    lhs = gpu(a).to(torch.bfloat16) if lhs_bf16 else gpu(a)
    rhs = [gpu(w) for w in ws]
    got = qmatmul_grouped(enc, lhs, rhs)
    assert [tuple(g.shape) for g in got] == [(m, n) for n in ns]
    for j, n in enumerate(ns):
        one = qmatmul(enc, None, lhs, rhs[j])
        if (enc, m, n, k) == (QE.Q4_K, 2, 1500, 8192):
            assert torch.allclose(got[j], one, rtol=1e-5, atol=1e-5), f"matrix {j} differs from the separate call"
        else:
            assert torch.equal(got[j], one), f"matrix {j} differs from the separate call"
        want = O.matmul_q4_0(a, ws[j]) if enc is QE.Q4_0 else O.matmul_f32(ENC[enc], a, ws[j])
        assert_close(got[j], want, f"grouped {enc.name} matrix {j} ({m}x{n}x{k})")


@pytest.mark.parametrize("enc,m,n,k,bf16", [(QE.Q4_K, 1, 14336, 4096, False), (QE.Q4_K, 1, 777, 2048, True), (QE.Q4_K, 1, 130, 14336, False),
                                            (QE.Q4_K, 1, 5, 256, False), (QE.Q4_K, 3, 200, 1024, False), (QE.Q6_K, 1, 300, 1024, False),
                                            (QE.Q4_0, 2, 96, 512, True), (QE.Q4_K, 40, 64, 512, True)])
def test_gated_pair_matches_two_matmuls(enc, m, n, k, bf16):
    """silu(lhs . gate^T) * (lhs . up^T): the fused epilogue of the decode kernel (Q4_K, one lhs row: one K part, several,
    a row count below the number of row streams) and the two-matmuls-and-combine route of every other shape, against
    the oracle's fp64 products combined in fp64, and against the library's own separate matmuls."""
    w, a = synth(61, 2 * n, k, m)
    if bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    a_eff = a
    if enc == QE.Q4_0:  # the Q4_0 path multiplies with the Q8_0 round trip of the lhs
        blocks = O.quantize_q8_0(a).reshape(m, -1, 34)
        d = O.f16_to_f32(np.ascontiguousarray(blocks[:, :, 0:2]).view(np.uint16)[..., 0])
        a_eff = (d[..., None] * blocks[:, :, 2:].view(np.int8).astype(np.float32)).reshape(m, k)
    wq = O.quantize(ENC[enc], w)
    gate, up = wq[:n], wq[n:]
    truth = O.swiglu(O.matmul_f64(ENC[enc], a_eff, gate), O.matmul_f64(ENC[enc], a_eff, up))
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    got = qmatmul_swiglu(enc, lhs, gpu(gate), gpu(up))
    assert got.shape == (m, n)
    assert_close(got, truth, f"gated pair {enc.name} {m}x{n}x{k} bf16={bf16}")
    g, u = qmatmul(enc, None, lhs, gpu(gate)).double(), qmatmul(enc, None, lhs, gpu(up)).double()
    assert_close(got, (g / (1.0 + torch.exp(-g)) * u).cpu().numpy(), "gated pair against the separate matmuls")


# ------------------------------------------------------------------ prefill shapes (m > 16)
@pytest.mark.parametrize("m,n,k", [(128, 256, 256), (17, 40, 512), (200, 300, 1024), (256, 512, 4096), (130, 64, 2048)])
def test_q4_k_gemm_bf16_lhs(m, n, k):
    """bf16 lhs (exact in the kernel's fp16 operands): against the fp32-weight oracle and fp64 truth."""
    w, a = synth(11, n, k, m)
    a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q4_K, w)
    want = O.matmul_f32(O.Q4_K, a, wq)
    truth = O.matmul_f64(O.Q4_K, a, wq)
    got = qmatmul(QE.Q4_K, None, gpu(a).to(torch.bfloat16), gpu(wq))
    assert_close(got, want, f"Q4_K GEMM {m}x{n}x{k} vs fp32 oracle")
    assert_close(got, truth, f"Q4_K GEMM {m}x{n}x{k} vs fp64 truth")


@pytest.mark.parametrize("m,n,k", [(64, 128, 512), (33, 64, 256), (32, 4096, 4096), (17, 1000, 4096), (100, 2050, 1024),
                                   (65, 520, 2560), (200, 16500, 512), (12, 16400, 8192)])
def test_q4_k_gemm_f32_lhs(m, n, k):
    """fp32 lhs: hi and residual fp16 planes (12 x 16400 x 8192: the GEMM from nine rows on, a large matrix with a long K).  From 1024 columns of K on (tiles cut into K shares) the residual plane is the
    second half of the rows of one lhs and a single pass multiplies both, and so it is up to 256 rows whatever the tiles (200 x
    16500: 455 tiles, no K shares); shorter K takes two passes.  Rows of very different magnitude (the row scales of both
    halves), ragged m and n."""
    w, a = synth(12, n, k, m)
    a *= np.logspace(-3, 3, m, dtype=np.float32)[:, None]
    wq = O.quantize(O.Q4_K, w)
    truth = O.matmul_f64(O.Q4_K, a, wq)
    got = qmatmul(QE.Q4_K, None, gpu(a), gpu(wq)).cpu().numpy()
    scale = np.abs(truth).max(axis=1, keepdims=True)
    assert np.all(np.abs(got - truth) <= 1e-4 * scale + 1e-3 * np.abs(truth)), f"Q4_K GEMM fp32 lhs {m}x{n}x{k}"
    one = qmatmul(QE.Q4_K, None, gpu(a[:1] / np.abs(a[:1]).max()), gpu(wq))
    assert_close(one, O.matmul_f32(O.Q4_K, a[:1] / np.abs(a[:1]).max(), wq), f"Q4_K fp32 lhs, first row alone {n}x{k}")


@pytest.mark.parametrize("m,n,k,bf16", [(512, 16384, 512, True), (500, 18600, 768, True), (300, 32768, 256, True),
                                        (520, 8200, 512, False)])
def test_q4_k_gemm_tile_kernel(m, n, k, bf16):
    """Shapes with at least 256 output tiles of 256 x 128 (and no more than 512 lhs rows or fewer than 160 tiles of
    256 x 256: beyond, the plane GEMM takes over) go to the kernel that unpacks each weight tile once per
    workgroup into LDS: whole rounds of tiles (256), a last round cut in two K halves that meet through atomic adds
    (292 tiles: 37 per XCD, 5 in the last round; K = 768 gives halves of 1 and 2 super-blocks), a single super-block
    (no halves possible), ragged edges, and an fp32 lhs (two planes; the second one adds to the first)."""
    w, a = synth(14, n, k, m)
    if bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q4_K, w)
    want = O.matmul_f32(O.Q4_K, a, wq)
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    wq_d = gpu(wq)
    got = qmatmul(QE.Q4_K, None, lhs, wq_d)
    assert_close(got, want, f"Q4_K tile GEMM {m}x{n}x{k}")
    again = qmatmul(QE.Q4_K, None, lhs, wq_d)  # the two halves of a tile may arrive in either order: same sum
    assert torch.equal(got, again)


@pytest.mark.parametrize("enc,m,n,k,bf16", [
    (QE.Q6_K, 65, 130, 512, True), (QE.Q6_K, 300, 257, 1024, False), (QE.Q6_K, 1000, 9300, 768, True), (QE.Q6_K, 256, 128, 256, True),
    (QE.Q5_K, 65, 130, 512, True), (QE.Q5_K, 33, 130, 768, True), (QE.Q5_K, 300, 257, 1024, False), (QE.Q5_K, 1000, 9300, 768, True), (QE.Q5_K, 520, 8200, 256, False),
    (QE.Q5_K, 40, 24, 36864, True), (QE.Q5_K, 20, 520, 2816, True), (QE.Q6_K, 16, 300, 5120, False), (QE.Q6_K, 12, 264, 18432, True)])
def test_q5_k_q6_k_prefill_on_the_matrix_cores(enc, m, n, k, bf16):
    """Q5_K and Q6_K above 64 lhs rows (from a few rows on where the small-batch kernel does not take K: Q5_K on 2816 and 36864
    columns, Q6_K on 5120 and 18432): the weights become fp16 integer planes (Q5_K sc * q; Q6_K two planes,
    (16 hi) * q and lo * q with sc = 16 hi + lo) and a tile GEMM multiplies them.  Ragged edges in m and n, one super-block,
    a last round of tiles cut in two K halves (292 tiles; for Q6_K the cut falls between or inside the planes), fp32 lhs
    (second pass on the residual), a K beyond what the Q5_K decode kernel takes; a third of the blocks carry random bytes
    (every scale byte value including negative Q6_K scales and the extremes -128 and 127, every code combination)."""
    e = ENC[enc]
    bpb = 210 if enc == QE.Q6_K else 176
    w, a = synth(61, n, k, m)
    if bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(e, w)
    rng = np.random.default_rng(62)
    blocks = wq.reshape(-1, bpb)
    rnd = rng.integers(0, 256, blocks.shape, dtype=np.uint8)
    keep = slice(208, 210) if enc == QE.Q6_K else slice(0, 4)  # the fp16 super-block scales stay finite
    rnd[:, keep] = blocks[:, keep]
    blocks[::3] = rnd[::3]
    if enc == QE.Q6_K:
        blocks[1, 192:208] = np.array([-128, 127, -1, 0, 15, 16, -16, -17, 1, -127, 126, 64, -64, 100, -100, 8], dtype=np.int8).view(np.uint8)
    truth = O.matmul_f64(e, a, wq)
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    wq_d = gpu(wq)
    got = qmatmul(enc, None, lhs, wq_d)
    assert_close(got, truth, f"{enc.name} planes GEMM {m}x{n}x{k} bf16={bf16}")
    if bf16 and n * k <= 1 << 22:
        assert_close(got, O.matmul_f32(e, a, wq), f"{enc.name} planes GEMM {m}x{n}x{k} vs fp32 oracle")
    again = qmatmul(enc, None, lhs, wq_d)
    assert torch.equal(got, again)


@pytest.mark.parametrize("kind,m,n,k,bf16", [
    ("Q5_K", 1030, 8200, 2304, False), ("Q4_K", 1600, 8200, 768, True), ("Q4_K", 1540, 10300, 2304, False),
    ("GPTQ128", 1600, 8200, 768, True), ("GPTQ256", 1540, 8200, 768, False), ("GPTQ128", 1536, 11016, 1280, False),
    ("Q4_K", 2000, 14192, 512, True), ("GPTQ128", 1990, 14192, 512, False), ("Q5_K", 1800, 14000, 256, True),
    ("GPTQ256", 1030, 10296, 1280, True), ("GPTQ128", 2000, 14192, 512, True), ("Q5_K", 200, 20600, 768, False)])
def test_plane_gemm_on_256_wide_tiles(kind, m, n, k, bf16):
    """Large problems of the single-plane encodings (from 160 tiles of 256 x 256; Q4_K and GPTQ from 513 lhs rows): the plane GEMM
    that keeps its accumulators in units of the current scale block's scale.  Q4_K / Q5_K carry their min term as extension
    blocks (K = 2304: nine super-blocks, a full extension block and one with a single super-block and zeros); GPTQ's scale
    blocks are its groups (two or four steps; K = 1280 with groups of 128 ends on half a 256-block); ragged m and n; an fp32
    lhs (second pass on the residual); 231, 287 and 264 tiles (one round; a second round of few tiles cut in K halves); 8 x 56 tiles on 256 compute units
    (one round of 256 x 256 tiles, then the remaining 6000 / 5808 columns as 256 x 192 tiles in a launch of their own, the last
    of them ragged and reaching past the last 128-column tile of the planes).  Every fifth K-quant block has
    d = 0 with its codes, scales and dmin in place (the weights are then -dmin * mn), every third carries random code and scale bytes."""
    w, a = synth(81, n, k, m)
    if bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    if kind.startswith("GPTQ"):
        group = int(kind[4:])
        qw, sc, qz, gi = O.quantize_gptq(w, group)
        sc[::2, ::7] = 0  # groups with a zero scale
        truth = O.matmul_gptq(a, qw, sc, qz, group=group, f64=True)
        args = (QE.GPTQ, QuantizationConfig(group_size=group), lhs, gpu(qw), gpu(sc.view(np.float16)), gpu(qz), gpu(gi))
    else:
        enc = QE[kind]
        e = ENC[enc]
        bpb = 176 if enc == QE.Q5_K else 144
        wq = O.quantize(e, w)
        blocks = wq.reshape(-1, bpb)
        rnd = np.random.default_rng(82).integers(0, 256, blocks.shape, dtype=np.uint8)
        rnd[:, 0:4] = blocks[:, 0:4]  # the fp16 super-block scales stay finite
        blocks[::3] = rnd[::3]
        blocks[::5, 0:2] = 0
        truth = O.matmul_f64(e, a, wq)
        args = (enc, None, lhs, gpu(wq))
    got = qmatmul(*args)
    assert_close(got, truth, f"{kind} wide plane GEMM {m}x{n}x{k} bf16={bf16}")
    again = qmatmul(*args)
    assert torch.equal(got, again)
    # a workspace too small for the planes: Q4_K and GPTQ then run their other prefill kernels, Q5_K has none (64 MiB hold its planes here)
    assert_close(qmatmul(*args, static_scratch=True), truth, f"{kind} {m}x{n}x{k} with the static scratch")


@pytest.mark.parametrize("enc,m,n,k", [(QE.Q4_K, 520, 16500, 512), (QE.Q6_K, 70, 300, 1024)])
def test_plane_gemm_non_finite_super_block_scale(enc, m, n, k):
    """A super-block scale of +inf or NaN makes every output of its weight row non-finite (as in the oracle, whose sums
    then hold inf - inf or 0 * inf) and leaves the other columns alone: the plane GEMMs carry their accumulators in units
    of the running scale, per column."""
    e = ENC[enc]
    bpb, doff = (144, 0) if enc == QE.Q4_K else (210, 208)
    w, a = synth(91, n, k, m)
    a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(e, w)
    rows = wq.reshape(n, k // 256, bpb)
    bad = {5: (0, 0x7C00), n - 3: (k // 256 - 1, 0x7E00), 130: (1, 0xFC00)}  # column: (super-block, fp16 bits)
    for col, (blk, bits16) in bad.items():
        rows[col, blk, doff:doff + 2] = np.frombuffer(np.uint16(bits16).tobytes(), dtype=np.uint8)
    want = O.matmul_f32(e, a, wq)
    got = qmatmul(enc, None, gpu(a).to(torch.bfloat16), gpu(wq)).cpu().numpy()
    good = np.ones(n, dtype=bool)
    for col in bad:
        good[col] = False
        assert not np.isfinite(want[:, col]).any()
        assert not np.isfinite(got[:, col]).any(), f"column {col}: finite outputs under a non-finite scale"
    assert np.isfinite(got[:, good]).all()
    assert O.isclose(got[:, good], want[:, good], RTOL, ATOL).all()


def test_q6_k_prefill_equals_the_decode_kernel_passes():
    """The same product through the planes GEMM (72 rows at once) and through the decode kernel (the rows in three calls
    of at most 64): two summation orders of the same exact products."""
    w, a = synth(63, 700, 2048, 72)
    a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq_d = gpu(O.quantize(O.Q6_K, w))
    lhs = gpu(a).to(torch.bfloat16)
    whole = qmatmul(QE.Q6_K, None, lhs, wq_d)
    parts = torch.cat([qmatmul(QE.Q6_K, None, lhs[i:i + 24], wq_d) for i in range(0, 72, 24)])
    assert_close(whole, parts.cpu().numpy(), "Q6_K planes GEMM against decode passes")


@pytest.mark.parametrize("enc,m,n,k,lhs_bf16", [
    (QE.Q4_K, 1, 1030, 4096, False), (QE.Q4_K, 1, 4096, 14336, True), (QE.Q4_K, 1, 66, 20480, False), (QE.Q4_K, 4, 512, 4096, False),
    (QE.Q4_K, 200, 300, 1024, True), (QE.Q6_K, 1, 777, 2048, False), (QE.Q6_K, 70, 130, 512, True), (QE.Q4_0, 3, 130, 4096, False),
    (QE.Q4_0, 40, 64, 1024, True), (QE.Q5_K, 40, 256, 512, True), (QE.GPTQ, 1, 256, 1024, False), (QE.GPTQ, 24, 128, 512, True)])
def test_bf16_output_is_the_fp32_result_narrowed(enc, m, n, k, lhs_bf16):
    """out_dtype=bfloat16: the bits are those of the fp32 result under the reference's narrowing rule (round to nearest
    even, NaN to the canonical quiet NaN; stdlib/src/builtin/simd.mojo:3279-3300, the oracle's f32_to_bf16), both where
    the kernel stores bf16 itself (Q4_K decode) and where an fp32 result in the workspace is narrowed afterwards.  A NaN
    in the first lhs row makes that whole output row NaN."""
    w, a = synth(71, n, k, m)
    a[0, 5] = np.nan
    lhs = gpu(a).to(torch.bfloat16) if lhs_bf16 else gpu(a)
    if enc == QE.GPTQ:
        qw, sc, qz, gi = O.quantize_gptq(w, 128)
        args = (QuantizationConfig(group_size=128), lhs, gpu(qw), gpu(sc.view(np.float16)), gpu(qz), gpu(gi))
    else:
        args = (None, lhs, gpu(O.quantize(ENC[enc], w)))
    f32 = qmatmul(enc, *args)
    b16 = qmatmul(enc, *args, out_dtype=torch.bfloat16)
    assert b16.dtype == torch.bfloat16 and b16.shape == f32.shape
    want = O.f32_to_bf16(f32.cpu().numpy())
    got = b16.cpu().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
    if enc != QE.Q4_0:  # (Q4_0 quantises the lhs first: a NaN does not survive as one)
        assert np.all((got[0] & 0x7fff) == 0x7fc0)
    into = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    qmatmul(enc, *args, out=into, out_dtype=torch.bfloat16)
    assert torch.equal(into.view(torch.int16), b16.view(torch.int16))


@pytest.mark.parametrize("enc,m,n,k,bf16", [
    (QE.Q4_0, 1, 1030, 4096, False), (QE.Q4_0, 1, 515, 4096, True), (QE.Q4_0, 4, 300, 2048, False), (QE.Q4_0, 2, 66, 8192, True),
    (QE.Q4_0, 3, 130, 1056, False), (QE.Q4_0, 9, 64, 1024, False), (QE.Q4_K, 1, 512, 4096, False), (QE.Q4_K, 40, 96, 1024, True),
    (QE.Q6_K, 2, 130, 2048, False)])
def test_rmsnorm_prologue(enc, m, n, k, bf16):
    """qmatmul_rmsnorm against the oracle: rmsnorm (fp32; bf16 x: rounded to bf16) then the encoding's matmul.  Q4_0 up
    to four rows is the decode kernel's own prologue (fused), the other cases a normalisation launch and the matmul; a
    fused result also has to agree with the two-step route through qmatmul on the normalised rows."""
    w, x = synth(81, n, k, m)
    x *= np.logspace(-2, 2, m, dtype=np.float32)[:, None]
    if bf16:
        x = O.bf16_to_f32(O.f32_to_bf16(x))
    gamma = np.random.default_rng(82).uniform(0.25, 2.0, k).astype(np.float32)
    eps = 1e-5
    wq = O.quantize(ENC[enc], w)
    y = O.rmsnorm(x, gamma, eps, to_bf16=bf16)
    want = O.matmul_q4_0(y, wq) if enc == QE.Q4_0 else O.matmul_f32(ENC[enc], y, wq)
    xd = gpu(x).to(torch.bfloat16) if bf16 else gpu(x)
    got = qmatmul_rmsnorm(enc, None, xd, gpu(gamma), eps, gpu(wq))
    assert_close(got, want, f"{enc.name} rmsnorm prologue {m}x{n}x{k} bf16={bf16}")
    yd = gpu(y).to(torch.bfloat16) if bf16 else gpu(y)
    assert_close(got, qmatmul(enc, None, yd, gpu(wq)).cpu().numpy(), "against qmatmul on the oracle's normalised rows")
    b16 = qmatmul_rmsnorm(enc, None, xd, gpu(gamma), eps, gpu(wq), out_dtype=torch.bfloat16)
    if not (enc == QE.Q4_0 and m <= 4):
        assert np.array_equal(b16.cpu().view(torch.int16).numpy().view(np.uint16), O.f32_to_bf16(got.cpu().numpy()))


def test_q4_k_gemm_wide_range_lhs():
    """Rows of very different magnitude: the per-row power-of-two scaling keeps fp16 operands exact."""
    w, a = synth(13, 96, 512, 40)
    a *= np.logspace(-6, 5, 40, dtype=np.float32)[:, None]
    a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q4_K, w)
    truth = O.matmul_f64(O.Q4_K, a, wq)
    got = qmatmul(QE.Q4_K, None, gpu(a).to(torch.bfloat16), gpu(wq)).cpu().numpy()
    scale = np.abs(truth).max(axis=1, keepdims=True)
    assert np.all(np.abs(got - truth) <= 1e-4 * scale + 1e-3 * np.abs(truth))


@pytest.mark.parametrize("m,n,k,group", [(128, 256, 256, 128), (17, 40, 512, 64), (200, 304, 1024, 128),
                                         (256, 512, 4096, 128), (130, 64, 2048, 256), (40, 72, 768, 64)])
def test_gptq_gemm_bf16_lhs(m, n, k, group):
    """GPTQ prefill kernel, bf16 lhs: against the fp32 oracle and the fp64 truth."""
    w, a = synth(21, n, k, m)
    a = O.bf16_to_f32(O.f32_to_bf16(a))
    qw, sc, qz, gi = O.quantize_gptq(w, group)
    want = O.matmul_gptq(a, qw, sc, qz, group)
    truth = O.matmul_gptq(a, qw, sc, qz, group, f64=True)
    cfg = QuantizationConfig(group_size=group)
    got = qmatmul(QE.GPTQ, cfg, gpu(a).to(torch.bfloat16), gpu(qw), gpu(sc.view(np.float16)), gpu(qz), gpu(gi))
    assert_close(got, want, f"GPTQ GEMM {m}x{n}x{k} g{group} vs fp32 oracle")
    assert_close(got, truth, f"GPTQ GEMM {m}x{n}x{k} g{group} vs fp64 truth")


@pytest.mark.parametrize("m,n,k,group", [(64, 128, 512, 128), (33, 64, 256, 64), (48, 96, 512, 256)])
def test_gptq_gemm_f32_lhs(m, n, k, group):
    w, a = synth(22, n, k, m)
    qw, sc, qz, gi = O.quantize_gptq(w, group)
    want = O.matmul_gptq(a, qw, sc, qz, group)
    got = qmatmul(QE.GPTQ, QuantizationConfig(group_size=group), gpu(a), gpu(qw), gpu(sc.view(np.float16)), gpu(qz),
                  gpu(gi))
    assert_close(got, want, f"GPTQ GEMM fp32 lhs {m}x{n}x{k} g{group}")


def test_gptq_gemm_arbitrary_zero_points():
    """Stored zero points other than 7: the zero term takes scale*zero as an exact fp16 hi + lo pair."""
    m, n, k, group = 64, 128, 1024, 128
    w, a = synth(23, n, k, m)
    a = O.bf16_to_f32(O.f32_to_bf16(a))
    qw, sc, qz, gi = O.quantize_gptq(w, group)
    rng = np.random.Generator(np.random.PCG64(24))
    qz = rng.integers(0, 2**32, size=qz.shape, dtype=np.uint64).astype(np.uint32).view(np.int32)
    truth = O.matmul_gptq(a, qw, sc, qz, group, f64=True)
    got = qmatmul(QE.GPTQ, QuantizationConfig(group_size=group), gpu(a).to(torch.bfloat16), gpu(qw),
                  gpu(sc.view(np.float16)), gpu(qz), gpu(gi))
    assert_close(got, truth, "GPTQ GEMM random zero points")


@pytest.mark.parametrize("lhs_bf16", [True, False])
def test_q4_k_gemm_many_tiles(lhs_bf16):
    """More tiles than the device holds at once, not a whole number of rounds: the leftover tiles are cut
    along K and summed in the output, which must not change the result beyond fp32 rounding."""
    m, n, k = 2048, 4352, 512
    w, a = synth(31, n, k, m)
    if lhs_bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q4_K, w)
    want = O.matmul_f32(O.Q4_K, a, wq)
    got = qmatmul(QE.Q4_K, None, gpu(a).to(torch.bfloat16) if lhs_bf16 else gpu(a), gpu(wq))
    assert_close(got, want, f"Q4_K GEMM {m}x{n}x{k} bf16={lhs_bf16}")


@pytest.mark.parametrize("lhs_bf16", [False, True])
def test_q6_k_decode_many_rows(lhs_bf16):
    """One lhs row against many weight rows (the vocabulary-projection shape): runs of 16 blocks with a
    partial last run, a row count that is not a multiple of the wavefront count."""
    n, k = 12418, 4864
    w, a = synth(41, n, k, 1)
    if lhs_bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q6_K, w)
    want = O.matmul_f32(O.Q6_K, a, wq)
    got = qmatmul(QE.Q6_K, None, gpu(a).to(torch.bfloat16) if lhs_bf16 else gpu(a), gpu(wq))
    assert_close(got, want, f"Q6_K 1x{n}x{k} bf16={lhs_bf16}")


@pytest.mark.parametrize("m,n,k,lhs_bf16", [(1, 12418, 4096, False), (1, 12301, 4096, True), (1, 13000, 2048, False),
                                            (2, 12418, 4096, False), (3, 12301, 4096, True), (5, 13000, 2048, False),
                                            (16, 12290, 4096, False), (1, 4096, 14336, False), (2, 2100, 14336, True),
                                            (1, 4100, 6144, False), (3, 2050, 10240, False), (1, 2049, 16384, True),
                                            (1, 8200, 2048, False)])
def test_q6_k_decode_vocabulary_shapes(m, n, k, lhs_bf16):
    """K = 4096 / 2048 with many rows: the kernel with compile-time field alignment and rows delivered straight
    into LDS (16 and 8 super-blocks per row; a row count that is not a multiple of the wavefront count); several
    lhs rows go through it in passes of two (an odd count ends with a pass of one); rows longer than 16 super-blocks
    are cut into 2 or 4 parts of 10, 12, 14 or 16 super-blocks (a last group of four with two blocks missing)."""
    w, a = synth(42, n, k, m)
    if lhs_bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q6_K, w)
    want = O.matmul_f32(O.Q6_K, a, wq)
    truth = O.matmul_f64(O.Q6_K, a, wq)
    got = qmatmul(QE.Q6_K, None, gpu(a).to(torch.bfloat16) if lhs_bf16 else gpu(a), gpu(wq))
    assert_close(got, want, f"Q6_K {m}x{n}x{k} bf16={lhs_bf16} vs fp32 oracle")
    assert_close(got, truth, f"Q6_K {m}x{n}x{k} bf16={lhs_bf16} vs fp64 truth")


@pytest.mark.parametrize("m,n,k,lhs_bf16", [(2, 16, 4096, False), (3, 33, 4096, True), (4, 1000, 4096, False), (5, 4099, 4096, True),
                                            (8, 250, 4096, False), (9, 47, 4096, False), (16, 530, 4096, True), (12, 9000, 4096, False),
                                            (20, 300, 4096, False), (40, 130, 4096, True), (64, 72, 4096, False),
                                            (4, 300, 14336, False), (8, 130, 8192, True), (5, 2100, 2048, False),
                                            (16, 77, 6144, False), (6, 40, 16384, True), (16, 300, 14336, True), (13, 50, 2048, True),
                                            (4, 4200, 14336, True), (2, 2100, 14336, False), (20, 1100, 8192, False),
                                            (4, 2100, 28672, False), (1, 2064, 20480, True)])
def test_q6_k_small_batch_matrix_core_kernel(m, n, k, lhs_bf16):
    """Q6_K with 2..64 lhs rows on K = 4096: weight rows decoded once for all lhs rows (codes as exact fp16 integers, one
    matrix-core instruction per 16-weight scale group and set of eight lhs rows; sixteen bf16 rows are one set without
    residual rows); the 2, 4, 8 and 16 row variants, further
    passes from 17 rows on, tiles that end past the matrix, more tiles than workgroups; K in rounds of 4096 columns, side by
    side in the grid, whose results a launch of their own adds in round order (a last round of 2048 with half the wavefronts;
    4200 weight rows: several tiles per workgroup and round).  Rows of very different magnitude share
    a pass (the lhs is scaled per row)."""
    w, a = synth(43, n, k, m)
    a[m - 1] *= 1000.0 if n < 2000 else 10.0  # (thousands of outputs of a row of 1e3-size terms: some cancel to below the bar's reach)
    a[0, :512] *= 1e-3
    if lhs_bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q6_K, w)
    want = O.matmul_f32(O.Q6_K, a, wq)
    truth = O.matmul_f64(O.Q6_K, a, wq)
    got = qmatmul(QE.Q6_K, None, gpu(a).to(torch.bfloat16) if lhs_bf16 else gpu(a), gpu(wq))
    assert_close(got, want, f"Q6_K {m}x{n}x{k} bf16={lhs_bf16} vs fp32 oracle")
    assert_close(got, truth, f"Q6_K {m}x{n}x{k} bf16={lhs_bf16} vs fp64 truth")


@pytest.mark.parametrize("m,n,k,lhs_bf16", [(200, 300, 1024, False), (64, 130, 4096, True), (17, 16, 96, False),
                                            (65, 33, 32, False), (130, 515, 608, True), (300, 258, 2048, False)])
def test_q4_0_matmul_int8_matrix_cores(m, n, k, lhs_bf16):
    """Q4_0 with many lhs rows: 16 x 16 integer block dots per matrix-core instruction, several passes of
    64 lhs rows, ragged N and a K that does not split evenly over the four wavefronts; from 65 lhs rows on the
    kernel with the weights as the first operand (N not a multiple of 4, 32 or 256, K of one block and of a
    partial last run, a last lhs tile with one row)."""
    w, a = synth(51, n, k, m)
    if lhs_bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q4_0, w)
    want = O.matmul_q4_0(a, wq)
    got = qmatmul(QE.Q4_0, None, gpu(a).to(torch.bfloat16) if lhs_bf16 else gpu(a), gpu(wq))
    assert_close(got, want, f"Q4_0 {m}x{n}x{k} bf16={lhs_bf16}")


@pytest.mark.parametrize("m,n,k,bf16", [(1024, 8192, 512, True), (1000, 9300, 768, False), (300, 32768, 256, True), (520, 8200, 1280, False)])
def test_q4_0_prefill_plane_gemm(m, n, k, bf16):
    """Q4_0 with more than 64 lhs rows: the fp16 matrix-core kernel over integer planes (lhs Q8_0 codes, weights
    q - 8; the block scale products made by the matrix cores too).  Whole rounds of tiles, a last round cut in two K halves, a
    single group of eight blocks, ragged edges; against the oracle's integer path."""
    w, a = synth(24, n, k, m)
    if bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    wq = O.quantize(O.Q4_0, w)
    want = O.matmul_q4_0(a, wq)
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    wq_d = gpu(wq)
    got = qmatmul(QE.Q4_0, None, lhs, wq_d)
    assert_close(got, want, f"Q4_0 plane GEMM {m}x{n}x{k}")
    assert torch.equal(got, qmatmul(QE.Q4_0, None, lhs, wq_d))


@pytest.mark.parametrize("one_hot", [True, False])
def test_q4_0_prefill_plane_gemm_gives_the_integer_block_dots(one_hot):
    """The same bit-exact check as for the other Q4_0 kernels, on a problem whose last round of tiles is cut along K."""
    lhs, wq, want = _integer_dot_case(300, 16384, 512, one_hot, False, 7)
    got = qmatmul(QE.Q4_0, None, lhs, wq).cpu().numpy()
    assert np.array_equal(got, want)


def test_graph_capture_and_replay_match_eager():
    """The library only enqueues kernels on the caller's stream (no allocation, no synchronisation, no memset), so
    calls can be captured into a HIP graph: replays with new lhs values in the same buffers must give what eager
    calls give, for a decode call, a small-batch call, a Q4_0 call with its workspace, a gated pair and a prefill GEMM
    with its lhs pass."""
    from mojo_amd import _lib
    import ctypes as C

    lib = _lib.load()
    n, k = 512, 1024
    w, _ = synth(81, 2 * n, k, 1)
    wk = gpu(O.quantize(O.Q4_K, w))
    w0 = gpu(O.quantize(O.Q4_0, w[:n]))
    cases = [(QE.Q4_K, wk[:n], 1), (QE.Q4_K, wk[:n], 4), (QE.Q4_0, w0, 3), (QE.Q4_K, wk[:n], 40)]
    bufs = []
    for enc, wt, m in cases:
        a = torch.zeros((m, k), dtype=torch.float32, device=DEV)
        out = torch.empty((m, n), dtype=torch.float32, device=DEV)
        need = lib.qmm_matmul_workspace_bytes(enc.code, _lib.QMM_F32, m, n, k)
        ws = torch.empty((max(need, 1),), dtype=torch.uint8, device=DEV)
        bufs.append((enc, wt, m, a, out, ws, need))
    ag = torch.zeros((1, k), dtype=torch.float32, device=DEV)
    og = torch.empty((1, n), dtype=torch.float32, device=DEV)

    def enqueue(stream):
        for enc, wt, m, a, out, ws, need in bufs:
            ptrs = (C.c_void_p * 1)(wt.data_ptr())
            rc = lib.qmm_matmul(enc.code, None, C.c_void_p(a.data_ptr()), _lib.QMM_F32, m, k, ptrs, 1, n,
                                C.c_void_p(out.data_ptr()), C.c_void_p(ws.data_ptr()), need, 0, C.c_void_p(stream))
            assert rc == 0, lib.qmm_last_error()
        rc = lib.qmm_matmul_swiglu(QE.Q4_K.code, C.c_void_p(ag.data_ptr()), _lib.QMM_F32, 1, k, C.c_void_p(wk[:n].data_ptr()),
                                   C.c_void_p(wk[n:].data_ptr()), n, C.c_void_p(og.data_ptr()), None, 0, C.c_void_p(stream))
        assert rc == 0, lib.qmm_last_error()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        enqueue(side.cuda_stream)  # warm every kernel outside the capture
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            enqueue(torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    rng = np.random.Generator(np.random.PCG64(82))
    for rep in range(3):
        for _, _, m, a, _, _, _ in bufs:
            a.copy_(gpu(rng.standard_normal((m, k), dtype=np.float32)))
        ag.copy_(gpu(rng.standard_normal((1, k), dtype=np.float32)))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for enc, wt, m, a, out, _, _ in bufs:
            want = qmatmul(enc, None, a, wt)
            assert torch.equal(out, want), f"replay {rep}: {enc.name} m={m} differs from the eager call"
        assert torch.equal(og, qmatmul_swiglu(QE.Q4_K, ag, wk[:n], wk[n:])), f"replay {rep}: gated pair differs"


def test_concurrent_calls_on_two_streams():
    """Entry points are re-entrant: two host threads, each with its own stream, issue different encodings at the same
    time (ctypes drops the GIL inside the calls); every result equals the single-threaded one."""
    import threading

    n, k = 1024, 2048
    w, a = synth(91, n, k, 4)
    jobs = [(QE.Q4_K, gpu(O.quantize(O.Q4_K, w)), gpu(a[:1])), (QE.Q6_K, gpu(O.quantize(O.Q6_K, w)), gpu(a[:1])),
            (QE.Q4_0, gpu(O.quantize(O.Q4_0, w)), gpu(a)), (QE.Q4_K, gpu(O.quantize(O.Q4_K, w)), gpu(a))]
    want = [qmatmul(enc, None, lhs, wq).clone() for enc, wq, lhs in jobs]
    torch.cuda.synchronize()
    errors = []

    def worker(offset):
        try:
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                for it in range(40):
                    j = (it + offset) % len(jobs)
                    enc, wq, lhs = jobs[j]
                    got = qmatmul(enc, None, lhs, wq)
                    s.synchronize()
                    if not torch.equal(got, want[j]):
                        errors.append(f"thread {offset} iteration {it}: {enc.name} differs")
        except Exception as e:  # noqa: BLE001
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(o,)) for o in (0, 2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors[:3]
