"""GPU parity of the weight planes kept across calls (repack_weights / qmatmul_repacked) against the CPU oracle and against
qmatmul, which converts per call.

Bars: fp32 outputs within rtol 1e-3 / atol 1e-4 under the reference's symmetric isclose
(stdlib/src/math/math.mojo:1023-1030); bit-identical to qmatmul wherever both run the same GEMM over the same planes.
"""
import numpy as np
import pytest
import torch

import oracle as O
from conftest import synth
from mojo_amd import QuantizationConfig, QuantizationEncoding as QE
from mojo_amd import qmatmul, qmatmul_repacked, repack_weights
from test_gpu_parity import ENC, assert_close, gpu

pytestmark = pytest.mark.gpu


def kquant_weights(enc, n, k, seed):
    """Quantised weights with every third block random bytes (finite scales) and every fifth with d = 0."""
    e = ENC[enc]
    bpb = {QE.Q4_K: 144, QE.Q5_K: 176, QE.Q6_K: 210}[enc]
    w, _ = synth(seed, n, k, 1)
    wq = O.quantize(e, w)
    blocks = wq.reshape(-1, bpb)
    rnd = np.random.default_rng(seed + 1).integers(0, 256, blocks.shape, dtype=np.uint8)
    keep = slice(208, 210) if enc == QE.Q6_K else slice(0, 4)
    rnd[:, keep] = blocks[:, keep]
    blocks[::3] = rnd[::3]
    blocks[::5, keep.start:keep.start + 2] = 0
    return wq


def lhs_rows(seed, m, k, bf16):
    _, a = synth(seed, 1, k, m)
    if bf16:
        a = O.bf16_to_f32(O.f32_to_bf16(a))
    return a, (gpu(a).to(torch.bfloat16) if bf16 else gpu(a))


@pytest.mark.parametrize("enc,n,k,rows", [
    # (row count, bf16 lhs, same route as qmatmul)
    (QE.Q6_K, 300, 1024, [(70, True, True), (300, False, True), (3, True, True)]),
    (QE.Q6_K, 9300, 768, [(1000, True, True)]),
    (QE.Q5_K, 8200, 2304, [(1030, False, True), (40, True, True), (700, True, True), (2, False, True)]),
    (QE.Q5_K, 257, 512, [(33, True, True), (300, False, True)]),
    (QE.Q5_K, 1100, 2560, [(300, True, True), (70, True, True), (300, False, True)]),
    (QE.Q6_K, 1100, 2560, [(300, True, True), (70, True, True), (300, False, True)]),
    (QE.Q4_K, 14080, 768, [(520, True, True), (1600, False, True), (300, True, False), (64, True, True)]),
    (QE.Q4_K, 20600, 256, [(2000, True, True), (300, True, False)]),
    (QE.Q4_K, 20600, 768, [(200, False, False), (90, False, False)]),
    (QE.Q5_K, 20600, 768, [(200, False, True), (130, True, True)]),
])
def test_repacked_kquant_matches_oracle_and_qmatmul(enc, n, k, rows):
    """One conversion, many calls.  Q4_K / Q5_K planes carry their min operands both as extension blocks (wide GEMM: 1030 x 8200,
    520 and 1600 x 14080, 2000 x 20600 in two launches) and as the table of the 256 x 128 kernel (40, 700 x 8200 and the small
    matrix), which then steps over the extension blocks (K = 2304: two of them, one with a single super-block); Q6_K has one
    layout.  Few tiles on K >= 2048 with a bf16 lhs (300 and 70 x 1100 x 2560: 18 and 9 tiles, ten super-blocks) are cut in four K quarters
    of 2, 3, 2 and 3 super-blocks that meet pairwise in two buffers; the fp32 lhs takes halves.  Row counts of the decode kernels are served from the packed tensors.  300 x 20600 (162 tiles of 256 x 256) takes the wide tiles
    here, 300 x 14080 the 256 x 128 plane kernel, and inside qmatmul both take kernels that unpack as they go: close, not identical.
    An fp32 lhs of up to 256 rows goes through the GEMMs as one lhs of twice the rows: 200 x 20600 is then 162 wide tiles (the residual
    rows' extension blocks are zeros), 90 x 20600 one row tile of the 256 x 128 kernel, 300 x 1100 x 2560 K quarters."""
    wq = kquant_weights(enc, n, k, 7 + n % 5)
    wq_d = gpu(wq)
    weights = repack_weights(enc, None, wq_d)
    assert weights.n == n and weights.k == k
    for m, bf16, same in rows:
        a, lhs = lhs_rows(m, m, k, bf16)
        truth = O.matmul_f64(ENC[enc], a, wq)
        got = qmatmul_repacked(lhs, weights)
        assert_close(got, truth, f"{enc.name} repacked {m}x{n}x{k} bf16={bf16}")
        assert torch.equal(got, qmatmul_repacked(lhs, weights))
        if same:
            assert torch.equal(got, qmatmul(enc, None, lhs, wq_d)), f"{enc.name} {m}x{n}x{k}: differs from qmatmul"


@pytest.mark.parametrize("group,n,k,rows", [
    (128, 8200, 768, [(1600, True, True), (1540, False, True), (300, True, True), (5, True, True)]),
    (256, 14192, 512, [(1990, False, True)]),
    (128, 11016, 1280, [(1536, True, True)]),
    (128, 4104, 1024, [(300, True, False), (120, False, False), (90, True, True)]),
])
def test_repacked_gptq_matches_oracle_and_qmatmul(group, n, k, rows):
    """GPTQ planes (q - zero, scale blocks = groups) made once; groups with a zero scale; one and two launches of the wide GEMM, a
    last round of tiles cut in K halves (1536 x 11016), K ending on half a 256-block; few tiles (300 and 120 x 4104: 34 and 17
    tiles of 256 x 256), which the kept planes leave to qmatmul's GEMM that unpacks as it goes (tiles cut into K shares)."""
    w, _ = synth(21, n, k, 1)
    qw, sc, qz, gi = O.quantize_gptq(w, group)
    sc[::2, ::7] = 0
    cfg = QuantizationConfig(group_size=group)
    rhs = (gpu(qw), gpu(sc.view(np.float16)), gpu(qz), gpu(gi))
    weights = repack_weights(QE.GPTQ, cfg, *rhs)
    for m, bf16, same in rows:
        a, lhs = lhs_rows(30 + m, m, k, bf16)
        truth = O.matmul_gptq(a, qw, sc, qz, group=group, f64=True)
        got = qmatmul_repacked(lhs, weights)
        assert_close(got, truth, f"GPTQ g{group} repacked {m}x{n}x{k} bf16={bf16}")
        if same:
            assert torch.equal(got, qmatmul(QE.GPTQ, cfg, lhs, *rhs)), f"GPTQ {m}x{n}x{k}: differs from qmatmul"


@pytest.mark.parametrize("n,k,rows", [(300, 1024, [(70, True, True), (300, False, True), (16, True, True)]),
                                      (9300, 768, [(1000, True, True)]), (1100, 2560, [(300, True, True), (70, False, True)]),
                                      (2000, 1024, [(96, True, False), (96, False, False)])])
def test_repacked_q4_0_matches_oracle_and_qmatmul(n, k, rows):
    """Q4_0: the plane of q - 8 and the block scales made once.  The lhs is quantised to Q8_0 per call as everywhere, so the
    result is that of the integer block dots: bit-identical with qmatmul wherever both run the same kernel (the plane GEMM at
    many rows, the 16-row int8 kernel at few), within the bar of the oracle's Q8_0 x Q4_0 product at every row count; without
    the packed tensor few rows run over the plane too.  1100 x 2560: few tiles on ten groups of 256, cut in four K quarters
    that meet pairwise in two buffers.  2000 x 1024 with 96 rows: the kept plane serves the call, while qmatmul, which would
    have to make the plane first, takes six passes of the 16-row kernel (another order of the block sums)."""
    w, _ = synth(17, n, k, 1)
    wq = O.quantize(O.Q4_0, w)
    wq_d = gpu(wq)
    weights = repack_weights(QE.Q4_0, None, wq_d)
    alone = repack_weights(QE.Q4_0, None, wq_d, keep_rhs=False)
    for m, bf16, same in rows:
        a, lhs = lhs_rows(60 + m, m, k, bf16)
        want = O.matmul_q4_0(a, wq)
        got = qmatmul_repacked(lhs, weights)
        assert_close(got, want, f"Q4_0 repacked {m}x{n}x{k} bf16={bf16}")
        per_call = qmatmul(QE.Q4_0, None, lhs, wq_d)
        if same:
            assert torch.equal(got, per_call), f"Q4_0 {m}x{n}x{k}: differs from qmatmul"
        else:
            assert_close(per_call, want, f"Q4_0 {m}x{n}x{k} bf16={bf16}")
        assert_close(qmatmul_repacked(lhs, alone), want, f"Q4_0 plane only {m}x{n}x{k}")


@pytest.mark.parametrize("enc", [QE.Q4_K, QE.Q5_K, QE.Q6_K, QE.GPTQ])
def test_repacked_without_the_packed_tensors(enc):
    """keep_rhs=False: the planes are all the caller holds, and every row count goes through the plane GEMMs (one lhs row, a
    few, a ragged row tile; small matrices run the 256 x 128 kernel, GPTQ the wide one)."""
    n, k = 264, 1024
    if enc == QE.GPTQ:
        w, _ = synth(41, n, k, 1)
        qw, sc, qz, gi = O.quantize_gptq(w, 128)
        cfg = QuantizationConfig(group_size=128)
        weights = repack_weights(enc, cfg, gpu(qw), gpu(sc.view(np.float16)), gpu(qz), gpu(gi), keep_rhs=False)
        truth_of = lambda a: O.matmul_gptq(a, qw, sc, qz, group=128, f64=True)
    else:
        wq = kquant_weights(enc, n, k, 43)
        weights = repack_weights(enc, None, gpu(wq), keep_rhs=False)
        truth_of = lambda a: O.matmul_f64(ENC[enc], a, wq)
    assert weights.rhs == ()
    for m, bf16 in [(1, True), (5, False), (270, True)]:
        a, lhs = lhs_rows(50 + m, m, k, bf16)
        assert_close(qmatmul_repacked(lhs, weights), truth_of(a), f"{enc.name} planes only, {m} rows")


def test_repack_refusals():
    w = torch.zeros((8, 18 * 4), dtype=torch.uint8, device="cuda:0")
    with pytest.raises(NotImplementedError):
        repack_weights(QE.Q4_0, None, w)  # K = 128: the plane GEMMs take multiples of 256
    n, k = 64, 512
    wq, _ = synth(3, n, k, 1)
    qw, sc, qz, gi = O.quantize_gptq(wq, 64)
    with pytest.raises(NotImplementedError):
        repack_weights(QE.GPTQ, QuantizationConfig(group_size=64), gpu(qw), gpu(sc.view(np.float16)), gpu(qz), gpu(gi))
    with pytest.raises(TypeError):
        qmatmul_repacked(torch.zeros((1, 256), device="cuda:0"), "weights")


def test_a_buffer_made_for_something_else_is_caught():
    """Planes of the same size made for another encoding or GPTQ group pass every size check.  The record at the head of the
    buffer does not: the call's result is all NaN, and qmm_repack_check names both descriptions; the right buffer passes both."""
    import ctypes as C

    from mojo_amd import _lib

    lib = _lib.load()
    n, k, m = 512, 1024, 300
    w, a = synth(5, n, k, m)
    lhs = gpu(O.bf16_to_f32(O.f32_to_bf16(a))).to(torch.bfloat16)
    s = torch.cuda.current_stream().cuda_stream
    w4, w5 = gpu(O.quantize(O.Q4_K, w)), gpu(O.quantize(O.Q5_K, w))
    size = lib.qmm_repack_bytes(QE.Q4_K.code, None, n, k)
    assert size == lib.qmm_repack_bytes(QE.Q5_K.code, None, n, k)  # same planes, other contents
    packed = torch.empty((size,), dtype=torch.uint8, device="cuda:0")
    out = torch.zeros((m, n), dtype=torch.float32, device="cuda:0")
    need = lib.qmm_matmul_repacked_workspace_bytes(QE.Q4_K.code, _lib.QMM_BF16, m, n, k)
    ws = torch.empty((max(need, 1),), dtype=torch.uint8, device="cuda:0")

    def repack(enc, t):
        _lib.check(lib.qmm_repack(enc.code, None, (C.c_void_p * 1)(t.data_ptr()), 1, n, k, C.c_void_p(packed.data_ptr()), size, C.c_void_p(s)), "qmm_repack")

    def matmul(enc):
        return lib.qmm_matmul_repacked(enc.code, None, C.c_void_p(lhs.data_ptr()), _lib.QMM_BF16, m, k, None, 0, C.c_void_p(packed.data_ptr()), size,
                                       n, C.c_void_p(out.data_ptr()), C.c_void_p(ws.data_ptr()), need, 0, C.c_void_p(s))

    def check(enc):
        return lib.qmm_repack_check(enc.code, None, n, k, C.c_void_p(packed.data_ptr()), size, C.c_void_p(s))

    packed.zero_()
    assert check(QE.Q4_K) == -1 and b"record" in lib.qmm_last_error()  # never written
    repack(QE.Q5_K, w5)
    assert check(QE.Q5_K) == 0
    assert check(QE.Q4_K) == -1 and b"encoding 4" in lib.qmm_last_error() and b"encoding 1" in lib.qmm_last_error()
    assert matmul(QE.Q4_K) == 0
    assert torch.isnan(out).all()
    repack(QE.Q4_K, w4)
    assert check(QE.Q4_K) == 0
    assert matmul(QE.Q4_K) == 0
    torch.cuda.synchronize()
    assert_close(out, O.matmul_f64(O.Q4_K, O.bf16_to_f32(O.f32_to_bf16(a)), O.quantize(O.Q4_K, w)), "Q4_K over its own planes")
    # GPTQ: groups of 128 and of 256 give buffers of one size
    cfg128, cfg256 = _lib.GptqConfig(4, 128, 0, 1), _lib.GptqConfig(4, 256, 0, 1)
    gsize = lib.qmm_repack_bytes(QE.GPTQ.code, C.byref(cfg128), n, k)
    if gsize == lib.qmm_repack_bytes(QE.GPTQ.code, C.byref(cfg256), n, k):
        from mojo_amd import quantize_gptq

        qw, sc, qz, _ = quantize_gptq(gpu(w), QuantizationConfig(quant_method="gptq", bits=4, group_size=128, desc_act=False, sym=True))
        gp = torch.empty((gsize,), dtype=torch.uint8, device="cuda:0")
        rhs = (C.c_void_p * 3)(qw.data_ptr(), sc.data_ptr(), qz.data_ptr())
        _lib.check(lib.qmm_repack(QE.GPTQ.code, C.byref(cfg128), rhs, 3, n, k, C.c_void_p(gp.data_ptr()), gsize, C.c_void_p(s)), "qmm_repack")
        assert lib.qmm_repack_check(QE.GPTQ.code, C.byref(cfg128), n, k, C.c_void_p(gp.data_ptr()), gsize, C.c_void_p(s)) == 0
        assert lib.qmm_repack_check(QE.GPTQ.code, C.byref(cfg256), n, k, C.c_void_p(gp.data_ptr()), gsize, C.c_void_p(s)) == -1
        assert b"group 128" in lib.qmm_last_error() and b"group 256" in lib.qmm_last_error()
