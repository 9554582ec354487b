"""GPU parity at the full sizes of the benchmark configurations.

The CPU oracle cannot finish these shapes in test time, so every case is checked two ways:
  * a random sample of output columns (weight rows) against the oracle's fp64 sums on exactly those rows
    (and the packed bytes of those rows against the oracle's packer);
  * every output against  lhs . dequantize(rhs)^T  summed in fp64 on the GPU, where ``dequantize`` is the
    library's own unpacker (bit-exact with the oracle, see test_gpu_parity.py): a matmul kernel that drops a
    term, a row or a tile anywhere in the full shape fails it.
Tolerance: rtol 1e-3 / atol 1e-4 under the reference's symmetric isclose (stdlib/src/math/math.mojo:1023-1030).
"""
import numpy as np
import pytest
import torch

import oracle as O
from mojo_amd import QuantizationConfig, QuantizationEncoding as QE
from mojo_amd import dequantize, qmatmul, quantize, quantize_gptq

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-3, 1e-4
DEV = "cuda:0"
ENC = {QE.Q4_0: O.Q4_0, QE.Q4_K: O.Q4_K, QE.Q6_K: O.Q6_K, QE.Q5_K: O.Q5_K}


def close_on_gpu(got: torch.Tensor, want64: torch.Tensor) -> torch.Tensor:
    g = got.double()
    return (g - want64).abs() <= torch.maximum(torch.full_like(want64, ATOL), RTOL * torch.maximum(g.abs(), want64.abs()))


def fp64_product(a64: torch.Tensor, w32: torch.Tensor) -> torch.Tensor:
    """a64 [M, K] . w32[N, K]^T in fp64, N in slabs so that the fp64 copy of the weights stays small."""
    out = torch.empty((a64.shape[0], w32.shape[0]), dtype=torch.float64, device=a64.device)
    for n0 in range(0, w32.shape[0], 16384):
        out[:, n0:n0 + 16384] = a64 @ w32[n0:n0 + 16384].double().T
    return out


def check_all(got, a64, w32, what):
    ok = close_on_gpu(got, fp64_product(a64, w32))
    bad = int((~ok).sum())
    assert bad == 0, f"{what}: {bad}/{ok.numel()} outputs outside rtol={RTOL} atol={ATOL} of the fp64 product"


def weights(seed, n, k):
    gen = torch.Generator(device=DEV)
    gen.manual_seed(seed)
    return torch.randn((n, k), dtype=torch.float32, device=DEV, generator=gen) * 0.02, gen


def q8_0_round_trip(a: np.ndarray) -> np.ndarray:
    """The values the Q4_0 path multiplies with: lhs rows after Q8_0 quantisation, d * q."""
    blocks = O.quantize_q8_0(a).reshape(a.shape[0], -1, 34)
    d = O.f16_to_f32(np.ascontiguousarray(blocks[:, :, 0:2]).view(np.uint16)[..., 0])
    q = blocks[:, :, 2:].view(np.int8).astype(np.float32)
    return (d[..., None] * q).reshape(a.shape).astype(np.float32)


@pytest.mark.parametrize("enc,m,n,k", [
    (QE.Q4_0, 1, 4096, 4096),      # Q4_0 decode
    (QE.Q4_0, 16, 14336, 4096),    # Q4_0 small batch, MLP up-projection
    (QE.Q4_K, 1, 4096, 4096), (QE.Q4_K, 4, 4096, 4096),        # q / o
    (QE.Q4_K, 1, 1024, 4096), (QE.Q4_K, 4, 1024, 4096),        # k / v
    (QE.Q4_K, 1, 14336, 4096), (QE.Q4_K, 4, 14336, 4096),      # gate / up
    (QE.Q4_K, 1, 4096, 14336), (QE.Q4_K, 4, 4096, 14336),      # down
    (QE.Q4_K, 16, 4096, 14336),    # down with 16 rows: the small-batch kernel that cuts K across workgroups
    (QE.Q6_K, 1, 128256, 4096),    # lm_head
])
def test_decode_configurations_full_size(enc, m, n, k):
    w, gen = weights(100 + n % 97 + m, n, k)
    packed = quantize(enc, w)
    a = torch.randn((m, k), dtype=torch.float32, device=DEV, generator=gen)
    got = qmatmul(enc, None, a, packed)
    assert got.shape == (m, n) and got.dtype == torch.float32
    # sampled weight rows: packed bytes and fp64 sums of the oracle
    idx = np.sort(np.random.default_rng(n + m).choice(n, 48, replace=False))
    rows = packed[torch.from_numpy(idx).to(DEV)].cpu().numpy()
    assert np.array_equal(rows, O.quantize(ENC[enc], w[torch.from_numpy(idx).to(DEV)].cpu().numpy()))
    a_np = a.cpu().numpy()
    a_eff = q8_0_round_trip(a_np) if enc == QE.Q4_0 else a_np
    truth = O.matmul_f64(ENC[enc], a_eff, rows)
    ok = O.isclose(got[:, torch.from_numpy(idx).to(DEV)].cpu().numpy(), truth, RTOL, ATOL)
    assert ok.all(), f"{enc.name} {m}x{n}x{k}: {(~ok).sum()} sampled outputs differ from the oracle"
    if enc == QE.Q4_0:
        want = O.matmul_q4_0(a_np, rows)  # the integer-dot path itself, same rows
        assert O.isclose(got[:, torch.from_numpy(idx).to(DEV)].cpu().numpy(), want, RTOL, ATOL).all()
    # every output
    check_all(got, torch.from_numpy(a_eff).to(DEV).double(), dequantize(enc, packed), f"{enc.name} {m}x{n}x{k}")


@pytest.mark.parametrize("kind", ["Q4_K", "Q6_K", "Q5_K", "GPTQ"])
def test_prefill_configuration_full_size(kind):
    m, n, k = 2048, 14336, 4096
    w, gen = weights(7, n, k)
    a = torch.randn((m, k), dtype=torch.float32, device=DEV, generator=gen).to(torch.bfloat16)
    idx = np.sort(np.random.default_rng(5).choice(n, 32, replace=False))
    tidx = torch.from_numpy(idx).to(DEV)
    a_np = a.float().cpu().numpy()
    if kind != "GPTQ":
        enc = QE[kind]
        packed = quantize(enc, w)
        got = qmatmul(enc, None, a, packed)
        truth = O.matmul_f64(ENC[enc], a_np, packed[tidx].cpu().numpy())
        w32 = dequantize(enc, packed)
    else:
        cfg = QuantizationConfig()
        qw, sc, qz, gi = quantize_gptq(w)
        got = qmatmul(QE.GPTQ, cfg, a, qw, sc, qz, gi)
        qz_cols = qz.cpu().numpy()
        # the sampled columns as a GPTQ problem of their own: N' = 8 * 32 columns (whole qzeros words)
        words = np.unique(idx // 8)
        cols = (words[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
        tcols = torch.from_numpy(cols).to(DEV)
        truth_cols = O.matmul_gptq(a_np, qw[:, tcols].cpu().numpy(), sc[:, tcols].cpu().numpy().view(np.uint16),
                                   np.ascontiguousarray(qz_cols[:, words]), f64=True)
        pos = {c: i for i, c in enumerate(cols.tolist())}
        truth = truth_cols[:, [pos[c] for c in idx.tolist()]]
        w32 = dequantize(QE.GPTQ, qw, sc, qz, gi, config=cfg)
    assert got.shape == (m, n)
    ok = O.isclose(got[:, tidx].cpu().numpy(), truth, RTOL, ATOL)
    assert ok.all(), f"{kind} prefill: {(~ok).sum()}/{ok.size} sampled outputs differ from the oracle"
    check_all(got, a.double(), w32, f"{kind} prefill {m}x{n}x{k}")
    if kind in ("Q4_K", "GPTQ"):
        # The weight planes of this shape do not fit the library's static scratch: the same call through it runs the
        # kernels that unpack as they go.
        if kind == "Q4_K":
            other = qmatmul(enc, None, a, packed, static_scratch=True)
        else:
            other = qmatmul(QE.GPTQ, cfg, a, qw, sc, qz, gi, static_scratch=True)
        ok = O.isclose(other[:, tidx].cpu().numpy(), truth, RTOL, ATOL)
        assert ok.all(), f"{kind} prefill, static scratch: {(~ok).sum()}/{ok.size} sampled outputs differ from the oracle"
        check_all(other, a.double(), w32, f"{kind} prefill {m}x{n}x{k}, static scratch")


@pytest.mark.parametrize("kind", ["Q4_K", "GPTQ"])
@pytest.mark.parametrize("m,n,k", [(512, 4096, 4096), (512, 4096, 14336), (512, 14336, 4096), (64, 4096, 4096), (200, 1024, 4096)])
def test_mid_size_prefill_full_size(kind, m, n, k):
    """A layer's projections with a few hundred lhs rows (a prefill chunk, a wide decode batch): the kernels below the plane
    GEMM's thresholds, with K cut across workgroups where the tiles are few.  Sampled columns against the oracle's fp64
    sums, every output against the fp64 product on the GPU."""
    w, gen = weights(500 + m + n % 89, n, k)
    a = torch.randn((m, k), dtype=torch.float32, device=DEV, generator=gen).to(torch.bfloat16)
    a_np = a.float().cpu().numpy()
    if kind == "Q4_K":
        packed = quantize(QE.Q4_K, w)
        got = qmatmul(QE.Q4_K, None, a, packed)
        idx = np.sort(np.random.default_rng(m + k).choice(n, 24, replace=False))
        tidx = torch.from_numpy(idx).to(DEV)
        truth = O.matmul_f64(O.Q4_K, a_np, packed[tidx].cpu().numpy())
        w32 = dequantize(QE.Q4_K, packed)
    else:
        cfg = QuantizationConfig()
        qw, sc, qz, gi = quantize_gptq(w)
        got = qmatmul(QE.GPTQ, cfg, a, qw, sc, qz, gi)
        words = np.sort(np.random.default_rng(m + k).choice(n // 8, 3, replace=False))
        idx = (words[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
        tidx = torch.from_numpy(idx).to(DEV)
        truth = O.matmul_gptq(a_np, qw[:, tidx].cpu().numpy(), sc[:, tidx].cpu().numpy().view(np.uint16),
                              np.ascontiguousarray(qz.cpu().numpy()[:, words]), f64=True)
        w32 = dequantize(QE.GPTQ, qw, sc, qz, gi, config=cfg)
    assert got.shape == (m, n)
    ok = O.isclose(got[:, tidx].cpu().numpy(), truth, RTOL, ATOL)
    assert ok.all(), f"{kind} {m}x{n}x{k}: {(~ok).sum()}/{ok.size} sampled outputs differ from the oracle"
    check_all(got, a.double(), w32, f"{kind} mid-size prefill {m}x{n}x{k}")


@pytest.mark.parametrize("m,n,k,bf16", [(16, 14336, 4096, False), (16, 14336, 4096, True), (4, 4096, 14336, False),
                                        (48, 4096, 14336, True), (2, 1024, 4096, True)])
def test_gptq_small_batch_full_size(m, n, k, bf16):
    """The GPTQ small-batch kernel on the projection shapes: 448 column strips on 256 workgroups (14336 x 4096), four K
    chunks with partial sums in the workspace (4096 x 14336), three passes of 16 rows (m = 48).  Sampled columns against
    the oracle's fp64 sums, every output against the fp64 product on the GPU."""
    w, gen = weights(300 + m, n, k)
    a = torch.randn((m, k), dtype=torch.float32, device=DEV, generator=gen)
    if bf16:
        a = a.to(torch.bfloat16)
    cfg = QuantizationConfig()
    qw, sc, qz, gi = quantize_gptq(w)
    got = qmatmul(QE.GPTQ, cfg, a, qw, sc, qz, gi)
    assert got.shape == (m, n)
    words = np.sort(np.random.default_rng(m + n).choice(n // 8, 6, replace=False))
    cols = (words[:, None] * 8 + np.arange(8)[None, :]).reshape(-1)
    tcols = torch.from_numpy(cols).to(DEV)
    truth = O.matmul_gptq(a.float().cpu().numpy(), qw[:, tcols].cpu().numpy(), sc[:, tcols].cpu().numpy().view(np.uint16),
                          np.ascontiguousarray(qz.cpu().numpy()[:, words]), f64=True)
    ok = O.isclose(got[:, tcols].cpu().numpy(), truth, RTOL, ATOL)
    assert ok.all(), f"GPTQ {m}x{n}x{k}: {(~ok).sum()}/{ok.size} sampled outputs differ from the oracle"
    check_all(got, a.double(), dequantize(QE.GPTQ, qw, sc, qz, gi, config=cfg), f"GPTQ small batch {m}x{n}x{k}")


@pytest.mark.parametrize("enc,m,k,period,reps", [
    (QE.Q4_K, 1, 4096, 9600, 100),    # 960 000 rows x 2304 B = 2.2 GB: the decode kernel's row offsets pass 2^31
    (QE.Q4_K, 4, 4096, 9600, 100),    # the small-batch kernel
    (QE.Q6_K, 1, 4096, 8000, 85),     # 680 000 rows x 3360 B = 2.3 GB: the vocabulary kernel
    (QE.Q4_0, 1, 4096, 9600, 100),
    (QE.Q4_0, 8, 4096, 9600, 100),
])
def test_row_offsets_beyond_two_gib(enc, m, k, period, reps):
    """A weight tensor larger than 2^31 bytes, made of `reps` copies of the same `period` rows: every copy must
    produce the same outputs, bit for bit (a row's arithmetic does not depend on where the row lies), and the first
    copy must match the oracle on sampled rows.  A byte offset computed in 32 bits anywhere fails this."""
    w, gen = weights(17, period, k)
    base = quantize(enc, w)
    packed = base.repeat(reps, 1)
    assert packed.numel() > 2**31
    a = torch.randn((m, k), dtype=torch.float32, device=DEV, generator=gen)
    got = qmatmul(enc, None, a, packed)
    assert got.shape == (m, period * reps)
    first = got[:, :period]
    assert torch.equal(got.view(m, reps, period), first.unsqueeze(1).expand(m, reps, period))
    idx = np.sort(np.random.default_rng(3).choice(period, 32, replace=False))
    tidx = torch.from_numpy(idx).to(DEV)
    a_np = a.cpu().numpy()
    a_eff = q8_0_round_trip(a_np) if enc == QE.Q4_0 else a_np
    truth = O.matmul_f64(ENC[enc], a_eff, base[tidx].cpu().numpy())
    assert O.isclose(first[:, tidx].cpu().numpy(), truth, RTOL, ATOL).all()
    # the unpacker over the same tensor: the last copy equals the first
    if m == 1:
        deq = dequantize(enc, packed[-period:])
        assert torch.equal(deq, dequantize(enc, base))
