"""qmm_matmul_static (scratch in the library's own static device buffer, nothing allocated) against qmm_matmul
(scratch in a caller tensor): same kernels, so the fp32 outputs must be bit-identical.  Called through the C ABI.

Collected last on purpose: the two calls per case share the static buffer with whatever ran before.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle as O
from conftest import synth
from mojo_amd import QuantizationConfig, QuantizationEncoding as QE, _lib, qmatmul

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def gpu(x):
    return torch.from_numpy(np.ascontiguousarray(x)).to(DEV)


def _call(static, enc, cfg, lhs, rhs, n):
    """One raw call of either entry point; returns the output tensor."""
    lib = _lib.load()
    m, k = lhs.shape
    dt = _lib.QMM_F32 if lhs.dtype == torch.float32 else _lib.QMM_BF16
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV)
    ptrs = (C.c_void_p * len(rhs))(*[t.data_ptr() for t in rhs])
    cfg_p = C.byref(cfg) if cfg is not None else None
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    if static:
        rc = lib.qmm_matmul_static(enc, cfg_p, C.c_void_p(lhs.data_ptr()), dt, m, k, ptrs, len(rhs), n,
                                   C.c_void_p(out.data_ptr()), 0, stream)
    else:
        need = lib.qmm_matmul_workspace_bytes(enc, dt, m, n, k)
        ws = torch.empty((max(need, 1),), dtype=torch.uint8, device=DEV)
        rc = lib.qmm_matmul(enc, cfg_p, C.c_void_p(lhs.data_ptr()), dt, m, k, ptrs, len(rhs), n,
                            C.c_void_p(out.data_ptr()), C.c_void_p(ws.data_ptr()), need, 0, stream)
    assert rc == 0, lib.qmm_last_error()
    torch.cuda.synchronize()
    return out


def _case(enc, m, n, k, bf16, seed):
    w, a = synth(seed, n, k, m)
    lhs = gpu(a).to(torch.bfloat16) if bf16 else gpu(a)
    if enc == QE.GPTQ:
        qw, sc, qz, _ = O.quantize_gptq(w)
        return lhs, [gpu(qw), gpu(sc.view(np.float16)), gpu(qz)], _lib.GptqConfig(4, 128, 0, 1), a, (qw, sc, qz)
    wq = O.quantize({QE.Q4_0: O.Q4_0, QE.Q4_K: O.Q4_K}[enc], w)
    return lhs, [gpu(wq)], None, a, wq


# every case needs scratch: Q8_0 planes (Q4_0), fp16 lhs planes (Q4_K / GPTQ from 9 / 17 rows), K-chunk partial sums
@pytest.mark.parametrize("enc,big,small", [
    (QE.Q4_0, (64, 520, 2048, False), (7, 130, 512, False)),
    (QE.Q4_K, (200, 520, 2048, True), (12, 130, 512, False)),
    (QE.Q4_K, (16, 72, 8192, False), (9, 33, 4352, True)),
    (QE.GPTQ, (130, 264, 1024, True), (33, 64, 512, False)),
])
def test_static_scratch_calls_match_workspace_calls(enc, big, small):
    """Two calls in a row on the shared static buffer, the second smaller than the first: each equals the
    caller-workspace call bit for bit, and the oracle within the matmul tolerance."""
    lib = _lib.load()
    for i, (m, n, k, bf16) in enumerate((big, small)):
        lhs, rhs, cfg, a, packed = _case(enc, m, n, k, bf16, seed=50 + i)
        dt = _lib.QMM_F32 if lhs.dtype == torch.float32 else _lib.QMM_BF16
        assert lib.qmm_matmul_workspace_bytes(enc.code, dt, m, n, k) > 0, "case does not exercise the scratch buffer"
        got = _call(True, enc.code, cfg, lhs, rhs, n)
        want = _call(False, enc.code, cfg, lhs, rhs, n)
        assert torch.equal(got, want), f"{enc.name} {m}x{n}x{k}: static-scratch output differs from the workspace call"
        af = O.bf16_to_f32(O.f32_to_bf16(a)) if bf16 else a
        if enc == QE.Q4_0:
            ref = O.matmul_q4_0(af, packed)
        elif enc == QE.Q4_K:
            ref = O.matmul_f32(O.Q4_K, af, packed)
        else:
            ref = O.matmul_gptq(af, *packed)
        assert O.isclose(got.cpu().numpy(), ref, 1e-3, 1e-4).all()


def test_static_scratch_through_the_python_mirror():
    w, a = synth(60, 200, 1024, 40)
    wq = gpu(O.quantize(O.Q4_0, w))
    out = torch.empty((40, 200), dtype=torch.float32, device=DEV)
    got = qmatmul(QE.Q4_0, None, gpu(a), wq, out=out, static_scratch=True)
    assert got.data_ptr() == out.data_ptr()
    assert torch.equal(got, qmatmul(QE.Q4_0, None, gpu(a), wq))


def test_static_scratch_rejects_what_does_not_fit():
    """More scratch than the static buffer holds: a status and a message, no launch (pointers are never read)."""
    lib = _lib.load()
    m, n, k = 8192, 4096, 8192  # fp32 lhs planes of a Q4_K prefill: 2 x 128 MiB
    assert lib.qmm_matmul_workspace_bytes(1, 0, m, n, k) > _lib.QMM_STATIC_SCRATCH_BYTES
    fake = C.c_void_p(0x10000)
    rhs = (C.c_void_p * 1)(0x20000)
    assert lib.qmm_matmul_static(1, None, fake, 0, m, k, rhs, 1, n, fake, 0, None) == -4
    assert b"static buffer" in lib.qmm_last_error()


def test_static_scratch_inside_a_captured_graph_and_with_bf16_output():
    """The stated use: after one call outside capture (the first call on a device looks the buffer's address up and sets
    kernel attributes), the entry point is recorded into a HIP graph and replayed, with the program's own eager work between
    the replays; every replay equals the eager call bit for bit.  With QMM_FLAG_OUT_BF16 the fp32 result sits in the static
    buffer on the way."""
    lib = _lib.load()
    m, n, k = 12, 130, 2048
    w, a = synth(61, n, k, m)
    wq = gpu(O.quantize(O.Q4_K, w))
    lhs = gpu(a)
    ptrs = (C.c_void_p * 1)(wq.data_ptr())
    for flags, dtype in ((0, torch.float32), (_lib.QMM_FLAG_OUT_BF16, torch.bfloat16)):
        out = torch.zeros((m, n), dtype=dtype, device=DEV)

        def call(stream):
            rc = lib.qmm_matmul_static(QE.Q4_K.code, None, C.c_void_p(lhs.data_ptr()), _lib.QMM_F32, m, k, ptrs, 1, n,
                                       C.c_void_p(out.data_ptr()), flags, C.c_void_p(stream))
            assert rc == 0, lib.qmm_last_error()

        call(torch.cuda.current_stream().cuda_stream)  # outside capture first
        torch.cuda.synchronize()
        eager = out.clone()
        g = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                call(torch.cuda.current_stream().cuda_stream)
        torch.cuda.current_stream().wait_stream(side)
        for i in range(3):
            out.zero_()
            other = qmatmul(QE.Q4_K, None, lhs[: 1 + i], wq)  # eager work of the program between the replays
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), f"replay {i} differs from the eager call (flags {flags})"
            assert other.shape == (1 + i, n)
    want = O.matmul_f32(O.Q4_K, a, O.quantize(O.Q4_K, w))
    assert O.isclose(eager.float().cpu().numpy(), O.bf16_to_f32(O.f32_to_bf16(want)), 1e-2, 1e-3).all()
