"""ctypes front end of the CPU oracle (``libqmm_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()``
and by the ``cpu_baseline`` leg of ``bench.py`` as the checker / timed CPU
baseline.  Nothing in the shipped package may import this module.

All functions take and return NumPy arrays; layouts are the on-disk GGUF /
AutoGPTQ ones described in ``qmm_oracle.c``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libqmm_oracle.so")

Q4_0, Q4_K, Q6_K, GPTQ, Q5_K = 0, 1, 2, 3, 4
BLOCK = {Q4_0: (32, 18), Q4_K: (256, 144), Q6_K: (256, 210), Q5_K: (256, 176)}


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (``make -C oracle``)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "libqmm_oracle.so"], check=True, capture_output=True)
    return _SO


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.qo_now.restype = C.c_double
        _lib.qo_f16_to_f32.restype = C.c_float
        _lib.qo_f16_to_f32.argtypes = [C.c_uint16]
        _lib.qo_f32_to_f16.restype = C.c_uint16
        _lib.qo_f32_to_f16.argtypes = [C.c_float]
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def _i64(v):
    return C.c_int64(int(v))


# ---------------------------------------------------------------- conversions
def f16_to_f32(h) -> np.ndarray:
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().qo_f16_to_f32_n(_p(h), _i64(h.size), _p(out))
    return out


def f32_to_f16(f) -> np.ndarray:
    f = _c(f, np.float32)
    out = np.empty(f.shape, np.uint16)
    lib().qo_f32_to_f16_n(_p(f), _i64(f.size), _p(out))
    return out


def f32_to_bf16(f) -> np.ndarray:
    f = _c(f, np.float32)
    out = np.empty(f.shape, np.uint16)
    lib().qo_f32_to_bf16_n(_p(f), _i64(f.size), _p(out))
    return out


def bf16_to_f32(h) -> np.ndarray:
    return (_c(h, np.uint16).astype(np.uint32) << 16).view(np.float32)


# ---------------------------------------------------------------- quantisers
def _rows_k(x):
    x = _c(x, np.float32)
    assert x.ndim == 2
    return x, x.shape[0], x.shape[1]


def quantize(enc: int, x) -> np.ndarray:
    """fp32 [rows, K] -> uint8 [rows, K/epb*bpb] (Q4_0 / Q4_K / Q5_K / Q6_K)."""
    x, rows, k = _rows_k(x)
    epb, bpb = BLOCK[enc]
    assert k % epb == 0
    out = np.empty((rows, k // epb * bpb), np.uint8)
    fn = {Q4_0: lib().qo_quantize_q4_0, Q4_K: lib().qo_quantize_q4_k, Q6_K: lib().qo_quantize_q6_k,
          Q5_K: lib().qo_quantize_q5_k}[enc]
    fn(_p(x), _i64(rows), _i64(k), _p(out))
    return out


def quantize_q8_0(x) -> np.ndarray:
    x, rows, k = _rows_k(x)
    assert k % 32 == 0
    out = np.empty((rows, k // 32 * 34), np.uint8)
    lib().qo_quantize_q8_0(_p(x), _i64(rows), _i64(k), _p(out))
    return out


def quantize_gptq(w, group: int = 128):
    """fp32 [N, K] -> (qweight i32[K/8,N], scales f16-bits u16[K/g,N], qzeros i32[K/g,N/8], g_idx i32[K])."""
    w, n, k = _rows_k(w)
    assert k % group == 0 and k % 8 == 0 and n % 8 == 0
    qweight = np.empty((k // 8, n), np.int32)
    scales = np.empty((k // group, n), np.uint16)
    qzeros = np.empty((k // group, n // 8), np.int32)
    g_idx = np.empty((k,), np.int32)
    lib().qo_quantize_gptq(_p(w), _i64(n), _i64(k), _i64(group), _p(qweight), _p(scales), _p(qzeros), _p(g_idx))
    return qweight, scales, qzeros, g_idx


def pack_scales_q4_k(sc, mn) -> np.ndarray:
    sc, mn = _c(sc, np.uint8), _c(mn, np.uint8)
    out = np.empty(12, np.uint8)
    lib().qo_pack_scales_q4_k(_p(sc), _p(mn), _p(out))
    return out


def unpack_scales_q4_k(s):
    s = _c(s, np.uint8)
    sc, mn = np.empty(8, np.uint8), np.empty(8, np.uint8)
    lib().qo_unpack_scales_q4_k(_p(s), _p(sc), _p(mn))
    return sc, mn


# ---------------------------------------------------------------- dequantisers
def dequantize(enc: int, w, k: int) -> np.ndarray:
    w = _c(w, np.uint8)
    rows = w.shape[0]
    epb, bpb = BLOCK[enc]
    assert w.shape[1] == k // epb * bpb
    out = np.empty((rows, k), np.float32)
    rc = lib().qo_dequantize(C.c_int(enc), _p(w), _i64(rows), _i64(k), _p(out))
    assert rc == 0
    return out


def dequantize_gptq(qweight, scales, qzeros, group: int = 128, g_idx=None) -> np.ndarray:
    """-> fp32 [N, K].  g_idx int32[K] (act-order checkpoints) names the group of every k; None: k // group."""
    qweight, scales, qzeros = _c(qweight, np.int32), _c(scales, np.uint16), _c(qzeros, np.int32)
    k, n = qweight.shape[0] * 8, qweight.shape[1]
    gi = None if g_idx is None else _c(g_idx, np.int32)
    assert gi is None or gi.shape == (k,)
    out = np.empty((n, k), np.float32)
    lib().qo_dequantize_gptq(_p(qweight), _p(scales), _p(qzeros), None if gi is None else _p(gi), _i64(n), _i64(k),
                             _i64(group), _p(out))
    return out


# ---------------------------------------------------------------- matmuls
def block_dots_q4_0_q8_0(a_q8, w_q4, k: int) -> np.ndarray:
    a_q8, w_q4 = _c(a_q8, np.uint8), _c(w_q4, np.uint8)
    m, n = a_q8.shape[0], w_q4.shape[0]
    out = np.empty((m, n, k // 32), np.int32)
    lib().qo_block_dots_q4_0_q8_0(_p(a_q8), _p(w_q4), _i64(m), _i64(n), _i64(k), _p(out))
    return out


def matmul_q4_0(a, w_q4) -> np.ndarray:
    """Reference-CPU-style Q4_0 path: activations -> Q8_0, integer block dots."""
    a, m, k = _rows_k(a)
    w_q4 = _c(w_q4, np.uint8)
    n = w_q4.shape[0]
    out = np.empty((m, n), np.float32)
    lib().qo_matmul_q4_0(_p(a), _p(w_q4), _i64(m), _i64(n), _i64(k), _p(out))
    return out


def matmul_q4_0_q8_0(a_q8, w_q4, k: int) -> np.ndarray:
    a_q8, w_q4 = _c(a_q8, np.uint8), _c(w_q4, np.uint8)
    m, n = a_q8.shape[0], w_q4.shape[0]
    out = np.empty((m, n), np.float32)
    lib().qo_matmul_q4_0_q8_0(_p(a_q8), _p(w_q4), _i64(m), _i64(n), _i64(k), _p(out))
    return out


def quantize_q8_k(x) -> np.ndarray:
    """fp32 [rows, K] -> Q8_K blocks uint8 [rows, K/256*292] (float d, 256 int8 codes, 16 int16 sums of 16)."""
    x, rows, k = _rows_k(x)
    assert k % 256 == 0
    out = np.empty((rows, k // 256 * 292), np.uint8)
    lib().qo_quantize_q8_k(_p(x), _i64(rows), _i64(k), _p(out))
    return out


def block_sums_q4_k_q8_k(a_q8k, w, k: int):
    """(isum, msum) int32 [M, N, K/256]: the integer parts of the Q4_K x Q8_K dot, block by block."""
    a_q8k, w = _c(a_q8k, np.uint8), _c(w, np.uint8)
    m, n = a_q8k.shape[0], w.shape[0]
    isum, msum = np.empty((m, n, k // 256), np.int32), np.empty((m, n, k // 256), np.int32)
    lib().qo_block_sums_q4_k_q8_k(_p(a_q8k), _p(w), _i64(m), _i64(n), _i64(k), _p(isum), _p(msum))
    return isum, msum


def matmul_q4_k_q8_k(a_q8k, w, k: int) -> np.ndarray:
    a_q8k, w = _c(a_q8k, np.uint8), _c(w, np.uint8)
    m, n = a_q8k.shape[0], w.shape[0]
    out = np.empty((m, n), np.float32)
    lib().qo_matmul_q4_k_q8_k(_p(a_q8k), _p(w), _i64(m), _i64(n), _i64(k), _p(out))
    return out


def block_sums_kquant_q8_k(enc: int, a_q8k, w, k: int):
    """(isum, msum) int32 [M, N, K/256] of Q4_K / Q5_K / Q6_K blocks against Q8_K blocks (msum = 0 for Q6_K)."""
    a_q8k, w = _c(a_q8k, np.uint8), _c(w, np.uint8)
    m, n = a_q8k.shape[0], w.shape[0]
    isum, msum = np.empty((m, n, k // 256), np.int32), np.empty((m, n, k // 256), np.int32)
    rc = lib().qo_block_sums_kquant_q8_k(C.c_int(enc), _p(a_q8k), _p(w), _i64(m), _i64(n), _i64(k), _p(isum), _p(msum))
    assert rc == 0
    return isum, msum


def matmul_kquant_act_q8_k(enc: int, a, w) -> np.ndarray:
    """The integer-activation path for Q4_K / Q5_K / Q6_K weights: fp32 activations -> Q8_K, integer sub-block dots."""
    a, m, k = _rows_k(a)
    w = _c(w, np.uint8)
    n = w.shape[0]
    out = np.empty((m, n), np.float32)
    rc = lib().qo_matmul_kquant_act_q8_k(C.c_int(enc), _p(a), _p(w), _i64(m), _i64(n), _i64(k), _p(out))
    assert rc == 0
    return out


def matmul_q4_k_act_q8_k(a, w) -> np.ndarray:
    """The integer-activation Q4_K path: fp32 activations -> Q8_K, integer sub-block dots."""
    a, m, k = _rows_k(a)
    w = _c(w, np.uint8)
    n = w.shape[0]
    out = np.empty((m, n), np.float32)
    lib().qo_matmul_q4_k_act_q8_k(_p(a), _p(w), _i64(m), _i64(n), _i64(k), _p(out))
    return out


def matmul_f32(enc: int, a, w, w_bf16: bool = False) -> np.ndarray:
    a, m, k = _rows_k(a)
    w = _c(w, np.uint8)
    n = w.shape[0]
    out = np.empty((m, n), np.float32)
    rc = lib().qo_matmul_f32(C.c_int(enc), _p(a), _p(w), _i64(m), _i64(n), _i64(k), C.c_int(int(w_bf16)), _p(out))
    assert rc == 0
    return out


def baseline_matmul_q4_k(a, w, _lib=None):
    """The hand-vectorised (AVX2) Q4_K x fp32 product that ``bench.py`` times as the CPU baseline; None where the host
    lacks AVX2.  Agrees with matmul_f32 to rounding only (another summation order): never used as a checker."""
    a, m, k = _rows_k(a)
    w = _c(w, np.uint8)
    n = w.shape[0]
    out = np.empty((m, n), np.float32)
    rc = (_lib or lib()).qo_baseline_matmul_q4_k(_p(a), _p(w), _i64(m), _i64(n), _i64(k), _p(out))
    return out if rc == 0 else None


def matmul_f64(enc: int, a, w, w_bf16: bool = False) -> np.ndarray:
    a, m, k = _rows_k(a)
    w = _c(w, np.uint8)
    n = w.shape[0]
    out = np.empty((m, n), np.float64)
    rc = lib().qo_matmul_f64(C.c_int(enc), _p(a), _p(w), _i64(m), _i64(n), _i64(k), C.c_int(int(w_bf16)), _p(out))
    assert rc == 0
    return out


def matmul_gptq(a, qweight, scales, qzeros, group: int = 128, w_bf16: bool = False, f64: bool = False, g_idx=None):
    a, m, k = _rows_k(a)
    qweight, scales, qzeros = _c(qweight, np.int32), _c(scales, np.uint16), _c(qzeros, np.int32)
    n = qweight.shape[1]
    gi = None if g_idx is None else _c(g_idx, np.int32)
    assert gi is None or gi.shape == (k,)
    out = np.empty((m, n), np.float64 if f64 else np.float32)
    lib().qo_matmul_gptq_f32(
        _p(a), _p(qweight), _p(scales), _p(qzeros), None if gi is None else _p(gi), _i64(m), _i64(n), _i64(k),
        _i64(group), C.c_int(int(w_bf16)),
        None if f64 else _p(out), _p(out) if f64 else None)
    return out


def swiglu(gate, up) -> np.ndarray:
    """silu(gate) * up in fp64, silu(x) = x / (1 + exp(-x)): the gated-MLP combination of two matmul results."""
    g = np.asarray(gate, np.float64)
    with np.errstate(over="ignore"):
        return g / (1.0 + np.exp(-g)) * np.asarray(up, np.float64)


def rmsnorm(x, gamma, eps: float, to_bf16: bool = False) -> np.ndarray:
    """y = x * rsqrt(mean(x^2) + eps) * gamma per row, fp32 (rounded to bf16 and widened again with to_bf16)."""
    x = _c(x, np.float32)
    rows, k = (1, x.shape[0]) if x.ndim == 1 else x.shape
    gamma = _c(gamma, np.float32)
    assert gamma.shape == (k,)
    y = np.empty(x.shape, np.float32)
    lib().qo_rmsnorm(_p(x), _p(gamma), C.c_float(eps), _i64(rows), _i64(k), C.c_int(int(to_bf16)), _p(y))
    return y


class _Native:
    """The same source built with -march=native (``make -C oracle native``): only the timed CPU baseline of
    ``bench.py`` uses it, never a test."""

    def __init__(self, path: str):
        self._lib = C.CDLL(path)

    def set_num_threads(self, n: int) -> None:
        self._lib.qo_set_num_threads(C.c_int(n))

    def matmul_f32(self, enc: int, a, w) -> np.ndarray:
        a, m, k = _rows_k(a)
        w = _c(w, np.uint8)
        n = w.shape[0]
        out = np.empty((m, n), np.float32)
        rc = self._lib.qo_matmul_f32(C.c_int(enc), _p(a), _p(w), _i64(m), _i64(n), _i64(k), C.c_int(0), _p(out))
        assert rc == 0
        return out

    def baseline_matmul_q4_k(self, a, w):
        return baseline_matmul_q4_k(a, w, self._lib)


def native() -> _Native:
    return _Native(os.path.join(_HERE, "_native", "libqmm_oracle_native.so"))


def num_threads() -> int:
    return int(lib().qo_num_threads())


def set_num_threads(n: int) -> None:
    lib().qo_set_num_threads(C.c_int(n))


def now() -> float:
    return float(lib().qo_now())


def isclose(a, b, rtol=1e-3, atol=1e-4) -> np.ndarray:
    """Symmetric closeness of the reference (stdlib/src/math/math.mojo:1023-1030):
    a == b or (both finite and |a-b| <= max(atol, rtol*max(|a|,|b|)))."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    fin = np.isfinite(a) & np.isfinite(b)
    with np.errstate(invalid="ignore"):
        close = np.abs(a - b) <= np.maximum(atol, rtol * np.maximum(np.abs(a), np.abs(b)))
    return (a == b) | (fin & close)
