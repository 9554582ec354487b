"""Host side of ``qmatmul``: shape/dtype checks, tensor allocation, C-ABI calls.

PyTorch is used only to allocate device memory and to name the stream; every
number is produced by the HIP kernels in ``libqmm.so``.
"""
from __future__ import annotations

import ctypes as C
from typing import List, Optional, Sequence

import torch

from . import _lib
from .quantization import QuantizationConfig, QuantizationEncoding

_DTYPES = {torch.float32: _lib.QMM_F32, torch.bfloat16: _lib.QMM_BF16}


def _stream(t: torch.Tensor) -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _require_gpu(t: torch.Tensor, name: str) -> None:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got device {t.device}); there is no CPU path")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def _ptr(t: Optional[torch.Tensor]) -> C.c_void_p:
    return C.c_void_p(0 if t is None else t.data_ptr())


def _gptq_cfg(config: Optional[QuantizationConfig]) -> _lib.GptqConfig:
    if config is None:
        raise ValueError("GPTQ needs a QuantizationConfig")
    if config.quant_method != "gptq":
        raise ValueError(f"unsupported quant_method {config.quant_method!r}")
    return _lib.GptqConfig(int(config.bits), int(config.group_size), int(bool(config.desc_act)), int(bool(config.sym)))


def _check_rhs(encoding: QuantizationEncoding, config: Optional[QuantizationConfig], k: int, rhs):
    """Validates the weight tensors of a qmatmul against the encoding and K; returns (N, pointer to the GPTQ config or None)."""
    if encoding == QuantizationEncoding.GPTQ:
        if len(rhs) not in (3, 4):
            raise TypeError(f"GPTQ qmatmul takes (qweight, scales, qzeros[, g_idx]); got {len(rhs)} rhs tensors")
        qweight, scales, qzeros = rhs[:3]
        for t, name, dt in ((qweight, "qweight", torch.int32), (scales, "scales", torch.float16),
                            (qzeros, "qzeros", torch.int32)):
            _require_gpu(t, name)
            if t.dtype != dt or t.dim() != 2:
                raise TypeError(f"{name} must be a rank-2 {dt} tensor")
        n = qweight.shape[1]
        cfg = _gptq_cfg(config)
        g = cfg.group_size
        if qweight.shape[0] * 8 != k:
            raise ValueError(f"qweight has K={qweight.shape[0] * 8}, lhs has K={k}")
        if g <= 0 or k % g or tuple(scales.shape) != (k // g, n) or tuple(qzeros.shape) != (k // g, n // 8):
            raise ValueError("scales/qzeros shapes do not match (K/group, N) and (K/group, N/8)")
        if len(rhs) == 4:
            _require_gpu(rhs[3], "g_idx")
            if rhs[3].dtype != torch.int32 or tuple(rhs[3].shape) != (k,):
                raise TypeError("g_idx must be int32[K]")
        elif cfg.desc_act:
            raise TypeError("GPTQ with desc_act=True needs g_idx as the fourth rhs tensor")
        cfg_p = C.byref(cfg)
    elif encoding.is_gguf:
        if len(rhs) != 1:
            raise TypeError(f"{encoding.name} qmatmul takes exactly one rhs tensor; got {len(rhs)}")
        (w,) = rhs
        _require_gpu(w, "rhs")
        if w.dtype != torch.uint8 or w.dim() != 2:
            raise TypeError("rhs must be a rank-2 uint8 tensor of packed blocks")
        n = w.shape[0]
        if w.shape[1] != encoding.packed_row_bytes(k):
            raise ValueError(
                f"rhs rows hold {w.shape[1]} bytes; K={k} in {encoding.name} needs {encoding.packed_row_bytes(k)}")
        cfg_p = None
    else:
        raise ValueError(f"{encoding.name} is not a weight encoding of qmatmul")
    return n, cfg_p


def qmatmul(encoding: QuantizationEncoding, config: Optional[QuantizationConfig], lhs: torch.Tensor,
            *rhs: torch.Tensor, w_bf16: bool = False, act_q8k: bool = False, out: Optional[torch.Tensor] = None,
            static_scratch: bool = False, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """``out[..., N] = lhs[..., K] @ dequantize(rhs)^T`` in fp32.

    ``out_dtype=torch.bfloat16`` returns the fp32 result rounded to bfloat16 (nearest even, canonical NaN:
    the narrowing rule of stdlib/src/builtin/simd.mojo:3279-3300) for a consumer that takes bf16 activations; the
    Q4_K decode kernel stores it directly, other shapes narrow an fp32 result held in the workspace.

    GGUF encodings take one ``uint8[N, K/epb*bpb]`` tensor of packed blocks (the
    transposed, quantised weight).  GPTQ takes the AutoGPTQ tensors
    ``(qweight int32[K/8, N], scales float16[K/g, N], qzeros int32[K/g, N/8][, g_idx int32[K]])``.
    ``lhs`` is float32 or bfloat16.  Q4_0 quantises ``lhs`` to Q8_0 blocks and
    takes integer block dots; the other encodings use ``lhs`` as given.  ``act_q8k=True`` (Q4_K, Q5_K,
    Q6_K) quantises ``lhs`` to Q8_K blocks and takes the products of the ggml-lineage CPU kernels' integer sub-block dots instead
    (integer sums in the kernel up to 16 lhs rows; beyond that the same products summed in fp32).
    ``w_bf16=True`` asks for the reserved mode that rounds the dequantised weights to bfloat16 first; the library
    has no kernel for it and raises ``NotImplementedError``.

    ``out`` (contiguous float32 ``[M, N]`` on the device of ``lhs``) receives the result instead of a new tensor.
    ``static_scratch=True`` goes through ``qmm_matmul_static``: the kernels' scratch is the buffer that is part of
    the library (64 MiB per GPU) instead of a tensor allocated here, so with ``out`` given the call allocates no
    device memory; calls that may overlap on one GPU must then be ordered by the caller.
    """
    if not isinstance(encoding, QuantizationEncoding):
        raise TypeError("encoding must be a QuantizationEncoding")
    _require_gpu(lhs, "lhs")
    if lhs.dtype not in _DTYPES:
        raise TypeError(f"lhs must be float32 or bfloat16, got {lhs.dtype}")
    if lhs.dim() < 1:
        raise ValueError("lhs must have at least one dimension")
    k = lhs.shape[-1]
    lead = lhs.shape[:-1]
    m = 1
    for d in lead:
        m *= d
    lib = _lib.load()
    n, cfg_p = _check_rhs(encoding, config, k, rhs)
    if m == 0 or n == 0:
        raise ValueError("qmatmul of an empty tensor")
    if out_dtype not in (torch.float32, torch.bfloat16):
        raise TypeError("out_dtype must be float32 or bfloat16")
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=lhs.device)
    else:
        _require_gpu(out, "out")
        if out.dtype != out_dtype or out.numel() != m * n or out.device != lhs.device:
            raise TypeError(f"out must be a contiguous {out_dtype} tensor of {m} x {n} elements on the device of lhs")
    lhs_dt = _DTYPES[lhs.dtype]
    flags = ((_lib.QMM_FLAG_W_BF16 if w_bf16 else 0) | (_lib.QMM_FLAG_ACT_Q8K if act_q8k else 0) |
             (_lib.QMM_FLAG_OUT_BF16 if out_dtype == torch.bfloat16 else 0))
    ptrs = (C.c_void_p * len(rhs))(*[t.data_ptr() for t in rhs])
    if static_scratch:
        rc = lib.qmm_matmul_static(encoding.code, cfg_p, _ptr(lhs), lhs_dt, m, k, ptrs, len(rhs), n, _ptr(out), flags,
                                   _stream(lhs))
    else:
        need = lib.qmm_matmul_workspace_bytes_flags(encoding.code, lhs_dt, m, n, k, flags)
        ws = torch.empty((need,), dtype=torch.uint8, device=lhs.device) if need > 0 else None
        rc = lib.qmm_matmul(encoding.code, cfg_p, _ptr(lhs), lhs_dt, m, k, ptrs, len(rhs), n, _ptr(out), _ptr(ws),
                            need, flags, _stream(lhs))
    if rc == -4:
        raise ValueError("qmatmul: " + lib.qmm_last_error().decode("utf-8", "replace"))
    _lib.check(rc, "qmatmul")
    return out.reshape(*lead, n)


class RepackedWeights:
    """The weights of one matrix as the plane GEMMs read them, made once by :func:`repack_weights` (an explicit form
    of the weight repack step that MAX is understood to fold into model load: external knowledge, the reference snapshot
    holds no MAX code).  ``rhs`` are the packed tensors the planes were made from, or
    an empty tuple if the caller does not keep them (then every row count goes through the planes)."""

    __slots__ = ("encoding", "config", "n", "k", "packed", "rhs")

    def __init__(self, encoding, config, n, k, packed, rhs):
        self.encoding, self.config, self.n, self.k, self.packed, self.rhs = encoding, config, n, k, packed, tuple(rhs)


def _k_of(encoding: QuantizationEncoding, rhs) -> int:
    if encoding == QuantizationEncoding.GPTQ:
        return rhs[0].shape[0] * 8
    bp = encoding.block_parameters
    return rhs[0].shape[1] // bp.block_size * bp.elements_per_block


def repack_weights(encoding: QuantizationEncoding, config: Optional[QuantizationConfig], *rhs: torch.Tensor,
                   keep_rhs: bool = True) -> RepackedWeights:
    """Converts the packed weights of one matrix (the ``rhs`` of :func:`qmatmul`) into fp16 integer planes and scale tables,
    once, for :func:`qmatmul_repacked`.  Q4_0, Q4_K, Q5_K, Q6_K and GPTQ with plain groups of 128 or 256 (K a multiple of 256);
    other encodings raise ``NotImplementedError``.  The planes take 2 bytes per weight (Q6_K 4)."""
    if not isinstance(encoding, QuantizationEncoding):
        raise TypeError("encoding must be a QuantizationEncoding")
    if not rhs or not isinstance(rhs[0], torch.Tensor) or rhs[0].dim() != 2:
        raise TypeError("repack_weights takes the rhs tensors of qmatmul")
    if not (encoding.is_gguf or encoding == QuantizationEncoding.GPTQ):
        raise ValueError(f"{encoding.name} is not a weight encoding of qmatmul")
    k = _k_of(encoding, rhs)
    n, cfg_p = _check_rhs(encoding, config, k, rhs)
    lib = _lib.load()
    size = lib.qmm_repack_bytes(encoding.code, cfg_p, n, k)
    if size <= 0:
        raise NotImplementedError(f"repack_weights: no weight planes for {encoding.name} with N={n}, K={k}")
    packed = torch.empty((size,), dtype=torch.uint8, device=rhs[0].device)
    ptrs = (C.c_void_p * len(rhs))(*[t.data_ptr() for t in rhs])
    _lib.check(lib.qmm_repack(encoding.code, cfg_p, ptrs, len(rhs), n, k, _ptr(packed), size, _stream(rhs[0])), "repack_weights")
    return RepackedWeights(encoding, config, n, k, packed, rhs if keep_rhs else ())


def qmatmul_repacked(lhs: torch.Tensor, weights: RepackedWeights, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """:func:`qmatmul` on weights converted beforehand: the same fp32 result, without the conversion pass that the prefill
    GEMMs of :func:`qmatmul` run per call.  Row counts that the decode kernels serve go to them (on ``weights.rhs``)."""
    if not isinstance(weights, RepackedWeights):
        raise TypeError("weights must come from repack_weights")
    _require_gpu(lhs, "lhs")
    if lhs.dtype not in _DTYPES:
        raise TypeError(f"lhs must be float32 or bfloat16, got {lhs.dtype}")
    if lhs.dim() < 1 or lhs.shape[-1] != weights.k:
        raise ValueError(f"lhs must end in K={weights.k}")
    if lhs.device != weights.packed.device:
        raise ValueError("lhs and the repacked weights must be on one device")
    lead = lhs.shape[:-1]
    m = 1
    for d in lead:
        m *= d
    if m == 0:
        raise ValueError("qmatmul of an empty tensor")
    n, k, enc = weights.n, weights.k, weights.encoding
    if out is None:
        out = torch.empty((m, n), dtype=torch.float32, device=lhs.device)
    else:
        _require_gpu(out, "out")
        if out.dtype != torch.float32 or out.numel() != m * n or out.device != lhs.device:
            raise TypeError(f"out must be a contiguous float32 tensor of {m} x {n} elements on the device of lhs")
    lib = _lib.load()
    cfg_p = C.byref(_gptq_cfg(weights.config)) if enc == QuantizationEncoding.GPTQ else None
    lhs_dt = _DTYPES[lhs.dtype]
    need = lib.qmm_matmul_repacked_workspace_bytes(enc.code, lhs_dt, m, n, k)
    ws = torch.empty((need,), dtype=torch.uint8, device=lhs.device) if need > 0 else None
    ptrs = (C.c_void_p * len(weights.rhs))(*[t.data_ptr() for t in weights.rhs]) if weights.rhs else None
    rc = lib.qmm_matmul_repacked(enc.code, cfg_p, _ptr(lhs), lhs_dt, m, k, ptrs, len(weights.rhs), _ptr(weights.packed),
                                 weights.packed.numel(), n, _ptr(out), _ptr(ws), need, 0, _stream(lhs))
    _lib.check(rc, "qmatmul_repacked")
    return out.reshape(*lead, n)


def qmatmul_rmsnorm(encoding: QuantizationEncoding, config: Optional[QuantizationConfig], x: torch.Tensor,
                    gamma: torch.Tensor, eps: float, *rhs: torch.Tensor, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """``qmatmul(encoding, config, rms_norm(x, gamma, eps), *rhs)`` as one call: the normalisation in front of the
    projections of a Llama block, ``y = x * rsqrt(mean(x^2) + eps) * gamma`` in fp32 (rounded to bfloat16 when ``x`` is
    bfloat16).  Q4_0 with up to four rows (K <= 8192) is one launch: the decode kernel normalises the rows it quantises
    to Q8_0 anyway; other problems run a normalisation launch and the matmul inside the library."""
    if not isinstance(encoding, QuantizationEncoding):
        raise TypeError("encoding must be a QuantizationEncoding")
    _require_gpu(x, "x")
    _require_gpu(gamma, "gamma")
    if x.dtype not in _DTYPES:
        raise TypeError(f"x must be float32 or bfloat16, got {x.dtype}")
    if x.dim() < 1:
        raise ValueError("x must have at least one dimension")
    k = x.shape[-1]
    if gamma.dtype != torch.float32 or tuple(gamma.shape) != (k,):
        raise TypeError(f"gamma must be float32[{k}]")
    if not eps >= 0.0:
        raise ValueError("eps must be non-negative")
    if out_dtype not in (torch.float32, torch.bfloat16):
        raise TypeError("out_dtype must be float32 or bfloat16")
    lead = x.shape[:-1]
    m = 1
    for d in lead:
        m *= d
    n, cfg_p = _check_rhs(encoding, config, k, rhs)
    if m == 0 or n == 0:
        raise ValueError("qmatmul of an empty tensor")
    lib = _lib.load()
    x_dt = _DTYPES[x.dtype]
    flags = _lib.QMM_FLAG_OUT_BF16 if out_dtype == torch.bfloat16 else 0
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    need = lib.qmm_matmul_rmsnorm_workspace_bytes(encoding.code, x_dt, m, n, k, flags)
    ws = torch.empty((need,), dtype=torch.uint8, device=x.device) if need > 0 else None
    ptrs = (C.c_void_p * len(rhs))(*[t.data_ptr() for t in rhs])
    rc = lib.qmm_matmul_rmsnorm(encoding.code, cfg_p, _ptr(x), x_dt, _ptr(gamma), C.c_float(eps), m, k, ptrs, len(rhs), n,
                                _ptr(out), _ptr(ws), need, flags, _stream(x))
    _lib.check(rc, "qmatmul_rmsnorm")
    return out.reshape(*lead, n)


def qmatmul_grouped(encoding: QuantizationEncoding, lhs: torch.Tensor, rhs: Sequence[torch.Tensor]) -> List[torch.Tensor]:
    """``[lhs @ dequantize(w)^T for w in rhs]`` for GGUF weight matrices that share ``lhs`` (q | k | v, gate | up).

    One launch where a kernel takes the whole group (Q4_K, a single lhs row, up to four matrices); otherwise
    the library runs one matmul per matrix.  Results are those of ``qmatmul`` on each matrix.
    """
    if not isinstance(encoding, QuantizationEncoding) or not encoding.is_gguf:
        raise TypeError("qmatmul_grouped takes a GGUF weight encoding")
    rhs = list(rhs)
    if not rhs:
        raise ValueError("qmatmul_grouped needs at least one rhs tensor")
    _require_gpu(lhs, "lhs")
    if lhs.dtype not in _DTYPES:
        raise TypeError(f"lhs must be float32 or bfloat16, got {lhs.dtype}")
    k = lhs.shape[-1]
    lead = lhs.shape[:-1]
    m = 1
    for d in lead:
        m *= d
    if m == 0:
        raise ValueError("qmatmul of an empty tensor")
    for w in rhs:
        _require_gpu(w, "rhs")
        if w.dtype != torch.uint8 or w.dim() != 2 or w.shape[0] == 0:
            raise TypeError("every rhs must be a non-empty rank-2 uint8 tensor of packed blocks")
        if w.shape[1] != encoding.packed_row_bytes(k):
            raise ValueError(
                f"rhs rows hold {w.shape[1]} bytes; K={k} in {encoding.name} needs {encoding.packed_row_bytes(k)}")
    lib = _lib.load()
    lhs_dt = _DTYPES[lhs.dtype]
    outs = [torch.empty((m, w.shape[0]), dtype=torch.float32, device=lhs.device) for w in rhs]
    need = max(lib.qmm_matmul_workspace_bytes(encoding.code, lhs_dt, m, w.shape[0], k) for w in rhs)
    ws = torch.empty((need,), dtype=torch.uint8, device=lhs.device) if need > 0 else None
    count = len(rhs)
    rhs_p = (C.c_void_p * count)(*[w.data_ptr() for w in rhs])
    out_p = (C.c_void_p * count)(*[o.data_ptr() for o in outs])
    n_p = (C.c_int64 * count)(*[w.shape[0] for w in rhs])
    rc = lib.qmm_matmul_grouped(encoding.code, _ptr(lhs), lhs_dt, m, k, count, rhs_p, n_p, out_p, _ptr(ws), need, _stream(lhs))
    _lib.check(rc, "qmatmul_grouped")
    return [o.reshape(*lead, o.shape[1]) for o in outs]


def qmatmul_swiglu(encoding: QuantizationEncoding, lhs: torch.Tensor, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``silu(lhs @ dequantize(gate)^T) * (lhs @ dequantize(up)^T)``: the gated-MLP step around two ``qmatmul`` calls.

    ``gate`` and ``up`` are packed GGUF tensors ``uint8[N, K/epb*bpb]`` of one encoding.  Q4_K with a single lhs row
    runs as one launch (the combination is the decode kernel's epilogue); other shapes run two matmuls and a
    combining kernel inside the library.
    """
    if not isinstance(encoding, QuantizationEncoding) or not encoding.is_gguf:
        raise TypeError("qmatmul_swiglu takes a GGUF weight encoding")
    _require_gpu(lhs, "lhs")
    if lhs.dtype not in _DTYPES:
        raise TypeError(f"lhs must be float32 or bfloat16, got {lhs.dtype}")
    k = lhs.shape[-1]
    lead = lhs.shape[:-1]
    m = 1
    for d in lead:
        m *= d
    if m == 0:
        raise ValueError("qmatmul of an empty tensor")
    for w, name in ((gate, "gate"), (up, "up")):
        _require_gpu(w, name)
        if w.dtype != torch.uint8 or w.dim() != 2 or w.shape[0] == 0:
            raise TypeError(f"{name} must be a non-empty rank-2 uint8 tensor of packed blocks")
        if w.shape[1] != encoding.packed_row_bytes(k):
            raise ValueError(
                f"{name} rows hold {w.shape[1]} bytes; K={k} in {encoding.name} needs {encoding.packed_row_bytes(k)}")
    if gate.shape != up.shape:
        raise ValueError(f"gate {tuple(gate.shape)} and up {tuple(up.shape)} must have the same shape")
    n = gate.shape[0]
    lib = _lib.load()
    lhs_dt = _DTYPES[lhs.dtype]
    out = torch.empty((m, n), dtype=torch.float32, device=lhs.device)
    need = lib.qmm_matmul_swiglu_workspace_bytes(encoding.code, lhs_dt, m, n, k)
    ws = torch.empty((need,), dtype=torch.uint8, device=lhs.device) if need > 0 else None
    rc = lib.qmm_matmul_swiglu(encoding.code, _ptr(lhs), lhs_dt, m, k, _ptr(gate), _ptr(up), n, _ptr(out), _ptr(ws), need,
                               _stream(lhs))
    _lib.check(rc, "qmatmul_swiglu")
    return out.reshape(*lead, n)


def dequantize(encoding: QuantizationEncoding, *quantized: torch.Tensor, k: Optional[int] = None,
               config: Optional[QuantizationConfig] = None, dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Unpack ``uint8[N, K/epb*bpb]`` blocks (or GPTQ tensors) to ``dtype[N, K]``."""
    if dtype not in _DTYPES:
        raise TypeError("dtype must be float32 or bfloat16")
    lib = _lib.load()
    if encoding == QuantizationEncoding.GPTQ:
        if len(quantized) not in (3, 4):
            raise TypeError("GPTQ dequantize takes (qweight, scales, qzeros[, g_idx])")
        for t in quantized:
            _require_gpu(t, "GPTQ tensor")
        qweight, scales, qzeros = quantized[:3]
        g_idx = quantized[3] if len(quantized) == 4 else None
        cfg = _gptq_cfg(config)
        for t, name, dt in ((qweight, "qweight", torch.int32), (scales, "scales", torch.float16), (qzeros, "qzeros", torch.int32)):
            if t.dtype != dt or t.dim() != 2:
                raise TypeError(f"{name} must be a rank-2 {dt} tensor")
        kk, n = qweight.shape[0] * 8, qweight.shape[1]
        g = cfg.group_size
        # (a group size smaller than the checkpoint's would make the kernel read scales and qzeros past their end)
        if g <= 0 or kk % g or n % 8 or tuple(scales.shape) != (kk // g, n) or tuple(qzeros.shape) != (kk // g, n // 8):
            raise ValueError("scales/qzeros shapes do not match (K/group, N) and (K/group, N/8) of this config")
        if g_idx is not None and (g_idx.dtype != torch.int32 or tuple(g_idx.shape) != (kk,)):
            raise TypeError("g_idx must be int32[K]")
        if g_idx is None and cfg.desc_act:
            raise TypeError("GPTQ with desc_act=True needs g_idx")
        out = torch.empty((n, kk), dtype=dtype, device=qweight.device)
        rc = lib.qmm_dequantize_gptq(C.byref(cfg), _ptr(qweight), _ptr(scales), _ptr(qzeros), _ptr(g_idx), n, kk,
                                     _ptr(out), _DTYPES[dtype], _stream(qweight))
        _lib.check(rc, "dequantize")
        return out
    if not encoding.is_gguf:
        raise ValueError(f"{encoding.name} cannot be dequantized here")
    (w,) = quantized
    _require_gpu(w, "quantized")
    if w.dtype != torch.uint8 or w.dim() != 2:
        raise TypeError("quantized must be a rank-2 uint8 tensor")
    bp = encoding.block_parameters
    if w.shape[1] % bp.block_size:
        raise ValueError(f"row length {w.shape[1]} is not a multiple of the {encoding.name} block size {bp.block_size}")
    kk = w.shape[1] // bp.block_size * bp.elements_per_block
    if k is not None and k != kk:
        raise ValueError(f"K={k} does not match the packed row length (K={kk})")
    n = w.shape[0]
    if n == 0 or kk == 0:
        raise ValueError("dequantize of an empty tensor")
    out = torch.empty((n, kk), dtype=dtype, device=w.device)
    rc = lib.qmm_dequantize(encoding.code, _ptr(w), n, kk, _ptr(out), _DTYPES[dtype], _stream(w))
    _lib.check(rc, "dequantize")
    return out


def quantize(encoding: QuantizationEncoding, x: torch.Tensor) -> torch.Tensor:
    """fp32 ``[rows, K]`` -> packed ``uint8[rows, K/epb*bpb]`` (Q4_0, Q8_0, Q8_K, Q4_K, Q5_K, Q6_K)."""
    _require_gpu(x, "x")
    if x.dtype != torch.float32 or x.dim() != 2:
        raise TypeError("x must be a rank-2 float32 tensor")
    rows, k = x.shape
    out = torch.empty((rows, encoding.packed_row_bytes(k)), dtype=torch.uint8, device=x.device)
    if rows == 0 or k == 0:
        raise ValueError("quantize of an empty tensor")
    rc = _lib.load().qmm_quantize(encoding.code, _ptr(x), rows, k, _ptr(out), _stream(x))
    _lib.check(rc, "quantize")
    return out


def quantize_gptq(w: torch.Tensor, config: QuantizationConfig = QuantizationConfig()) -> Sequence[torch.Tensor]:
    """fp32 ``[N, K]`` -> ``(qweight, scales, qzeros, g_idx)`` in the AutoGPTQ v1 layout."""
    _require_gpu(w, "w")
    if w.dtype != torch.float32 or w.dim() != 2:
        raise TypeError("w must be a rank-2 float32 tensor")
    n, k = w.shape
    cfg = _gptq_cfg(config)
    g = cfg.group_size
    if g <= 0 or k % g or k % 8 or n % 8:
        raise ValueError("GPTQ needs K % group_size == 0 and N % 8 == 0")
    dev = w.device
    qweight = torch.empty((k // 8, n), dtype=torch.int32, device=dev)
    scales = torch.empty((k // g, n), dtype=torch.float16, device=dev)
    qzeros = torch.empty((k // g, n // 8), dtype=torch.int32, device=dev)
    g_idx = torch.empty((k,), dtype=torch.int32, device=dev)
    rc = _lib.load().qmm_quantize_gptq(C.byref(cfg), _ptr(w), n, k, _ptr(qweight), _ptr(scales), _ptr(qzeros),
                                       _ptr(g_idx), _stream(w))
    _lib.check(rc, "quantize_gptq")
    return qweight, scales, qzeros, g_idx


def block_dots_q4_0(lhs_q8_0: torch.Tensor, rhs_q4_0: torch.Tensor) -> torch.Tensor:
    """Raw int32 block sums ``[M, N, K/32]`` of Q8_0 lhs blocks against Q4_0 rhs blocks."""
    _require_gpu(lhs_q8_0, "lhs_q8_0")
    _require_gpu(rhs_q4_0, "rhs_q4_0")
    if lhs_q8_0.dtype != torch.uint8 or rhs_q4_0.dtype != torch.uint8:
        raise TypeError("both operands must be uint8 block tensors")
    m, n = lhs_q8_0.shape[0], rhs_q4_0.shape[0]
    if lhs_q8_0.shape[1] % 34 or rhs_q4_0.shape[1] % 18 or lhs_q8_0.shape[1] // 34 != rhs_q4_0.shape[1] // 18:
        raise ValueError("operands disagree on K")
    nb = rhs_q4_0.shape[1] // 18
    out = torch.empty((m, n, nb), dtype=torch.int32, device=rhs_q4_0.device)
    rc = _lib.load().qmm_block_dots_q4_0(_ptr(lhs_q8_0), _ptr(rhs_q4_0), m, n, nb * 32, _ptr(out), _stream(rhs_q4_0))
    _lib.check(rc, "block_dots_q4_0")
    return out
