"""Readers for the two containers whose tensors feed ``qmatmul``: GGUF files and AutoGPTQ safetensors.

Pure host code.  A GGUF tensor of a block encoding is handed out exactly as it lies in the file,
viewed as ``uint8[N, K / elements_per_block * block_size]``: the layout ``qmatmul`` takes as ``rhs``.
Nothing is repacked.  The GGUF layout follows the published container specification (ggml
``docs/gguf.md``, versions 2 and 3, little-endian): header, key/value metadata, tensor-info table,
padding to ``general.alignment`` (default 32), tensor data.  AutoGPTQ checkpoints are safetensors
files with ``<prefix>.qweight / .scales / .qzeros / .g_idx`` and a ``quantize_config.json``.
"""
from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass
from typing import Any, Dict, Iterator, Optional, Tuple

import numpy as np

from .quantization import QuantizationConfig, QuantizationEncoding

GGUF_MAGIC = 0x46554747  # "GGUF"
GGUF_DEFAULT_ALIGNMENT = 32

# ggml tensor type code -> (name, elements per block, bytes per block)
GGML_TYPES: Dict[int, Tuple[str, int, int]] = {
    0: ("F32", 1, 4),
    1: ("F16", 1, 2),
    2: ("Q4_0", 32, 18),
    3: ("Q4_1", 32, 20),
    6: ("Q5_0", 32, 22),
    7: ("Q5_1", 32, 24),
    8: ("Q8_0", 32, 34),
    9: ("Q8_1", 32, 36),
    10: ("Q2_K", 256, 84),
    11: ("Q3_K", 256, 110),
    12: ("Q4_K", 256, 144),
    13: ("Q5_K", 256, 176),
    14: ("Q6_K", 256, 210),
    15: ("Q8_K", 256, 292),
    24: ("I8", 1, 1),
    25: ("I16", 1, 2),
    26: ("I32", 1, 4),
    27: ("I64", 1, 8),
    28: ("F64", 1, 8),
    30: ("BF16", 1, 2),
}
_ENCODINGS = {"Q4_0": QuantizationEncoding.Q4_0, "Q4_K": QuantizationEncoding.Q4_K, "Q5_K": QuantizationEncoding.Q5_K,
              "Q6_K": QuantizationEncoding.Q6_K}
_PLAIN_DTYPES = {"F32": np.float32, "F16": np.float16, "I8": np.int8, "I16": np.int16, "I32": np.int32,
                 "I64": np.int64, "F64": np.float64, "BF16": np.uint16}

# metadata value type code -> struct format
_SCALARS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}
_T_STRING, _T_ARRAY = 8, 9


@dataclass(frozen=True)
class GGUFTensorInfo:
    name: str
    shape: Tuple[int, ...]            # outermost dimension first: (N, K) for a weight matrix
    ggml_type: str                    # "Q4_K", "F32", ...
    encoding: Optional[QuantizationEncoding]  # set for the block encodings qmatmul takes
    offset: int                       # absolute byte offset in the file
    nbytes: int


class _Cursor:
    def __init__(self, buf, pos: int = 0):
        self.buf, self.pos = buf, pos

    def take(self, fmt: str):
        size = struct.calcsize(fmt)
        if self.pos + size > len(self.buf):
            raise ValueError("GGUF file is truncated")
        (v,) = struct.unpack_from(fmt, self.buf, self.pos)
        self.pos += size
        return v

    def string(self) -> str:
        n = self.take("<Q")
        if self.pos + n > len(self.buf):
            raise ValueError("GGUF file is truncated")
        s = bytes(self.buf[self.pos:self.pos + n]).decode("utf-8")
        self.pos += n
        return s

    def value(self, vtype: int) -> Any:
        if vtype in _SCALARS:
            return self.take(_SCALARS[vtype])
        if vtype == _T_STRING:
            return self.string()
        if vtype == _T_ARRAY:
            etype, count = self.take("<I"), self.take("<Q")
            if etype in _SCALARS and etype != 7:
                fmt = _SCALARS[etype]
                size = struct.calcsize(fmt)
                if self.pos + size * count > len(self.buf):
                    raise ValueError("GGUF file is truncated")
                arr = np.frombuffer(self.buf, dtype=np.dtype(fmt), count=count, offset=self.pos).copy()
                self.pos += size * count
                return arr
            return [self.value(etype) for _ in range(count)]
        raise ValueError(f"unknown GGUF metadata value type {vtype}")


class GGUFWeights:
    """Memory-mapped view of a GGUF file: ``metadata`` (dict) and ``tensors`` (name -> GGUFTensorInfo)."""

    def __init__(self, path: str):
        self.path = os.fspath(path)
        self._map = np.memmap(self.path, dtype=np.uint8, mode="r")
        cur = _Cursor(self._map)
        if len(self._map) < 24 or cur.take("<I") != GGUF_MAGIC:
            raise ValueError(f"{self.path}: not a GGUF file (bad magic)")
        self.version = cur.take("<I")
        if self.version not in (2, 3):
            raise ValueError(f"{self.path}: GGUF version {self.version} is not supported (2 and 3 are)")
        n_tensors, n_kv = cur.take("<Q"), cur.take("<Q")
        self.metadata: Dict[str, Any] = {}
        for _ in range(n_kv):
            key = cur.string()
            self.metadata[key] = cur.value(cur.take("<I"))
        self.alignment = int(self.metadata.get("general.alignment", GGUF_DEFAULT_ALIGNMENT))
        if self.alignment <= 0 or self.alignment & (self.alignment - 1):
            raise ValueError(f"{self.path}: general.alignment {self.alignment} is not a power of two")
        raw = []
        for _ in range(n_tensors):
            name = cur.string()
            n_dims = cur.take("<I")
            if n_dims > 4:
                raise ValueError(f"{self.path}: tensor {name!r} has {n_dims} dimensions")
            dims = [cur.take("<Q") for _ in range(n_dims)]  # innermost first
            raw.append((name, dims, cur.take("<I"), cur.take("<Q")))
        self.data_offset = (cur.pos + self.alignment - 1) // self.alignment * self.alignment
        self.tensors: Dict[str, GGUFTensorInfo] = {}
        for name, dims, tcode, rel in raw:
            if tcode not in GGML_TYPES:
                raise ValueError(f"{self.path}: tensor {name!r} has unknown ggml type {tcode}")
            tname, epb, bpb = GGML_TYPES[tcode]
            if rel % self.alignment:
                raise ValueError(f"{self.path}: tensor {name!r} offset {rel} is not aligned to {self.alignment}")
            k = dims[0] if dims else 1
            if k % epb:
                raise ValueError(f"{self.path}: tensor {name!r} row length {k} is not a multiple of the {tname} block")
            count = int(np.prod(dims, dtype=np.int64)) if dims else 1
            nbytes = count // epb * bpb
            off = self.data_offset + rel
            if off + nbytes > len(self._map):
                raise ValueError(f"{self.path}: tensor {name!r} runs past the end of the file")
            self.tensors[name] = GGUFTensorInfo(name, tuple(reversed(dims)), tname, _ENCODINGS.get(tname), off, nbytes)

    def __contains__(self, name: str) -> bool:
        return name in self.tensors

    def __iter__(self) -> Iterator[str]:
        return iter(self.tensors)

    def encoding(self, name: str) -> Optional[QuantizationEncoding]:
        return self.tensors[name].encoding

    def raw(self, name: str) -> np.ndarray:
        """The tensor's bytes in the file (a view of the mapping, no copy).

        Block encodings: ``uint8[..., N, K / epb * bpb]``.  Plain types: the typed array in its own shape
        (BF16 as ``uint16`` bit patterns).
        """
        t = self.tensors[name]
        flat = self._map[t.offset:t.offset + t.nbytes]
        _, epb, bpb = next(v for v in GGML_TYPES.values() if v[0] == t.ggml_type)
        if t.ggml_type in _PLAIN_DTYPES:
            return flat.view(_PLAIN_DTYPES[t.ggml_type]).reshape(t.shape)
        row_bytes = (t.shape[-1] if t.shape else 1) // epb * bpb
        return flat.reshape(t.shape[:-1] + (row_bytes,))

    def tensor(self, name: str, device="cuda:0"):
        """The tensor on ``device`` as torch memory, ready to be the ``rhs`` of ``qmatmul``."""
        import torch

        return torch.from_numpy(np.array(self.raw(name))).to(device)  # one host copy out of the read-only mapping


def load_gptq_config(path: str) -> QuantizationConfig:
    """``quantize_config.json`` of an AutoGPTQ checkpoint (a file, or the directory that holds it)."""
    if os.path.isdir(path):
        path = os.path.join(path, "quantize_config.json")
    with open(path, "r", encoding="utf-8") as f:
        d = json.load(f)
    return QuantizationConfig(quant_method=d.get("quant_method", "gptq"), bits=int(d.get("bits", 4)),
                              group_size=int(d.get("group_size", 128)), desc_act=bool(d.get("desc_act", False)),
                              sym=bool(d.get("sym", True)))


def load_gptq_linear(path: str, prefix: str, device="cuda:0"):
    """``(qweight, scales, qzeros, g_idx)`` of the linear layer ``prefix`` from an AutoGPTQ safetensors file.

    Shapes are checked against the v1 layout ``qmatmul`` takes: ``qweight int32[K/8, N]``,
    ``scales f16[K/g, N]``, ``qzeros int32[K/g, N/8]``, ``g_idx int32[K]`` (absent in some checkpoints:
    then ``k // group`` is implied and an explicit one is made).
    """
    import torch
    from safetensors import safe_open

    with safe_open(path, framework="pt", device="cpu") as f:
        keys = set(f.keys())
        missing = [s for s in ("qweight", "scales", "qzeros") if f"{prefix}.{s}" not in keys]
        if missing:
            raise KeyError(f"{path}: {prefix} lacks {', '.join(missing)}")
        qweight, scales, qzeros = (f.get_tensor(f"{prefix}.{s}") for s in ("qweight", "scales", "qzeros"))
        g_idx = f.get_tensor(f"{prefix}.g_idx") if f"{prefix}.g_idx" in keys else None
    if qweight.dtype != torch.int32 or qzeros.dtype != torch.int32 or scales.dtype != torch.float16:
        raise ValueError(f"{prefix}: expected int32 qweight / qzeros and float16 scales")
    k8, n = qweight.shape
    groups = scales.shape[0]
    if scales.shape != (groups, n) or qzeros.shape != (groups, n // 8) or (k8 * 8) % groups:
        raise ValueError(f"{prefix}: shapes {tuple(qweight.shape)}, {tuple(scales.shape)}, {tuple(qzeros.shape)} "
                         "are not the AutoGPTQ v1 4-bit layout")
    k = k8 * 8
    if g_idx is None:
        g_idx = (torch.arange(k, dtype=torch.int32) // (k // groups)).to(torch.int32)
    elif g_idx.shape != (k,):
        raise ValueError(f"{prefix}: g_idx has shape {tuple(g_idx.shape)}, expected ({k},)")
    return tuple(t.to(device) for t in (qweight, scales, qzeros, g_idx.to(torch.int32)))
