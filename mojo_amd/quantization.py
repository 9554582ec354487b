"""``QuantizationEncoding`` / ``QuantizationConfig``: the metadata half of the qmatmul API.

MAX's Python package is not part of the reference snapshot (binary dependency,
``magic.lock:135-137``); names and fields follow its public documentation.
"""
from __future__ import annotations

import enum
from dataclasses import dataclass


@dataclass(frozen=True)
class BlockParameters:
    """Elements and bytes of one packed block of a GGUF encoding."""

    elements_per_block: int
    block_size: int


class QuantizationEncoding(enum.Enum):
    Q4_0 = "Q4_0"
    Q4_K = "Q4_K"
    Q5_K = "Q5_K"
    Q6_K = "Q6_K"
    GPTQ = "GPTQ"
    # activation-side block format of the Q4_0 path; not a weight encoding of qmatmul
    Q8_0 = "Q8_0"
    # activation-side block format of the optional integer Q4_K path (``qmatmul(..., act_q8k=True)``)
    Q8_K = "Q8_K"

    @property
    def code(self) -> int:
        """Value of ``enum qmm_encoding`` in ``include/qmm.h``."""
        return _CODES[self]

    @property
    def is_gguf(self) -> bool:
        return self in (QuantizationEncoding.Q4_0, QuantizationEncoding.Q4_K, QuantizationEncoding.Q5_K,
                        QuantizationEncoding.Q6_K)

    @property
    def block_parameters(self) -> BlockParameters:
        if self not in _BLOCKS:
            raise ValueError(f"{self.name} has no fixed block layout")
        return _BLOCKS[self]

    def packed_row_bytes(self, k: int) -> int:
        bp = self.block_parameters
        if k % bp.elements_per_block:
            raise ValueError(f"K={k} is not a multiple of the {self.name} block size {bp.elements_per_block}")
        return k // bp.elements_per_block * bp.block_size


_CODES = {
    QuantizationEncoding.Q4_0: 0,
    QuantizationEncoding.Q4_K: 1,
    QuantizationEncoding.Q6_K: 2,
    QuantizationEncoding.GPTQ: 3,
    QuantizationEncoding.Q5_K: 4,
    QuantizationEncoding.Q8_0: 8,
    QuantizationEncoding.Q8_K: 9,
}
_BLOCKS = {
    QuantizationEncoding.Q4_0: BlockParameters(32, 18),
    QuantizationEncoding.Q8_0: BlockParameters(32, 34),
    QuantizationEncoding.Q8_K: BlockParameters(256, 292),
    QuantizationEncoding.Q4_K: BlockParameters(256, 144),
    QuantizationEncoding.Q6_K: BlockParameters(256, 210),
    QuantizationEncoding.Q5_K: BlockParameters(256, 176),
}


@dataclass(frozen=True)
class QuantizationConfig:
    """GPTQ checkpoint parameters (``quantize_config.json`` of AutoGPTQ)."""

    quant_method: str = "gptq"
    bits: int = 4
    group_size: int = 128
    desc_act: bool = False
    sym: bool = True
