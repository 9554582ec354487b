"""MI355X-native quantized-weight matmul behind the ``max.graph.ops.qmatmul`` call shape.

``qmatmul(encoding, config, lhs, *rhs)``, ``dequantize`` and the
``QuantizationEncoding`` / ``QuantizationConfig`` types mirror the MAX graph API;
the arithmetic runs in hand-written HIP kernels for gfx950 reached through the
C ABI of ``libqmm.so`` (``include/qmm.h``).  There is no CPU fallback: a missing
library or a non-GPU tensor is an error.
"""
from .quantization import BlockParameters, QuantizationConfig, QuantizationEncoding
from .ops import (
    block_dots_q4_0,
    dequantize,
    qmatmul,
    qmatmul_grouped,
    qmatmul_repacked,
    qmatmul_rmsnorm,
    qmatmul_swiglu,
    quantize,
    quantize_gptq,
    repack_weights,
    RepackedWeights,
)
from .weights import GGUFWeights, load_gptq_config, load_gptq_linear

__all__ = [
    "BlockParameters",
    "QuantizationConfig",
    "QuantizationEncoding",
    "qmatmul",
    "qmatmul_grouped",
    "qmatmul_repacked",
    "repack_weights",
    "RepackedWeights",
    "qmatmul_rmsnorm",
    "qmatmul_swiglu",
    "dequantize",
    "quantize",
    "quantize_gptq",
    "block_dots_q4_0",
    "GGUFWeights",
    "load_gptq_config",
    "load_gptq_linear",
]
