"""Quant plugin records and GGUF block metadata for the k-quant matmul path."""

from hipengine_amd.quant.base import QuantPlugin
from hipengine_amd.quant.gguf import (
    GGUF_QUANT_LAYOUTS,
    QK_K,
    GGMLQuantizationType,
    GGUFQuantLayout,
    dequantization_supported,
    ggml_type,
    nbytes_for_shape,
    quant_layout,
    quant_shape_from_byte_shape,
    quant_shape_to_byte_shape,
)
from hipengine_amd.quant.gguf_k import GGUF_Q6_K, GGUF_Q8_0, GGUFQ6KQuant, GGUFQ80Quant
from hipengine_amd.quant.gguf_q4_k import (
    GGUF_Q4_K,
    GGUF_Q4_K_BLOCK,
    GGUF_Q4_K_BLOCK_BYTES,
    GGUF_Q4_K_SUBBLOCK,
    GGUF_Q4_K_SUBBLOCKS,
    GGUF_Q8_1_BLOCK,
    GGUF_Q8_1_BLOCK_BYTES,
    GGUF_Q8_1_D4S4_BYTES,
    GGUF_Q8_1_MMQ_BLOCK,
    GGUF_Q8_1_MMQ_DS4_BYTES,
    GGUFQ4KQuant,
)
from hipengine_amd.quant.registry import (
    DuplicateQuantError,
    MissingQuantError,
    register_quant,
    registered_quants,
    resolve_quant,
)

GGUF_Q6_K_BLOCK_BYTES = 210
GGUF_Q8_0_BLOCK_BYTES = 34
GGUF_Q5_K_BLOCK_BYTES = 176

__all__ = [name for name in dir() if not name.startswith("_")]
