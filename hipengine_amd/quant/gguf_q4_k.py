"""Quant plugin record and block constants of the Q4_K weight format
(hipEngine: ``hipengine/quant/gguf_q4_k.py:14-20,105-120``)."""

from __future__ import annotations

from dataclasses import dataclass

from hipengine_amd.quant.registry import register_quant

GGUF_Q4_K_BLOCK = 256
GGUF_Q4_K_BLOCK_BYTES = 144
GGUF_Q4_K_SUBBLOCK = 32
GGUF_Q4_K_SUBBLOCKS = 8
GGUF_Q8_1_BLOCK = 32
GGUF_Q8_1_BLOCK_BYTES = 36
GGUF_Q8_1_MMQ_BLOCK = 128
GGUF_Q8_1_MMQ_DS4_BYTES = 144
GGUF_Q8_1_D4S4_BYTES = 160


@dataclass(frozen=True)
class GGUFQ4KQuant:
    name: str = "gguf_q4_k"
    weight_storage: str = "gguf_block_q4_k"
    activation_preprocess: str = "none"
    compute_dtype: str = "fp32_accum"
    scale_granularity: str = "block256_subblock32_scale_min"
    calibration_artifact: str = "gguf"
    kernel_family: str = "gguf_q4_k_gemv"


GGUF_Q4_K = register_quant(GGUFQ4KQuant(), replace=True)
