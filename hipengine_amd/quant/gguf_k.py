"""Quant plugin records of the Q8_0 / Q6_K weight formats
(hipEngine: ``hipengine/quant/gguf_k.py:10-20,101-121``)."""

from __future__ import annotations

from dataclasses import dataclass

from hipengine_amd.quant.registry import register_quant


@dataclass(frozen=True)
class GGUFQ80Quant:
    name: str = "gguf_q8_0"
    weight_storage: str = "gguf_block_q8_0"
    activation_preprocess: str = "none"
    compute_dtype: str = "fp32_accum"
    scale_granularity: str = "block32_scale"
    calibration_artifact: str = "gguf"
    kernel_family: str = "gguf_k_gemv"


@dataclass(frozen=True)
class GGUFQ6KQuant:
    name: str = "gguf_q6_k"
    weight_storage: str = "gguf_block_q6_k"
    activation_preprocess: str = "none"
    compute_dtype: str = "fp32_accum"
    scale_granularity: str = "block256_subblock16_scale"
    calibration_artifact: str = "gguf"
    kernel_family: str = "gguf_k_gemv"


GGUF_Q8_0 = register_quant(GGUFQ80Quant(), replace=True)
GGUF_Q6_K = register_quant(GGUFQ6KQuant(), replace=True)
