"""GGML tensor-type table and byte-shape helpers for the block types this path
streams (hipEngine: ``hipengine/quant/gguf.py:20-57,115-298,428-485``).

Only metadata lives here.  Dequantization happens on the device
(``hipengine_amd.kernels.hip_gfx950.quant.gguf_verify.gguf_dequantize_f32``);
there is no NumPy dequantizer in this package.
"""

from __future__ import annotations

from dataclasses import dataclass
from enum import IntEnum
from math import prod
from typing import Sequence

QK_K = 256


class GGMLQuantizationType(IntEnum):
    F32 = 0
    F16 = 1
    Q8_0 = 8
    Q8_1 = 9
    Q4_K = 12
    Q5_K = 13
    Q6_K = 14
    BF16 = 30


@dataclass(frozen=True)
class GGUFQuantLayout:
    type_id: int
    name: str
    block_size: int
    type_size: int
    storage_dtype: str
    dequant_supported: bool = False
    native_status: str = "unsupported"

    @property
    def is_block_quantized(self) -> bool:
        return self.block_size != 1 or self.storage_dtype == "uint8_blocks"


def _blocks(qtype: GGMLQuantizationType, block: int, nbytes: int, native: bool) -> GGUFQuantLayout:
    return GGUFQuantLayout(int(qtype), qtype.name, block, nbytes, "uint8_blocks", native,
                           "hip_gfx950" if native else "unsupported")


GGUF_QUANT_LAYOUTS: dict[GGMLQuantizationType, GGUFQuantLayout] = {
    GGMLQuantizationType.F32: GGUFQuantLayout(0, "F32", 1, 4, "float32", True),
    GGMLQuantizationType.F16: GGUFQuantLayout(1, "F16", 1, 2, "float16", True),
    GGMLQuantizationType.BF16: GGUFQuantLayout(30, "BF16", 1, 2, "bf16", True),
    # half d; int8 qs[32]
    GGMLQuantizationType.Q8_0: _blocks(GGMLQuantizationType.Q8_0, 32, 2 + 32, True),
    # float-pair header as GGML defines it on disk (the 36-byte half d/half s
    # activation block used by the kernels is a device-side format, not a tensor type)
    GGMLQuantizationType.Q8_1: _blocks(GGMLQuantizationType.Q8_1, 32, 4 + 4 + 32, False),
    # half d; half dmin; u8 scales[12]; u8 qs[128]
    GGMLQuantizationType.Q4_K: _blocks(GGMLQuantizationType.Q4_K, QK_K, 2 + 2 + 12 + QK_K // 2, True),
    # half d; half dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]
    GGMLQuantizationType.Q5_K: _blocks(GGMLQuantizationType.Q5_K, QK_K, 2 + 2 + 12 + QK_K // 8 + QK_K // 2, True),
    # u8 ql[128]; u8 qh[64]; i8 scales[16]; half d
    GGMLQuantizationType.Q6_K: _blocks(GGMLQuantizationType.Q6_K, QK_K, QK_K // 2 + QK_K // 4 + QK_K // 16 + 2, True),
}


def ggml_type(type_id: int | GGMLQuantizationType) -> GGMLQuantizationType:
    if isinstance(type_id, GGMLQuantizationType):
        return type_id
    try:
        return GGMLQuantizationType(int(type_id))
    except ValueError as exc:
        raise KeyError(f"unknown GGML quantization type id {int(type_id)!r}") from exc


def quant_layout(type_id: int | GGMLQuantizationType) -> GGUFQuantLayout:
    qtype = ggml_type(type_id)
    try:
        return GGUF_QUANT_LAYOUTS[qtype]
    except KeyError as exc:
        raise KeyError(f"missing GGUF layout for GGML type {qtype.name}") from exc


def nbytes_for_shape(shape: Sequence[int], type_id: int | GGMLQuantizationType) -> int:
    layout = quant_layout(type_id)
    count = int(prod(int(d) for d in shape))
    if count % layout.block_size:
        raise ValueError(
            f"shape {tuple(shape)} has {count} elements, not a multiple of {layout.name} block size {layout.block_size}"
        )
    return count // layout.block_size * layout.type_size


def quant_shape_to_byte_shape(shape: Sequence[int], type_id: int | GGMLQuantizationType) -> tuple[int, ...]:
    dims = tuple(int(d) for d in shape)
    layout = quant_layout(type_id)
    if layout.storage_dtype != "uint8_blocks":
        return dims
    if not dims:
        raise ValueError(f"block-quantized {layout.name} tensor must have at least one dimension")
    if dims[-1] % layout.block_size:
        raise ValueError(
            f"quantized tensor row size {dims[-1]} is not a multiple of {layout.name} block size {layout.block_size}"
        )
    return (*dims[:-1], dims[-1] // layout.block_size * layout.type_size)


def quant_shape_from_byte_shape(shape: Sequence[int], type_id: int | GGMLQuantizationType) -> tuple[int, ...]:
    dims = tuple(int(d) for d in shape)
    layout = quant_layout(type_id)
    if layout.storage_dtype != "uint8_blocks":
        return dims
    if not dims:
        raise ValueError(f"block-quantized {layout.name} byte tensor must have at least one dimension")
    if dims[-1] % layout.type_size:
        raise ValueError(
            f"quantized tensor bytes per row {dims[-1]} is not a multiple of {layout.name} type size {layout.type_size}"
        )
    return (*dims[:-1], dims[-1] // layout.type_size * layout.block_size)


def dequantization_supported(type_id: int | GGMLQuantizationType) -> bool:
    return quant_layout(type_id).dequant_supported
