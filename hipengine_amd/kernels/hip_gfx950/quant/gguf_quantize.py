"""q8_1 activation quantizers: 36-byte GEMV blocks, 144-byte DS4 blocks and
160-byte D4S4 blocks.

Wrapper signatures follow hipEngine's ``gguf_q4_k_quantize_{bf16,f32}_q8_1``
(``kernels/hip_gfx1100/quant/gguf_q4_k_gemv.py:1158-1268``),
``gguf_q8_1_mmq_ds4_pack_bf16`` (``gguf_q4_k_q8_1_selected_prefill.py``) and
``gguf_q8_1_d4s4_f32_quantize_bf16`` (``gguf_k_mmq_prefill.py:244-276``).
"""

from __future__ import annotations

import ctypes

from hipengine_amd.core.hip import HipRuntime
from hipengine_amd.kernels.hip_gfx950._launch import I64, VOID, check_launch, entry, validate_pointers
from hipengine_amd.kernels.registry import KernelKey, register

_ARGS = [VOID, VOID, I64, I64, VOID]


def _quantize(symbol: str, x_ptr: int, xq_ptr: int, rows: int, in_features: int, block: int, stream: int,
              library: ctypes.CDLL | None, runtime: HipRuntime | None) -> None:
    if rows <= 0:
        raise ValueError("rows must be positive")
    if in_features <= 0 or in_features % block != 0:
        raise ValueError(f"in_features must be positive and divisible by {block}")
    validate_pointers(x_ptr=x_ptr, xq_ptr=xq_ptr)
    check_launch(entry(symbol, _ARGS, library)(x_ptr, xq_ptr, rows, in_features, stream), runtime)


def gguf_q4_k_quantize_f32_q8_1(x_ptr: int, xq_ptr: int, rows: int, in_features: int, *, stream: int = 0,
                                library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """float32 ``[rows, in_features]`` -> ``[rows, in_features/32]`` 36-byte q8_1 blocks."""
    _quantize("hipengine_gguf_q4_k_quantize_f32_q8_1", x_ptr, xq_ptr, rows, in_features, 32, stream, library, runtime)


def gguf_q4_k_quantize_bf16_q8_1(x_ptr: int, xq_ptr: int, rows: int, in_features: int, *, stream: int = 0,
                                 library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """bf16 ``[rows, in_features]`` -> ``[rows, in_features/32]`` 36-byte q8_1 blocks."""
    _quantize("hipengine_gguf_q4_k_quantize_bf16_q8_1", x_ptr, xq_ptr, rows, in_features, 32, stream, library, runtime)


def gguf_q4_k_quantize_bf16_q8_1x2(x_ptr: int, xq_ptr: int, rows: int, in_features: int, *, stream: int = 0,
                                   library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """bf16 ``[rows, in_features]`` -> two planes ``[2, rows, in_features/32]`` of 36-byte q8_1 blocks: the plain
    quantization and the same quantization of its residual (``gguf_q4_k_gemv.py:1195-1233``).  The planes are
    consecutive, so a pre-quantized GEMV over ``2 * rows`` rows yields the two partial products to add."""
    _quantize("hipengine_gguf_q4_k_quantize_bf16_q8_1x2", x_ptr, xq_ptr, rows, in_features, 32, stream, library, runtime)


def gguf_q8_1_mmq_ds4_pack_bf16(x_ptr: int, xq_ptr: int, rows: int, hidden: int, *, stream: int = 0,
                                library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """bf16 ``[rows, hidden]`` -> ``[rows, hidden/128]`` 144-byte DS4 blocks."""
    _quantize("hipengine_gguf_q8_1_mmq_ds4_pack_bf16", x_ptr, xq_ptr, rows, hidden, 128, stream, library, runtime)


def gguf_q8_1_mmq_gather_ds4_pack_bf16(hidden_bf16_ptr: int, sorted_lanes_ptr: int, out_q8_ptr: int, rows: int,
                                       hidden: int, tokens: int, top_k: int, *, stream: int = 0,
                                       library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """Gather + DS4 pack in one pass (hipEngine ``gguf_q4_k_q8_1_selected_prefill.py:432-490``): output row ``r`` is
    the pack of token ``sorted_lanes[r] // top_k`` of the bf16 ``[tokens, hidden]`` input, a row of zeros for a
    negative lane or a token outside the input.  ``rows`` counts packed lanes."""
    for name, value in (("rows", rows), ("hidden", hidden), ("tokens", tokens), ("top_k", top_k)):
        if value <= 0:
            raise ValueError(f"{name} must be positive")
    if hidden % 128 != 0:
        raise ValueError("hidden must be divisible by DS4 Q8_1 MMQ block size 128")
    validate_pointers(hidden_bf16_ptr=hidden_bf16_ptr, sorted_lanes_ptr=sorted_lanes_ptr, out_q8_ptr=out_q8_ptr)
    fn = entry("hipengine_gguf_q8_1_mmq_gather_ds4_pack_bf16", [VOID, VOID, VOID, I64, I64, I64, I64, VOID], library)
    check_launch(fn(hidden_bf16_ptr, sorted_lanes_ptr, out_q8_ptr, rows, hidden, tokens, top_k, stream), runtime)


def gguf_q8_1_d4s4_f32_quantize_bf16(x_ptr: int, xq_ptr: int, rows: int, hidden: int, *, stream: int = 0,
                                     library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """bf16 ``[rows, hidden]`` -> ``[rows, hidden/128]`` 160-byte D4S4 blocks."""
    _quantize("hipengine_gguf_q8_1_d4s4_f32_quantize_bf16", x_ptr, xq_ptr, rows, hidden, 128, stream, library, runtime)


def q8_1_workspace_nbytes(rows: int, in_features: int) -> int:
    return rows * (in_features // 32) * 36


def ds4_workspace_nbytes(rows: int, hidden: int) -> int:
    return rows * (hidden // 128) * 144


def d4s4_workspace_nbytes(rows: int, hidden: int) -> int:
    return rows * (hidden // 128) * 160


def register_kernels(backend: str = "hip_gfx950", *, replace: bool = False) -> None:
    # activation-quant keys in the style of gguf_k_mmq_prefill.py:726-752
    for quant, variant, fn in (
        ("q8_1", "f32", gguf_q4_k_quantize_f32_q8_1),
        ("q8_1", "bf16", gguf_q4_k_quantize_bf16_q8_1),
        ("q8_1x2", "bf16", gguf_q4_k_quantize_bf16_q8_1x2),
        ("q8_1_ds4", "bf16", gguf_q8_1_mmq_ds4_pack_bf16),
        ("q8_1_ds4", "gather_bf16", gguf_q8_1_mmq_gather_ds4_pack_bf16),
        ("q8_1_d4s4_f32", "bf16", gguf_q8_1_d4s4_f32_quantize_bf16),
    ):
        register(KernelKey(backend, "activation_quant", quant, variant), fn, replace=replace)
