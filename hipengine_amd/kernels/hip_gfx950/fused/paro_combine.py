"""MoE tail fused with the next layer's RMSNorm: what follows the routed down projection of a MoE FFN block.

``residual' = bf16((residual + selected) + sigmoid(gate_logits[token, 0]) * shared)`` and
``norm = bf16(residual' / sqrt(mean(residual'^2) + eps) * norm_weight)`` for bf16 rows and a float32 norm weight,
where ``selected`` is the routed sum, given or formed here in slot order and rounded to bf16.

Names, argument order and checks follow the GGUF entries of hipEngine's
``kernels/hip_gfx1100/fused/paro_combine.py`` (``shared_gate_combine_residual_rmsnorm_gguf_bf16_out`` :1205-1240,
``weighted_sum_shared_gate_combine_residual_rmsnorm_gguf_bf16_out`` :1243-1282, ``_launch_tail_rms_weighted``
:1987-2030, registry keys :1820-1838); the module keeps hipEngine's file name so that imports carry over, and holds
only these entries (its PARO and fp16 flavours belong to other quantization families).
``moe_gather_tail_rmsnorm_bf16`` is new here: the same step reading the compact rows of the grouped down projection
through ``lane_to_compact``, in place of a weighted gather followed by the tail.
"""

from __future__ import annotations

import ctypes

from hipengine_amd.core.hip import HipRuntime
from hipengine_amd.kernels.hip_gfx950._launch import I64, VOID, check_launch, entry, validate_pointers
from hipengine_amd.kernels.registry import KernelKey, register

F32 = ctypes.c_float


def _check_positive(value: int, name: str) -> None:
    if value <= 0:
        raise ValueError(f"{name} must be positive")


def shared_gate_combine_residual_rmsnorm_gguf_bf16_out(selected_ptr: int, shared_ptr: int, gate_logits_ptr: int,
                                                       residual_ptr: int, norm_weight_ptr: int, norm_out_ptr: int,
                                                       residual_out_ptr: int, tokens: int, features: int,
                                                       gate_stride: int, eps: float = 1e-6, *, stream: int = 0,
                                                       library: ctypes.CDLL | None = None,
                                                       runtime: HipRuntime | None = None) -> None:
    """The tail over an already formed, bf16-rounded routed sum ``[tokens, features]``."""
    for value, name in ((tokens, "tokens"), (features, "features"), (gate_stride, "gate_stride")):
        _check_positive(value, name)
    validate_pointers(selected_ptr=selected_ptr, shared_ptr=shared_ptr, gate_logits_ptr=gate_logits_ptr,
                      residual_ptr=residual_ptr, norm_weight_ptr=norm_weight_ptr, norm_out_ptr=norm_out_ptr,
                      residual_out_ptr=residual_out_ptr)
    fn = entry("hipengine_shared_gate_combine_residual_rmsnorm_gguf_bf16_out", [VOID] * 7 + [I64] * 3 + [F32, VOID],
               library)
    check_launch(fn(selected_ptr, shared_ptr, gate_logits_ptr, residual_ptr, norm_weight_ptr, norm_out_ptr,
                    residual_out_ptr, tokens, features, gate_stride, float(eps), stream), runtime)


def weighted_sum_shared_gate_combine_residual_rmsnorm_gguf_bf16_out(values_ptr: int, weights_ptr: int, shared_ptr: int,
                                                                    gate_logits_ptr: int, residual_ptr: int,
                                                                    norm_weight_ptr: int, norm_out_ptr: int,
                                                                    residual_out_ptr: int, tokens: int,
                                                                    rows_per_token: int, features: int,
                                                                    gate_stride: int, eps: float = 1e-6, *,
                                                                    stream: int = 0,
                                                                    library: ctypes.CDLL | None = None,
                                                                    runtime: HipRuntime | None = None) -> None:
    """The tail over slot rows ``[tokens * rows_per_token, features]`` and their float32 routing weights."""
    for value, name in ((tokens, "tokens"), (rows_per_token, "rows_per_token"), (features, "features"),
                        (gate_stride, "gate_stride")):
        _check_positive(value, name)
    validate_pointers(values_ptr=values_ptr, weights_ptr=weights_ptr, shared_ptr=shared_ptr,
                      gate_logits_ptr=gate_logits_ptr, residual_ptr=residual_ptr, norm_weight_ptr=norm_weight_ptr,
                      norm_out_ptr=norm_out_ptr, residual_out_ptr=residual_out_ptr)
    fn = entry("hipengine_weighted_sum_shared_gate_combine_residual_rmsnorm_gguf_bf16_out",
               [VOID] * 8 + [I64] * 4 + [F32, VOID], library)
    check_launch(fn(values_ptr, weights_ptr, shared_ptr, gate_logits_ptr, residual_ptr, norm_weight_ptr, norm_out_ptr,
                    residual_out_ptr, tokens, rows_per_token, features, gate_stride, float(eps), stream), runtime)


def moe_gather_tail_rmsnorm_bf16(down_ptr: int, lane_to_compact_ptr: int, weights_ptr: int, shared_ptr: int,
                                 gate_logits_ptr: int, residual_ptr: int, norm_weight_ptr: int, norm_out_ptr: int,
                                 residual_out_ptr: int, tokens: int, top_k: int, features: int, compact_rows: int,
                                 gate_stride: int, eps: float = 1e-6, *, stream: int = 0,
                                 library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """The tail over compact rows ``[compact_rows, features]`` of the grouped down projection: slot ``s`` of token
    ``t`` reads row ``lane_to_compact[t * top_k + s]`` (a negative entry contributes nothing)."""
    for value, name in ((tokens, "tokens"), (top_k, "top_k"), (features, "features"), (compact_rows, "compact_rows"),
                        (gate_stride, "gate_stride")):
        _check_positive(value, name)
    validate_pointers(down_ptr=down_ptr, lane_to_compact_ptr=lane_to_compact_ptr, weights_ptr=weights_ptr,
                      shared_ptr=shared_ptr, gate_logits_ptr=gate_logits_ptr, residual_ptr=residual_ptr,
                      norm_weight_ptr=norm_weight_ptr, norm_out_ptr=norm_out_ptr, residual_out_ptr=residual_out_ptr)
    fn = entry("hipengine_gfx950_moe_gather_tail_rmsnorm_bf16", [VOID] * 9 + [I64] * 5 + [F32, VOID], library)
    check_launch(fn(down_ptr, lane_to_compact_ptr, weights_ptr, shared_ptr, gate_logits_ptr, residual_ptr,
                    norm_weight_ptr, norm_out_ptr, residual_out_ptr, tokens, top_k, features, compact_rows, gate_stride,
                    float(eps), stream), runtime)


def register_kernels(backend: str = "hip_gfx950", *, replace: bool = False) -> None:
    register(KernelKey(backend, "shared_gate_combine+residual+rmsnorm", "gguf_f32_weight", "bf16_out"),
             shared_gate_combine_residual_rmsnorm_gguf_bf16_out, replace=replace)
    register(KernelKey(backend, "weighted_sum+shared_gate+residual+rmsnorm", "gguf_f32_weight", "bf16_out"),
             weighted_sum_shared_gate_combine_residual_rmsnorm_gguf_bf16_out, replace=replace)
    register(KernelKey(backend, "weighted_sum+shared_gate+residual+rmsnorm", "gguf_f32_weight",
                       "gather_compact_bf16_out"), moe_gather_tail_rmsnorm_bf16, replace=replace)
