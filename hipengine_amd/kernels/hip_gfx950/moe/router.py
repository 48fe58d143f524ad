"""Router selection of the MoE path: top-k experts of precomputed router logits and
the softmax over the selected logits.

Signature and checks follow hipEngine's ``kernels/hip_gfx1100/moe/router.py``
(``qwen35_router_select`` :661-683, ``_check_router_select_shape`` :1362-1377);
registry key as in :1264-1268.  Raw device pointers: float32 logits, int64 selected
experts, float32 routing weights.
"""

from __future__ import annotations

import ctypes

from hipengine_amd.core.hip import HipRuntime
from hipengine_amd.kernels.hip_gfx950._launch import I64, VOID, check_launch, entry, validate_pointers
from hipengine_amd.kernels.registry import KernelKey, register

MAX_EXPERTS = 1024


def _check_router_select_shape(tokens: int, logits_stride: int, num_experts: int, top_k: int) -> None:
    for name, value in (("tokens", tokens), ("logits_stride", logits_stride), ("num_experts", num_experts),
                        ("top_k", top_k)):
        if value <= 0:
            raise ValueError(f"{name} must be positive")
    if top_k > 16:
        raise ValueError("top_k must be <= 16")
    if top_k > num_experts:
        raise ValueError("top_k must be <= num_experts")
    if num_experts > logits_stride:
        raise ValueError("num_experts must be <= logits_stride")
    if num_experts > MAX_EXPERTS:
        raise ValueError(f"num_experts must be <= {MAX_EXPERTS}")


def qwen35_router_select(logits_ptr: int, selected_ptr: int, routing_ptr: int, tokens: int, logits_stride: int,
                         num_experts: int, top_k: int, *, threads: int = 512, stream: int = 0,
                         library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """Top-k + softmax over the selected logits for precomputed router logits."""
    _check_router_select_shape(tokens, logits_stride, num_experts, top_k)
    if threads not in (64, 128, 256, 512):
        raise ValueError("threads must be one of 64, 128, 256, 512")
    validate_pointers(logits_ptr=logits_ptr, selected_ptr=selected_ptr, routing_ptr=routing_ptr)
    fn = entry("hipengine_qwen35_router_select", [VOID, VOID, VOID, I64, I64, I64, I64, I64, VOID], library)
    check_launch(fn(logits_ptr, selected_ptr, routing_ptr, tokens, logits_stride, num_experts, top_k, threads, stream),
                 runtime)


def _make_router_logits(name: str, what: str):
    symbol = f"hipengine_{name}"

    def wrapper(hidden_ptr: int, weight_ptr: int, logits_ptr: int, tokens: int, hidden_size: int, num_rows: int, *,
                threads: int = 512, stream: int = 0, library: ctypes.CDLL | None = None,
                runtime: HipRuntime | None = None) -> None:
        for value, label in ((tokens, "tokens"), (hidden_size, "hidden_size"), (num_rows, "num_rows")):
            if value <= 0:
                raise ValueError(f"{label} must be positive")
        if threads not in (64, 128, 256, 512):
            raise ValueError("threads must be one of 64, 128, 256, 512")
        validate_pointers(hidden_ptr=hidden_ptr, weight_ptr=weight_ptr, logits_ptr=logits_ptr)
        fn = entry(symbol, [VOID, VOID, VOID, I64, I64, I64, I64, VOID], library)
        check_launch(fn(hidden_ptr, weight_ptr, logits_ptr, tokens, hidden_size, num_rows, threads, stream), runtime)

    wrapper.__name__ = name
    wrapper.__doc__ = (f"Router logits ``logits[t, e] = hidden[t] . weight[e]`` in float32 for {what} "
                       f"(hipEngine's ``moe/router.py:209-538``; C symbol ``{symbol}``).")
    return wrapper


qwen35_router_logits_bf16 = _make_router_logits("qwen35_router_logits_bf16", "bf16 hidden rows and bf16 weights")
qwen35_router_logits_fp16 = _make_router_logits("qwen35_router_logits_fp16", "fp16 hidden rows and fp16 weights")
qwen35_router_logits_bf16_f32w = _make_router_logits("qwen35_router_logits_bf16_f32w",
                                                     "bf16 hidden rows and float32 weights")
qwen35_router_logits_fp16_f32w = _make_router_logits("qwen35_router_logits_fp16_f32w",
                                                     "fp16 hidden rows and float32 weights")
qwen35_router_logits_f32_f32w = _make_router_logits("qwen35_router_logits_f32_f32w",
                                                    "float32 hidden rows and float32 weights")


def register_kernels(backend: str = "hip_gfx950", *, replace: bool = False) -> None:
    register(KernelKey(backend, "router_select", "fp32"), qwen35_router_select, replace=replace)
    # keys of hipEngine's moe/router.py:1158-1228
    register(KernelKey(backend, "router_logits", "bf16"), qwen35_router_logits_bf16, replace=replace)
    register(KernelKey(backend, "router_logits", "bf16", "bf16_hidden"), qwen35_router_logits_bf16, replace=replace)
    register(KernelKey(backend, "router_logits", "fp16"), qwen35_router_logits_fp16, replace=replace)
    register(KernelKey(backend, "router_logits", "f32", "bf16_hidden"), qwen35_router_logits_bf16_f32w, replace=replace)
    register(KernelKey(backend, "router_logits", "f32", "fp16_hidden"), qwen35_router_logits_fp16_f32w, replace=replace)
    register(KernelKey(backend, "router_logits", "f32", "f32_hidden"), qwen35_router_logits_f32_f32w, replace=replace)
