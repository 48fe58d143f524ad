"""MMQ prefill GEMM wrappers (int8 MFMA): raw Q4_K x DS4 q8_1 and raw Q6_K x D4S4 q8_1.

Signature ``fn(xq_ptr, qweight_ptr, out_ptr, rows, hidden, out_features, *, stream,
library, runtime)`` as in hipEngine's ``gguf_q4_k_q8_1_mmq_prefill.py`` /
``gguf_k_mmq_prefill.py:349-397``; registry variants as in
``tests/test_gpu_gguf_q4_k_q8_1_mmq_prefill.py:362-382`` and ``gguf_k_mmq_prefill.py:793-802``.
"""

from __future__ import annotations

import ctypes

from hipengine_amd.core.hip import HipRuntime
from hipengine_amd.kernels.hip_gfx950._launch import I64, VOID, check_launch, entry, validate_pointers
from hipengine_amd.kernels.registry import KernelKey, register

_ARGS = [VOID, VOID, VOID, I64, I64, I64, VOID]


def _validate(rows: int, hidden: int, out_features: int, out_multiple: int, hidden_multiple: int = 256) -> None:
    if rows <= 0 or rows > (1 << 20):
        raise ValueError("rows must be in 1..2^20")
    if hidden <= 0 or hidden % hidden_multiple != 0:
        raise ValueError("hidden must be positive and divisible by " +
                         ("the GGUF block size 256" if hidden_multiple == 256 else f"{hidden_multiple}"))
    if out_features <= 0 or out_features % out_multiple != 0:
        raise ValueError(f"out_features must be positive and divisible by {out_multiple}")


def _make(name: str, symbol: str, out_multiple: int, hidden_multiple: int = 256):
    def wrapper(xq_ptr: int, qweight_ptr: int, out_ptr: int, rows: int, hidden: int, out_features: int, *,
                stream: int = 0, library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
        _validate(rows, hidden, out_features, out_multiple, hidden_multiple)
        validate_pointers(xq_ptr=xq_ptr, qweight_ptr=qweight_ptr, out_ptr=out_ptr)
        check_launch(entry(symbol, _ARGS, library)(xq_ptr, qweight_ptr, out_ptr, rows, hidden, out_features, stream),
                     runtime)

    wrapper.__name__ = name
    wrapper.__doc__ = f"MMQ prefill GEMM over pre-quantized q8_1 activations (C symbol ``{symbol}``)."
    return wrapper


gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_f32_out = _make(
    "gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_f32_out", "hipengine_gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_f32_out", 32)
gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_bf16_out = _make(
    "gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_bf16_out", "hipengine_gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_bf16_out", 32)
gguf_q4_k_q8_1_mmq32_ctl_dense_bf16_f32_out = _make(
    "gguf_q4_k_q8_1_mmq32_ctl_dense_bf16_f32_out", "hipengine_gguf_q4_k_q8_1_mmq32_ctl_dense_bf16_f32_out", 32)
gguf_q4_k_q8_1_mmq32_ctl_dense_bf16_bf16_out = _make(
    "gguf_q4_k_q8_1_mmq32_ctl_dense_bf16_bf16_out", "hipengine_gguf_q4_k_q8_1_mmq32_ctl_dense_bf16_bf16_out", 32)

gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_f32_out = _make(
    "gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_f32_out", "hipengine_gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_f32_out", 32)
gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out = _make(
    "gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out", "hipengine_gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out", 32)
gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_f32_out = _make(
    "gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_f32_out", "hipengine_gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_f32_out", 1)
gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out = _make(
    "gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out", "hipengine_gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out", 1)

# hipEngine's scheduling variants of the Q5_K GEMM (gguf_k_mmq_prefill.py:459-640): the one kernel form here
gguf_q5_k_mmq32_pipe_q8_1_d4s4_f32_bf16_bf16_out = _make(
    "gguf_q5_k_mmq32_pipe_q8_1_d4s4_f32_bf16_bf16_out", "hipengine_gguf_q5_k_mmq32_pipe_q8_1_d4s4_f32_bf16_bf16_out", 32)
gguf_q5_k_mmq32_mb4_q8_1_d4s4_f32_bf16_bf16_out = _make(
    "gguf_q5_k_mmq32_mb4_q8_1_d4s4_f32_bf16_bf16_out", "hipengine_gguf_q5_k_mmq32_mb4_q8_1_d4s4_f32_bf16_bf16_out", 32)
gguf_q5_k_mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_bf16_out = _make(
    "gguf_q5_k_mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_bf16_out",
    "hipengine_gguf_q5_k_mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_bf16_out", 32)
gguf_q5_k_mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_f32_out = _make(
    "gguf_q5_k_mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_f32_out",
    "hipengine_gguf_q5_k_mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_f32_out", 32)

# Q8_0 x D4S4 (new here: hipEngine has no MMQ for Q8_0): 128 values per D4S4 block
gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_f32_out = _make(
    "gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_f32_out", "hipengine_gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_f32_out", 1, 128)
gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_bf16_out = _make(
    "gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_bf16_out", "hipengine_gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_bf16_out", 1, 128)


def gguf_q4_k_q8_1_mmq_tuned(xq_ptr: int, qweight_ptr: int, out_ptr: int, rows: int, hidden: int, out_features: int, *,
                             out_kind: int = 0, variant: int = 0, stream: int = 0,
                             library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """Q4_K x DS4 MMQ with an explicit kernel form (``hipengine_gfx950_gguf_q4_k_mmq_tuned``)."""
    _validate(rows, hidden, out_features, 32)
    validate_pointers(xq_ptr=xq_ptr, qweight_ptr=qweight_ptr, out_ptr=out_ptr)
    fn = entry("hipengine_gfx950_gguf_q4_k_mmq_tuned", [VOID, VOID, VOID, ctypes.c_int, I64, I64, I64, ctypes.c_int, VOID],
               library)
    check_launch(fn(xq_ptr, qweight_ptr, out_ptr, out_kind, rows, hidden, out_features, variant, stream), runtime)


_Q4 = (
    ("mmq32_vdr_dense_bf16_f32_out", gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_f32_out),
    ("mmq32_vdr_dense_bf16_bf16_out", gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_bf16_out),
    ("mmq32_ctl_dense_bf16_f32_out", gguf_q4_k_q8_1_mmq32_ctl_dense_bf16_f32_out),
    ("mmq32_ctl_dense_bf16_bf16_out", gguf_q4_k_q8_1_mmq32_ctl_dense_bf16_bf16_out),
)


def register_kernels(backend: str = "hip_gfx950", *, replace: bool = False) -> None:
    for variant, fn in _Q4:
        register(KernelKey(backend, "linear", "gguf_q4_k", variant), fn, replace=replace)
    register(KernelKey(backend, "linear", "gguf_q5_k", "mmq32_q8_1_d4s4_f32_bf16_f32_out"),
             gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, replace=replace)
    register(KernelKey(backend, "linear", "gguf_q5_k", "mmq32_q8_1_d4s4_f32_bf16_bf16_out"),
             gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out, replace=replace)
    for variant, fn in (("mmq32_pipe_q8_1_d4s4_f32_bf16_bf16_out", gguf_q5_k_mmq32_pipe_q8_1_d4s4_f32_bf16_bf16_out),
                        ("mmq32_mb4_q8_1_d4s4_f32_bf16_bf16_out", gguf_q5_k_mmq32_mb4_q8_1_d4s4_f32_bf16_bf16_out),
                        ("mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_bf16_out", gguf_q5_k_mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_bf16_out),
                        ("mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_f32_out", gguf_q5_k_mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_f32_out)):
        register(KernelKey(backend, "linear", "gguf_q5_k", variant), fn, replace=replace)
    register(KernelKey(backend, "linear", "gguf_q6_k", "mmq32_q8_1_d4s4_f32_bf16_f32_out"),
             gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, replace=replace)
    register(KernelKey(backend, "linear", "gguf_q6_k", "mmq32_q8_1_d4s4_f32_bf16_bf16_out"),
             gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out, replace=replace)
    register(KernelKey(backend, "linear", "gguf_q8_0", "mmq32_q8_1_d4s4_f32_bf16_f32_out"),
             gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_f32_out, replace=replace)
    register(KernelKey(backend, "linear", "gguf_q8_0", "mmq32_q8_1_d4s4_f32_bf16_bf16_out"),
             gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_bf16_out, replace=replace)
