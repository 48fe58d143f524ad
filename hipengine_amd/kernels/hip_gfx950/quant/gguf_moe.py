"""Expert-indexed GGUF k-quant matmul wrappers: decode selected GEMV (single,
gate/up with SiLU, routed down sum) and the expert-grouped Q4_K x DS4 MMQ.

Signatures of the named wrappers follow hipEngine
(``gguf_q4_k_gemv.py:667-715,1403`` for the selected GEMV family,
``gguf_q4_k_q8_1_selected_prefill.py`` for the grouped MMQ); registry keys as in
``gguf_q4_k_gemv.py:1534-1567``.  Raw device pointers throughout.
"""

from __future__ import annotations

import ctypes

from hipengine_amd.core.hip import HipRuntime
from hipengine_amd.kernels.hip_gfx950._launch import (ALLOWED_THREADS, GGML_Q4_K, I32, I64, QUANT_KEY_TO_GGML, VOID,
                                                       check_launch, entry, validate_pointers)
from hipengine_amd.kernels.registry import KernelKey, register

SEL_SINGLE, SEL_DUAL_SILU, SEL_DOWN_SUM = 0, 1, 2
_KIND = {"f32": 0, "bf16": 1, "fp16": 2}


def _validate_selected(x_rows: int, rows: int, num_experts: int, in_features: int, out_features: int,
                       threads: int) -> None:
    """Checks of hipEngine's ``_validate_selected`` (``gguf_q4_k_gemv.py:960-985``)."""
    if x_rows <= 0 or rows <= 0:
        raise ValueError("x_rows and rows must be positive")
    if rows % x_rows != 0:
        raise ValueError("rows must be a multiple of x_rows")
    if rows > 65535:
        raise ValueError("rows must be at most 65535 lanes")
    if num_experts <= 0:
        raise ValueError("num_experts must be positive")
    if in_features <= 0 or in_features % 256 != 0:
        raise ValueError("in_features must be positive and divisible by the GGUF block size 256")
    if out_features <= 0:
        raise ValueError("out_features must be positive")
    if threads not in ALLOWED_THREADS:
        raise ValueError("threads must be one of 64, 128, 256")


def gguf_q4_k_selected_gemv_bf16_bf16_out(x_ptr: int, selected_ptr: int, qweight_ptr: int, out_ptr: int, x_rows: int,
                                          rows: int, num_experts: int, in_features: int, out_features: int, *,
                                          threads: int = 128, stream: int = 0, library: ctypes.CDLL | None = None,
                                          runtime: HipRuntime | None = None) -> None:
    """``out[lane] = W[selected[lane]] . x[lane // (rows // x_rows)]``, bf16 in and out."""
    _validate_selected(x_rows, rows, num_experts, in_features, out_features, threads)
    validate_pointers(x_ptr=x_ptr, selected_ptr=selected_ptr, qweight_ptr=qweight_ptr, out_ptr=out_ptr)
    fn = entry("hipengine_gguf_q4_k_selected_gemv_bf16_bf16_out", [VOID] * 4 + [I64] * 6 + [VOID], library)
    check_launch(fn(x_ptr, selected_ptr, qweight_ptr, out_ptr, x_rows, rows, num_experts, in_features, out_features,
                    threads, stream), runtime)


def _make_selected_k(quant: str):
    """``gguf_<q>_selected_gemv_bf16_bf16_out`` and ``gguf_<q>_selected_silu_gemv_bf16_bf16_out`` for Q5_K, Q6_K and
    Q8_0 experts (hipEngine ``gguf_k_gemv.py:229-232,497,713-716,789-792,1587-1634``)."""
    single_symbol = f"hipengine_gguf_{quant}_selected_gemv_bf16_bf16_out"
    silu_symbol = f"hipengine_gguf_{quant}_selected_silu_gemv_bf16_bf16_out"

    def single(x_ptr: int, selected_ptr: int, qweight_ptr: int, out_ptr: int, x_rows: int, rows: int,
               num_experts: int, in_features: int, out_features: int, *, threads: int = 128, stream: int = 0,
               library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
        _validate_selected(x_rows, rows, num_experts, in_features, out_features, threads)
        validate_pointers(x_ptr=x_ptr, selected_ptr=selected_ptr, qweight_ptr=qweight_ptr, out_ptr=out_ptr)
        fn = entry(single_symbol, [VOID] * 4 + [I64] * 6 + [VOID], library)
        check_launch(fn(x_ptr, selected_ptr, qweight_ptr, out_ptr, x_rows, rows, num_experts, in_features,
                        out_features, threads, stream), runtime)

    def silu(gate_ptr: int, up_ptr: int, selected_ptr: int, qweight_ptr: int, out_ptr: int, x_rows: int, rows: int,
             num_experts: int, in_features: int, out_features: int, *, threads: int = 128, stream: int = 0,
             library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
        _validate_selected(x_rows, rows, num_experts, in_features, out_features, threads)
        validate_pointers(gate_ptr=gate_ptr, up_ptr=up_ptr, selected_ptr=selected_ptr, qweight_ptr=qweight_ptr,
                          out_ptr=out_ptr)
        fn = entry(silu_symbol, [VOID] * 5 + [I64] * 6 + [VOID], library)
        check_launch(fn(gate_ptr, up_ptr, selected_ptr, qweight_ptr, out_ptr, x_rows, rows, num_experts, in_features,
                        out_features, threads, stream), runtime)

    single.__name__ = f"gguf_{quant}_selected_gemv_bf16_bf16_out"
    single.__doc__ = (f"``out[lane] = W[selected[lane]] . x[lane // (rows // x_rows)]`` for {quant.upper()} experts, "
                      f"bf16 in and out (C symbol ``{single_symbol}``).")
    silu.__name__ = f"gguf_{quant}_selected_silu_gemv_bf16_bf16_out"
    silu.__doc__ = (f"``out[lane] = W[selected[lane]] . bf16(silu(gate[r]) * up[r])``, ``r = lane // (rows // x_rows)``, "
                    f"for {quant.upper()} experts (C symbol ``{silu_symbol}``).")
    return single, silu


SELECTED_K: dict[str, tuple[object, object]] = {}
for _quant in ("q5_k", "q6_k", "q8_0"):
    SELECTED_K[_quant] = _make_selected_k(_quant)
    for _fn in SELECTED_K[_quant]:
        globals()[_fn.__name__] = _fn


def gguf_q4_k_selected_dual_silu_gemv_bf16_bf16_out(x_ptr: int, selected_ptr: int, qweight_a_ptr: int,
                                                    qweight_b_ptr: int, out_ptr: int, x_rows: int, rows: int,
                                                    num_experts: int, in_features: int, out_features: int, *,
                                                    threads: int = 128, stream: int = 0,
                                                    library: ctypes.CDLL | None = None,
                                                    runtime: HipRuntime | None = None) -> None:
    """``out[lane] = silu(gate) * up`` with gate/up rounded to bf16 first, bf16 in and out."""
    _validate_selected(x_rows, rows, num_experts, in_features, out_features, threads)
    validate_pointers(x_ptr=x_ptr, selected_ptr=selected_ptr, qweight_a_ptr=qweight_a_ptr, qweight_b_ptr=qweight_b_ptr,
                      out_ptr=out_ptr)
    fn = entry("hipengine_gguf_q4_k_selected_dual_silu_gemv_bf16_bf16_out", [VOID] * 5 + [I64] * 6 + [VOID], library)
    check_launch(fn(x_ptr, selected_ptr, qweight_a_ptr, qweight_b_ptr, out_ptr, x_rows, rows, num_experts, in_features,
                    out_features, threads, stream), runtime)


def gguf_q4_k_selected_dual_gemv_bf16_bf16_out(x_ptr: int, selected_ptr: int, qweight_a_ptr: int, qweight_b_ptr: int,
                                               out_a_ptr: int, out_b_ptr: int, x_rows: int, rows: int,
                                               num_experts: int, in_features: int, out_features: int, *,
                                               threads: int = 128, stream: int = 0,
                                               library: ctypes.CDLL | None = None,
                                               runtime: HipRuntime | None = None) -> None:
    """Gate and up of every lane in one pass, each to its own output (the ``dual`` call kind;
    hipEngine ``gguf_q4_k_gemv.py`` ``gguf_q4_k_selected_dual_gemv_bf16_bf16_out``)."""
    _validate_selected(x_rows, rows, num_experts, in_features, out_features, threads)
    validate_pointers(x_ptr=x_ptr, selected_ptr=selected_ptr, qweight_a_ptr=qweight_a_ptr, qweight_b_ptr=qweight_b_ptr,
                      out_a_ptr=out_a_ptr, out_b_ptr=out_b_ptr)
    fn = entry("hipengine_gguf_q4_k_selected_dual_gemv_bf16_bf16_out", [VOID] * 6 + [I64] * 6 + [VOID], library)
    check_launch(fn(x_ptr, selected_ptr, qweight_a_ptr, qweight_b_ptr, out_a_ptr, out_b_ptr, x_rows, rows, num_experts,
                    in_features, out_features, threads, stream), runtime)


def gguf_q4_k_selected_dual_gemv_q8_1_dp4a_bf16_bf16_out(xq_ptr: int, selected_ptr: int, qweight_a_ptr: int,
                                                         qweight_b_ptr: int, out_a_ptr: int, out_b_ptr: int,
                                                         x_rows: int, rows: int, num_experts: int, in_features: int,
                                                         out_features: int, *, threads: int = 128, stream: int = 0,
                                                         library: ctypes.CDLL | None = None,
                                                         runtime: HipRuntime | None = None) -> None:
    """The ``dual`` form over pre-quantized 36-byte q8_1 activation rows (caller-owned scratch, written by
    ``gguf_q4_k_quantize_bf16_q8_1``)."""
    _validate_selected(x_rows, rows, num_experts, in_features, out_features, threads)
    validate_pointers(xq_ptr=xq_ptr, selected_ptr=selected_ptr, qweight_a_ptr=qweight_a_ptr, qweight_b_ptr=qweight_b_ptr,
                      out_a_ptr=out_a_ptr, out_b_ptr=out_b_ptr)
    fn = entry("hipengine_gguf_q4_k_selected_dual_gemv_q8_1_dp4a_bf16_bf16_out", [VOID] * 6 + [I64] * 6 + [VOID], library)
    check_launch(fn(xq_ptr, selected_ptr, qweight_a_ptr, qweight_b_ptr, out_a_ptr, out_b_ptr, x_rows, rows, num_experts,
                    in_features, out_features, threads, stream), runtime)


def _make_weighted_down(quant: str):
    symbol = f"hipengine_gguf_{quant}_weighted_selected_down_bf16_bf16_out"

    def wrapper(x_ptr: int, selected_ptr: int, routing_weights_ptr: int, qweight_ptr: int, out_ptr: int, *,
                tokens: int, top_k: int, num_experts: int, in_features: int, out_features: int, threads: int = 0,
                stream: int = 0, library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
        if tokens <= 0:
            raise ValueError("tokens must be positive")
        if top_k <= 0 or top_k > 8:
            raise ValueError("top_k must be in 1..8")
        _validate_selected(tokens, tokens * top_k, num_experts, in_features, out_features, threads or 128)
        validate_pointers(x_ptr=x_ptr, selected_ptr=selected_ptr, routing_weights_ptr=routing_weights_ptr,
                          qweight_ptr=qweight_ptr, out_ptr=out_ptr)
        fn = entry(symbol, [VOID] * 5 + [I64] * 6 + [VOID], library)
        check_launch(fn(x_ptr, selected_ptr, routing_weights_ptr, qweight_ptr, out_ptr, tokens, top_k, num_experts,
                        in_features, out_features, threads or 128, stream), runtime)

    wrapper.__name__ = f"gguf_{quant}_weighted_selected_down_bf16_bf16_out"
    wrapper.__doc__ = ("Routed down projection with the weighted sum over a token's experts fused: the ``weighted_down`` "
                       "call kind, keyword geometry as in hipEngine's ``gguf_iq4_xs_weighted_selected_down_bf16_bf16_out`` "
                       "(``gguf_iq_gemv.py:956-972``).")
    return wrapper


gguf_q4_k_weighted_selected_down_bf16_bf16_out = _make_weighted_down("q4_k")
gguf_q6_k_weighted_selected_down_bf16_bf16_out = _make_weighted_down("q6_k")


def gguf_q4_k_selected_grouped_prefill_compact_rowbatch8_bf16_bf16_out(
        x_ptr: int, expert_start_ptr: int, qweight_ptr: int, out_ptr: int, compact_rows: int, num_experts: int,
        in_features: int, out_features: int, *, stream: int = 0, library: ctypes.CDLL | None = None,
        runtime: HipRuntime | None = None) -> None:
    """Grouped GEMV over gathered compact rows: rows ``[expert_start[e], expert_start[e+1])`` of ``x`` take
    expert ``e`` (hipEngine ``gguf_q4_k_gemv.py:1406-1451``)."""
    if compact_rows <= 0:
        raise ValueError("compact_rows must be positive")
    if num_experts <= 0 or num_experts > 65535:
        raise ValueError("num_experts must be in 1..65535")
    if in_features <= 0 or in_features % 256 != 0:
        raise ValueError("in_features must be positive and divisible by the GGUF block size 256")
    if out_features <= 0:
        raise ValueError("out_features must be positive")
    validate_pointers(x_ptr=x_ptr, expert_start_ptr=expert_start_ptr, qweight_ptr=qweight_ptr, out_ptr=out_ptr)
    fn = entry("hipengine_gguf_q4_k_selected_grouped_prefill_compact_rowbatch8_bf16_bf16_out",
               [VOID] * 4 + [I64] * 4 + [VOID], library)
    check_launch(fn(x_ptr, expert_start_ptr, qweight_ptr, out_ptr, compact_rows, num_experts, in_features, out_features,
                    stream), runtime)


def gguf_grouped_gemv(quant: str, x_ptr: int, expert_start_ptr: int, qweight_ptr: int, out_ptr: int,
                      compact_rows: int, num_experts: int, in_features: int, out_features: int, *,
                      x_dtype: str = "bf16", out_dtype: str = "bf16", stream: int = 0,
                      library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """The grouped GEMV for expert weights of any of the four block types (``hipengine_gfx950_gguf_grouped_gemv``)."""
    if quant not in QUANT_KEY_TO_GGML:
        raise ValueError("quant must be one of " + ", ".join(sorted(QUANT_KEY_TO_GGML)))
    if compact_rows <= 0:
        raise ValueError("compact_rows must be positive")
    if num_experts <= 0 or num_experts > 65535:
        raise ValueError("num_experts must be in 1..65535")
    if in_features <= 0 or in_features % 256 != 0:
        raise ValueError("in_features must be positive and divisible by the GGUF block size 256")
    if out_features <= 0:
        raise ValueError("out_features must be positive")
    validate_pointers(x_ptr=x_ptr, expert_start_ptr=expert_start_ptr, qweight_ptr=qweight_ptr, out_ptr=out_ptr)
    fn = entry("hipengine_gfx950_gguf_grouped_gemv", [I32, VOID, I32, VOID, VOID, VOID, I32, I64, I64, I64, I64, VOID],
               library)
    check_launch(fn(QUANT_KEY_TO_GGML[quant], x_ptr, _KIND[x_dtype], expert_start_ptr, qweight_ptr, out_ptr,
                    _KIND[out_dtype], compact_rows, num_experts, in_features, out_features, stream), runtime)


def gguf_selected_gemv(quant: str, mode: int, x_ptr: int, selected_ptr: int, qweight_a_ptr: int, out_ptr: int,
                       x_rows: int, lanes: int, num_experts: int, in_features: int, out_features: int, *,
                       x_dtype: str = "f32", out_dtype: str = "f32", routing_weights_ptr: int = 0,
                       qweight_b_ptr: int = 0, top_k: int = 1, round_mid: bool = False, stream: int = 0,
                       library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """The decode kernels with every choice explicit (``hipengine_gfx950_gguf_selected_gemv``):
    mode 0 single, 1 gate/up with SiLU, 2 routed down projection summed per token."""
    if quant not in ("gguf_q4_k", "gguf_q5_k", "gguf_q6_k", "gguf_q8_0"):
        raise ValueError("quant must be gguf_q4_k, gguf_q5_k, gguf_q6_k or gguf_q8_0")
    if mode == SEL_DUAL_SILU and quant in ("gguf_q5_k", "gguf_q8_0") and in_features > 4096:
        raise ValueError("the gate/up form takes gguf_q5_k and gguf_q8_0 experts up to in_features 4096")
    if mode not in (SEL_SINGLE, SEL_DUAL_SILU, SEL_DOWN_SUM):
        raise ValueError("mode must be 0, 1 or 2")
    if mode == SEL_DOWN_SUM:
        if lanes != x_rows * top_k:
            raise ValueError("lanes must equal x_rows * top_k for the routed down sum")
        if top_k > 8:
            raise ValueError("the routed down sum handles at most 8 experts per token")
        _validate_selected(x_rows, lanes, num_experts, in_features, out_features, 128)
        validate_pointers(routing_weights_ptr=routing_weights_ptr)
    else:
        _validate_selected(x_rows, lanes, num_experts, in_features, out_features, 128)
    if mode == SEL_DUAL_SILU:
        validate_pointers(qweight_b_ptr=qweight_b_ptr)
    validate_pointers(x_ptr=x_ptr, selected_ptr=selected_ptr, qweight_a_ptr=qweight_a_ptr, out_ptr=out_ptr)
    fn = entry("hipengine_gfx950_gguf_selected_gemv",
               [I32, I32, VOID, I32, VOID, VOID, VOID, VOID, VOID, I32, I64, I64, I64, I64, I64, I64, I32, VOID], library)
    check_launch(fn(QUANT_KEY_TO_GGML[quant], mode, x_ptr, _KIND[x_dtype], selected_ptr, routing_weights_ptr or None,
                    qweight_a_ptr, qweight_b_ptr or None, out_ptr, _KIND[out_dtype], x_rows, lanes, num_experts, top_k,
                    in_features, out_features, 1 if round_mid else 0, stream), runtime)


def _validate_grouped(compact_rows: int, in_features: int, out_features_a: int, out_features_b: int, num_experts: int,
                      mmq_total_rows: int) -> None:
    if compact_rows <= 0 or num_experts <= 0:
        raise ValueError("compact_rows and num_experts must be positive")
    if in_features <= 0 or in_features % 256 != 0:
        raise ValueError("in_features must be positive and divisible by the GGUF block size 256")
    if out_features_a <= 0 or out_features_a % 32 != 0 or out_features_b < 0 or out_features_b % 32 != 0:
        raise ValueError("out_features_a / out_features_b must be multiples of 32")
    if mmq_total_rows <= 0 or mmq_total_rows % 32 != 0:
        raise ValueError("mmq_total_rows must be a positive multiple of 32")


def gguf_q4_k_selected_dual_q8_1_ds4_mmq32_prefill_compact32_bf16_bf16_out(
        x_q8_ptr: int, compact_to_source_ptr: int, expert_start_compact_ptr: int, expert_start_mmq32_ptr: int,
        tile_expert_ptr: int, qweight_a_ptr: int, qweight_b_ptr: int, out_ptr: int, compact_rows: int,
        in_features: int, out_features_a: int, out_features_b: int, num_experts: int, mmq_total_rows: int, *,
        expert_stride_rows: int = 0, stream: int = 0, library: ctypes.CDLL | None = None,
        runtime: HipRuntime | None = None) -> None:
    """Expert-grouped gate|up MMQ over DS4 activations, bf16 out ``[compact_rows, Na+Nb]``."""
    _validate_grouped(compact_rows, in_features, out_features_a, out_features_b, num_experts, mmq_total_rows)
    validate_pointers(x_q8_ptr=x_q8_ptr, compact_to_source_ptr=compact_to_source_ptr,
                      expert_start_compact_ptr=expert_start_compact_ptr, expert_start_mmq32_ptr=expert_start_mmq32_ptr,
                      tile_expert_ptr=tile_expert_ptr, qweight_a_ptr=qweight_a_ptr, qweight_b_ptr=qweight_b_ptr,
                      out_ptr=out_ptr)
    fn = entry("hipengine_gguf_q4_k_selected_dual_q8_1_ds4_mmq32_prefill_compact32_bf16_bf16_out",
               [VOID] * 8 + [I64] * 7 + [VOID], library)
    check_launch(fn(x_q8_ptr, compact_to_source_ptr, expert_start_compact_ptr, expert_start_mmq32_ptr, tile_expert_ptr,
                    qweight_a_ptr, qweight_b_ptr, out_ptr, compact_rows, in_features, out_features_a, out_features_b,
                    num_experts, mmq_total_rows, expert_stride_rows, stream), runtime)


def gguf_q4_k_selected_dual_q8_1_ds4_mmq32x128_prefill_compact32_bf16_bf16_out(
        x_q8_ptr: int, compact_to_source_ptr: int, expert_start_compact_ptr: int, expert_start_mmq32_ptr: int,
        mmq_tile_expert_ptr: int, qweight_a_ptr: int, qweight_b_ptr: int, out_ptr: int, compact_rows: int,
        in_features: int, out_features_a: int, out_features_b: int, num_experts: int, mmq_total_rows: int, *,
        stream: int = 0, library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """hipEngine's 128-wide K pass of the same GEMM (``gguf_q4_k_q8_1_selected_prefill.py:1895-1960``): identical
    arithmetic, the one kernel form here."""
    _validate_grouped(compact_rows, in_features, out_features_a, out_features_b, num_experts, mmq_total_rows)
    validate_pointers(x_q8_ptr=x_q8_ptr, compact_to_source_ptr=compact_to_source_ptr,
                      expert_start_compact_ptr=expert_start_compact_ptr, expert_start_mmq32_ptr=expert_start_mmq32_ptr,
                      mmq_tile_expert_ptr=mmq_tile_expert_ptr, qweight_a_ptr=qweight_a_ptr, qweight_b_ptr=qweight_b_ptr,
                      out_ptr=out_ptr)
    fn = entry("hipengine_gguf_q4_k_selected_dual_q8_1_ds4_mmq32x128_prefill_compact32_bf16_bf16_out",
               [VOID] * 8 + [I64] * 6 + [VOID], library)
    check_launch(fn(x_q8_ptr, compact_to_source_ptr, expert_start_compact_ptr, expert_start_mmq32_ptr,
                    mmq_tile_expert_ptr, qweight_a_ptr, qweight_b_ptr, out_ptr, compact_rows, in_features,
                    out_features_a, out_features_b, num_experts, mmq_total_rows, stream), runtime)


def gguf_q4_k_grouped_mmq(x_q8_ptr: int, expert_start_compact_ptr: int, expert_start_mmq32_ptr: int,
                          tile_expert_ptr: int, qweight_a_ptr: int, out_ptr: int, compact_rows: int, source_rows: int,
                          in_features: int, out_features_a: int, num_experts: int, mmq_total_rows: int, *,
                          compact_to_source_ptr: int = 0, qweight_b_ptr: int = 0, out_features_b: int = 0,
                          out_dtype: str = "f32", expert_stride_rows: int = 0, stream: int = 0,
                          library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None,
                          _symbol: str = "hipengine_gfx950_gguf_q4_k_grouped_mmq") -> None:
    """The grouped MMQ with explicit output type, optional row map and optional second weight."""
    _validate_grouped(compact_rows, in_features, out_features_a, out_features_b, num_experts, mmq_total_rows)
    if source_rows <= 0:
        raise ValueError("source_rows must be positive")
    validate_pointers(x_q8_ptr=x_q8_ptr, expert_start_compact_ptr=expert_start_compact_ptr,
                      expert_start_mmq32_ptr=expert_start_mmq32_ptr, tile_expert_ptr=tile_expert_ptr,
                      qweight_a_ptr=qweight_a_ptr, out_ptr=out_ptr)
    fn = entry(_symbol, [VOID] * 8 + [I32] + [I64] * 8 + [VOID], library)
    check_launch(fn(x_q8_ptr, compact_to_source_ptr or None, expert_start_compact_ptr, expert_start_mmq32_ptr,
                    tile_expert_ptr, qweight_a_ptr, qweight_b_ptr or None, out_ptr, _KIND[out_dtype], compact_rows,
                    source_rows, in_features, out_features_a, out_features_b, num_experts, mmq_total_rows,
                    expert_stride_rows, stream), runtime)


def gguf_q5_k_grouped_mmq(x_d4s4_ptr: int, expert_start_compact_ptr: int, expert_start_mmq32_ptr: int,
                          tile_expert_ptr: int, qweight_a_ptr: int, out_ptr: int, compact_rows: int, source_rows: int,
                          in_features: int, out_features_a: int, num_experts: int, mmq_total_rows: int,
                          **kwargs) -> None:
    """``gguf_q4_k_grouped_mmq`` for Q5_K experts over D4S4 activation blocks (the same 32-row tile map and
    keyword arguments; C symbol ``hipengine_gfx950_gguf_q5_k_grouped_mmq``)."""
    gguf_q4_k_grouped_mmq(x_d4s4_ptr, expert_start_compact_ptr, expert_start_mmq32_ptr, tile_expert_ptr,
                          qweight_a_ptr, out_ptr, compact_rows, source_rows, in_features, out_features_a, num_experts,
                          mmq_total_rows, _symbol="hipengine_gfx950_gguf_q5_k_grouped_mmq", **kwargs)


def moe_silu_mul(gate_up_ptr: int, out_ptr: int, rows: int, inter: int, *, in_dtype: str = "f32",
                 out_dtype: str = "f32", stream: int = 0, library: ctypes.CDLL | None = None,
                 runtime: HipRuntime | None = None) -> None:
    """``out[r, c] = silu(gate_up[r, c]) * gate_up[r, inter + c]``."""
    if rows <= 0 or inter <= 0:
        raise ValueError("rows and inter must be positive")
    validate_pointers(gate_up_ptr=gate_up_ptr, out_ptr=out_ptr)
    fn = entry("hipengine_gfx950_moe_silu_mul", [VOID, VOID, I64, I64, ctypes.c_int, ctypes.c_int, VOID], library)
    check_launch(fn(gate_up_ptr, out_ptr, rows, inter, _KIND[in_dtype], _KIND[out_dtype], stream), runtime)


def moe_silu_mul_ds4_pack(gate_up_ptr: int, out_ptr: int, rows: int, inter: int, *, in_dtype: str = "f32",
                          stream: int = 0, library: ctypes.CDLL | None = None,
                          runtime: HipRuntime | None = None) -> None:
    """``silu(gate) * up`` rounded to bf16 and packed to DS4 blocks ``[rows, inter/128]`` in one launch."""
    if rows <= 0 or inter <= 0 or inter % 128 != 0:
        raise ValueError("rows must be positive and inter a positive multiple of 128")
    validate_pointers(gate_up_ptr=gate_up_ptr, out_ptr=out_ptr)
    fn = entry("hipengine_gfx950_moe_silu_mul_ds4_pack", [VOID, ctypes.c_int, VOID, I64, I64, VOID], library)
    check_launch(fn(gate_up_ptr, _KIND[in_dtype], out_ptr, rows, inter, stream), runtime)


def moe_silu_mul_d4s4_pack(gate_up_ptr: int, out_ptr: int, rows: int, inter: int, *, in_dtype: str = "f32",
                           stream: int = 0, library: ctypes.CDLL | None = None,
                           runtime: HipRuntime | None = None) -> None:
    """``silu(gate) * up`` rounded to bf16 and packed to D4S4 blocks ``[rows, inter/128]`` in one launch."""
    if rows <= 0 or inter <= 0 or inter % 128 != 0:
        raise ValueError("rows must be positive and inter a positive multiple of 128")
    validate_pointers(gate_up_ptr=gate_up_ptr, out_ptr=out_ptr)
    fn = entry("hipengine_gfx950_moe_silu_mul_d4s4_pack", [VOID, ctypes.c_int, VOID, I64, I64, VOID], library)
    check_launch(fn(gate_up_ptr, _KIND[in_dtype], out_ptr, rows, inter, stream), runtime)


def gguf_q6_k_grouped_mmq(x_d4s4_ptr: int, expert_start_compact_ptr: int, expert_start_tiles_ptr: int,
                          tile_expert_ptr: int, qweight_a_ptr: int, out_ptr: int, compact_rows: int, source_rows: int,
                          in_features: int, out_features_a: int, num_experts: int, total_rows: int, *,
                          compact_to_source_ptr: int = 0, qweight_b_ptr: int = 0, out_features_b: int = 0,
                          out_dtype: str = "f32", expert_stride_rows: int = 0, stream: int = 0,
                          library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None,
                          _symbol: str = "hipengine_gfx950_gguf_q6_k_grouped_mmq", _block: int = 256) -> None:
    """The expert-grouped MMQ for Q6_K experts over D4S4 activation blocks and a map of 128-row tiles
    (``hipengine_gfx950_gguf_q6_k_grouped_mmq``; tile map from ``group_scatter.moe_tile_map(..., tile_rows=128)``)."""
    if compact_rows <= 0 or num_experts <= 0 or source_rows <= 0:
        raise ValueError("compact_rows, source_rows and num_experts must be positive")
    if in_features <= 0 or in_features % _block != 0:
        raise ValueError("in_features must be positive and divisible by " +
                         ("the GGUF block size 256" if _block == 256 else f"{_block}"))
    if out_features_a <= 0 or out_features_b < 0:
        raise ValueError("out_features_a must be positive and out_features_b non-negative")
    if total_rows <= 0 or total_rows % 128 != 0:
        raise ValueError("total_rows must be a positive multiple of 128")
    validate_pointers(x_d4s4_ptr=x_d4s4_ptr, expert_start_compact_ptr=expert_start_compact_ptr,
                      expert_start_tiles_ptr=expert_start_tiles_ptr, tile_expert_ptr=tile_expert_ptr,
                      qweight_a_ptr=qweight_a_ptr, out_ptr=out_ptr)
    fn = entry(_symbol, [VOID] * 8 + [I32] + [I64] * 8 + [VOID], library)
    check_launch(fn(x_d4s4_ptr, compact_to_source_ptr or None, expert_start_compact_ptr, expert_start_tiles_ptr,
                    tile_expert_ptr, qweight_a_ptr, qweight_b_ptr or None, out_ptr, _KIND[out_dtype], compact_rows,
                    source_rows, in_features, out_features_a, out_features_b, num_experts, total_rows,
                    expert_stride_rows, stream), runtime)


def gguf_q8_0_grouped_mmq(x_d4s4_ptr: int, expert_start_compact_ptr: int, expert_start_tiles_ptr: int,
                          tile_expert_ptr: int, qweight_a_ptr: int, out_ptr: int, compact_rows: int, source_rows: int,
                          in_features: int, out_features_a: int, num_experts: int, total_rows: int, **kwargs) -> None:
    """``gguf_q6_k_grouped_mmq`` for Q8_0 experts (the same 128-row tile map and keyword arguments, in_features a
    multiple of 128; C symbol ``hipengine_gfx950_gguf_q8_0_grouped_mmq``)."""
    gguf_q6_k_grouped_mmq(x_d4s4_ptr, expert_start_compact_ptr, expert_start_tiles_ptr, tile_expert_ptr, qweight_a_ptr,
                          out_ptr, compact_rows, source_rows, in_features, out_features_a, num_experts, total_rows,
                          _symbol="hipengine_gfx950_gguf_q8_0_grouped_mmq", _block=128, **kwargs)


def moe_weighted_gather_sum(down_ptr: int, lane_to_compact_ptr: int, routing_weights_ptr: int, out_ptr: int,
                            tokens: int, top_k: int, hidden: int, compact_rows: int, *, in_dtype: str = "f32",
                            out_dtype: str = "f32", stream: int = 0, library: ctypes.CDLL | None = None,
                            runtime: HipRuntime | None = None) -> None:
    """``out[t] = sum_s routing[t, s] * down[lane_to_compact[t*top_k+s]]`` in slot order."""
    if tokens <= 0 or tokens > 65535 or top_k <= 0 or hidden <= 0 or compact_rows <= 0:
        raise ValueError("tokens (<= 65535), top_k, hidden and compact_rows must be positive")
    validate_pointers(down_ptr=down_ptr, lane_to_compact_ptr=lane_to_compact_ptr,
                      routing_weights_ptr=routing_weights_ptr, out_ptr=out_ptr)
    fn = entry("hipengine_gfx950_moe_weighted_gather_sum",
               [VOID, VOID, VOID, VOID, I64, I64, I64, I64, ctypes.c_int, ctypes.c_int, VOID], library)
    check_launch(fn(down_ptr, lane_to_compact_ptr, routing_weights_ptr, out_ptr, tokens, top_k, hidden, compact_rows,
                    _KIND[in_dtype], _KIND[out_dtype], stream), runtime)


def register_kernels(backend: str = "hip_gfx950", *, replace: bool = False) -> None:
    register(KernelKey(backend, "linear", "gguf_q4_k", "selected_gemv_bf16_bf16_out"),
             gguf_q4_k_selected_gemv_bf16_bf16_out, replace=replace)
    register(KernelKey(backend, "linear", "gguf_q4_k", "selected_dual_silu_gemv_bf16_bf16_out"),
             gguf_q4_k_selected_dual_silu_gemv_bf16_bf16_out, replace=replace)
    for quant, (single, silu) in SELECTED_K.items():     # keys of hipEngine's gguf_k_gemv.py:1938,1987-1989,2022-2023
        register(KernelKey(backend, "linear", f"gguf_{quant}", "selected_gemv_bf16_bf16_out"), single, replace=replace)
        register(KernelKey(backend, "linear", f"gguf_{quant}", "selected_silu_gemv_bf16_bf16_out"), silu,
                 replace=replace)
    register(KernelKey(backend, "linear", "gguf_q4_k", "selected_dual_gemv_bf16_bf16_out"),
             gguf_q4_k_selected_dual_gemv_bf16_bf16_out, replace=replace)
    register(KernelKey(backend, "linear", "gguf_q4_k", "selected_dual_gemv_q8_1_dp4a_bf16_bf16_out"),
             gguf_q4_k_selected_dual_gemv_q8_1_dp4a_bf16_bf16_out, replace=replace)
    register(KernelKey(backend, "moe_linear", "gguf_q4_k", "selected_grouped_prefill_compact_rowbatch8_bf16_bf16_out"),
             gguf_q4_k_selected_grouped_prefill_compact_rowbatch8_bf16_bf16_out, replace=replace)
    # the generic call-kind names of loading/gguf_selected_contract.py:50-54
    register(KernelKey(backend, "moe_linear", "gguf_q4_k", "selected_gemv_decode_bf16_bf16_out"),
             gguf_q4_k_selected_gemv_bf16_bf16_out, replace=replace)
    register(KernelKey(backend, "moe_linear", "gguf_q4_k", "selected_dual_silu_gemv_decode_bf16_bf16_out"),
             gguf_q4_k_selected_dual_silu_gemv_bf16_bf16_out, replace=replace)
    register(KernelKey(backend, "moe_linear", "gguf_q4_k", "selected_weighted_down_gemv_decode_bf16_bf16_out"),
             gguf_q4_k_weighted_selected_down_bf16_bf16_out, replace=replace)
    register(KernelKey(backend, "moe_linear", "gguf_q6_k", "selected_weighted_down_gemv_decode_bf16_bf16_out"),
             gguf_q6_k_weighted_selected_down_bf16_bf16_out, replace=replace)
    register(KernelKey(backend, "moe_linear", "gguf_q4_k",
                       "selected_dual_q8_1_ds4_mmq32_prefill_compact32_bf16_bf16_out"),
             gguf_q4_k_selected_dual_q8_1_ds4_mmq32_prefill_compact32_bf16_bf16_out, replace=replace)
    register(KernelKey(backend, "moe_linear", "gguf_q4_k",
                       "selected_dual_q8_1_ds4_mmq32x128_prefill_compact32_bf16_bf16_out"),
             gguf_q4_k_selected_dual_q8_1_ds4_mmq32x128_prefill_compact32_bf16_bf16_out, replace=replace)
    for _q in ("gguf_q4_k", "gguf_q5_k", "gguf_q6_k", "gguf_q8_0"):
        register(KernelKey(backend, "moe_linear", _q, "grouped_gemv_rowbatch8"),
                 (lambda q: lambda *a, **k: gguf_grouped_gemv(q, *a, **k))(_q), replace=replace)
    register(KernelKey(backend, "moe_linear", "gguf_q4_k", "grouped_mmq32_q8_1_ds4"), gguf_q4_k_grouped_mmq,
             replace=replace)
    register(KernelKey(backend, "moe_linear", "gguf_q6_k", "grouped_mmq128_q8_1_d4s4"), gguf_q6_k_grouped_mmq,
             replace=replace)
    register(KernelKey(backend, "moe_linear", "gguf_q5_k", "grouped_mmq32_q8_1_d4s4"), gguf_q5_k_grouped_mmq,
             replace=replace)
    register(KernelKey(backend, "moe_linear", "gguf_q8_0", "grouped_mmq128_q8_1_d4s4"), gguf_q8_0_grouped_mmq,
             replace=replace)
    for quant in ("gguf_q4_k", "gguf_q5_k", "gguf_q6_k", "gguf_q8_0"):
        register(KernelKey(backend, "moe_linear", quant, "selected_gemv_q8_1"), gguf_selected_gemv, replace=replace)
