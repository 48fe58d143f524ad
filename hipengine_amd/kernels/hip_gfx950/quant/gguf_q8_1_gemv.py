"""Decode GEMV wrappers (batch 1..8 per launch) for Q4_K / Q6_K / Q8_0 weights
with q8_1 activations.

Two families, both with hipEngine's dense wrapper signature
``fn(x_ptr, qweight_ptr, out_ptr, rows, in_features, out_features, *, threads,
stream, library, runtime)`` (``kernels/hip_gfx1100/quant/gguf_q4_k_gemv.py:115-142``):

* ``gguf_<q>_q8_1_fused_gemv_<act>_<out>_out`` take float activations and
  quantize them to q8_1 inside the kernel;
* ``gguf_<q>_gemv_<act>_<out>_out`` / ``gguf_<q>_prefill_<act>_<out>_out`` are hipEngine's own dense names
  (``gguf_q4_k_gemv.py:175-202,524-576``, ``gguf_k_gemv.py:1920-2049``), registered under the keys its
  dispatcher asks for, ``("linear", quant, "gemv_*" / "prefill_*")``; they run the fused kernels;
* ``gguf_q4_k_q8_1_dp4a_vdr_*``, ``gguf_q6_k_q8_1_dp4a_gemv_*`` and
  ``gguf_q8_0_dp4a_[rowtile4_|dual_split_rowtile4_|triple_split_rowtile4_]gemv_*`` take pre-quantized 36-byte
  q8_1 blocks, as hipEngine's ``gguf_q4_k_q8_1_dp4a_vdr_gemv.py`` / ``gguf_q8_0_dp4a_gemv.py`` do.
"""

from __future__ import annotations

import ctypes

from hipengine_amd.core.hip import HipRuntime
from hipengine_amd.kernels.hip_gfx950._launch import (
    I32,
    I64,
    KIND_BF16,
    KIND_F16,
    KIND_F32,
    KIND_Q8_1,
    QUANT_KEY_TO_GGML,
    VOID,
    check_launch,
    entry,
    validate_linear,
    validate_pointers,
)
from hipengine_amd.kernels.hip_gfx950 import _launch
from hipengine_amd.kernels.registry import KernelKey, register

_FUSED_ARGS = [VOID, VOID, VOID, I64, I64, I64, I64, VOID]
_Q8_1_ARGS = [VOID, VOID, VOID, I64, I64, I64, VOID]
_QUANTS = ("q4_k", "q5_k", "q6_k", "q8_0")
_FUSED_DTYPES = (("f32", "f32"), ("bf16", "f32"), ("bf16", "bf16"), ("bf16", "fp16"), ("fp16", "f32"), ("fp16", "fp16"))
_KINDS = {"f32": KIND_F32, "bf16": KIND_BF16, "fp16": KIND_F16, "q8_1": KIND_Q8_1}


def _make_fused(quant: str, act: str, out: str):
    symbol = f"hipengine_gguf_{quant}_q8_1_fused_gemv_{act}_{out}_out"

    default_fn = []          # the configured C function of the default library, resolved at the first call

    def wrapper(x_ptr: int, qweight_ptr: int, out_ptr: int, rows: int, in_features: int, out_features: int, *,
                threads: int = 128, stream: int = 0, library: ctypes.CDLL | None = None,
                runtime: HipRuntime | None = None) -> None:
        if _launch.VALIDATE:
            validate_linear(rows, in_features, out_features, threads)
            validate_pointers(x_ptr=x_ptr, qweight_ptr=qweight_ptr, out_ptr=out_ptr)
        if library is None:
            if not default_fn:
                default_fn.append(entry(symbol, _FUSED_ARGS, None))
            fn = default_fn[0]
        else:
            fn = entry(symbol, _FUSED_ARGS, library)
        code = fn(x_ptr, qweight_ptr, out_ptr, rows, in_features, out_features, threads, stream)
        if code:
            check_launch(code, runtime)

    wrapper.__name__ = f"gguf_{quant}_q8_1_fused_gemv_{act}_{out}_out"
    wrapper.__doc__ = (f"GGUF {quant.upper()} GEMV, {act} activations quantized to q8_1 in the kernel, {out} output "
                       f"(C symbol ``{symbol}``).")
    return wrapper


def _make_q8_1(name: str, symbol: str):
    def wrapper(xq_ptr: int, qweight_ptr: int, out_ptr: int, rows: int, in_features: int, out_features: int, *,
                threads: int = 128, stream: int = 0, library: ctypes.CDLL | None = None,
                runtime: HipRuntime | None = None) -> None:
        validate_linear(rows, in_features, out_features, threads)
        validate_pointers(xq_ptr=xq_ptr, qweight_ptr=qweight_ptr, out_ptr=out_ptr)
        check_launch(entry(symbol, _Q8_1_ARGS, library)(xq_ptr, qweight_ptr, out_ptr, rows, in_features, out_features,
                                                        stream), runtime)

    wrapper.__name__ = name
    wrapper.__doc__ = f"GGUF GEMV over pre-quantized 36-byte q8_1 activation blocks (C symbol ``{symbol}``)."
    return wrapper


_DENSE_DTYPES = (("f32", "f32"), ("f32", "fp16"), ("fp16", "f32"), ("fp16", "fp16"), ("bf16", "f32"), ("bf16", "fp16"),
                 ("bf16", "bf16"))
_MMQ_MIN_ROWS = 32          # from here on a prefill with a workspace goes through pack + MMQ
_PREFILL_ARGS = [I32, VOID, VOID, VOID, I32, I64, I64, I64, VOID, I64, VOID]


def gguf_prefill_workspace_bytes(quant_key: str, rows: int, in_features: int) -> int:
    """Bytes of the workspace a ``prefill_bf16_*`` call takes to run on the MMQ (0: that quant has none)."""
    if quant_key not in ("gguf_q4_k", "gguf_q5_k", "gguf_q6_k", "gguf_q8_0") or in_features % 128:
        return 0
    return rows * (in_features // 128) * (144 if quant_key == "gguf_q4_k" else 160)


def _make_dense(quant: str, family: str, act: str, out: str):
    symbol = f"hipengine_gguf_{quant}_gemv_{'rowtile_' if family == 'gemv_rowtile' else ''}{act}_{out}_out"
    quant_key = f"gguf_{quant}"

    def wrapper(x_ptr: int, qweight_ptr: int, out_ptr: int, rows: int, in_features: int, out_features: int, *,
                threads: int = 128, stream: int = 0, library: ctypes.CDLL | None = None,
                runtime: HipRuntime | None = None, workspace_ptr: int = 0, workspace_bytes: int = 0) -> None:
        validate_linear(rows, in_features, out_features, threads)
        validate_pointers(x_ptr=x_ptr, qweight_ptr=qweight_ptr, out_ptr=out_ptr)
        need = gguf_prefill_workspace_bytes(quant_key, rows, in_features)
        if (family == "prefill" and act == "bf16" and rows >= _MMQ_MIN_ROWS and workspace_ptr and need
                and workspace_bytes >= need and (quant in ("q6_k", "q8_0") or out_features % 32 == 0)):
            code = entry("hipengine_gfx950_gguf_prefill_bf16", _PREFILL_ARGS, library)(
                QUANT_KEY_TO_GGML[quant_key], x_ptr, qweight_ptr, out_ptr, _KINDS[out], rows, in_features, out_features,
                workspace_ptr, workspace_bytes, stream)
        else:
            code = entry(symbol, _FUSED_ARGS, library)(x_ptr, qweight_ptr, out_ptr, rows, in_features, out_features,
                                                       threads, stream)
        check_launch(code, runtime)

    wrapper.__name__ = f"gguf_{quant}_{family}_{act}_{out}_out"
    wrapper.__doc__ = (
        f"hipEngine's dense {family} entry for {quant.upper()} (C symbol ``{symbol}``): {act} activations, quantized to "
        f"q8_1 inside the kernel, {out} output; any number of rows, 8 per launch"
        + ("; from 32 rows of bf16 activations on the C entry runs the int8-MFMA MMQ over chunks of 512 rows packed "
           "into a buffer the library holds (at most two such calls in flight per device)." if act == "bf16" else ".")
        + (" With ``workspace_ptr`` / ``workspace_bytes`` (see ``gguf_prefill_workspace_bytes``) and 32 rows or more, "
           "bf16 activations are packed into the caller's workspace instead and the MMQ runs once over all rows "
           "(same bits)." if family == "prefill" else ""))
    return wrapper


def _make_dense_dual(quant: str, act: str, out: str):
    symbol = f"hipengine_gguf_{quant}_dual_gemv_{act}_{out}_out"

    def wrapper(x_ptr: int, qweight_a_ptr: int, qweight_b_ptr: int, out_a_ptr: int, out_b_ptr: int, rows: int,
                in_features: int, out_features: int, *, threads: int = 128, stream: int = 0,
                library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
        validate_linear(rows, in_features, out_features, threads)
        validate_pointers(x_ptr=x_ptr, qweight_a_ptr=qweight_a_ptr, qweight_b_ptr=qweight_b_ptr, out_a_ptr=out_a_ptr,
                          out_b_ptr=out_b_ptr)
        code = entry(symbol, [VOID] * 5 + [I64] * 4 + [VOID], library)(
            x_ptr, qweight_a_ptr, qweight_b_ptr, out_a_ptr, out_b_ptr, rows, in_features, out_features, threads, stream)
        check_launch(code, runtime)

    wrapper.__name__ = f"gguf_{quant}_dual_gemv_{act}_{out}_out"
    wrapper.__doc__ = (f"Two {quant.upper()} matrices over one activation: ``out_a = W_a x``, ``out_b = W_b x`` "
                       f"(C symbol ``{symbol}``; hipEngine ``gguf_k_gemv.py`` dual wrappers).")
    return wrapper


DENSE: dict[tuple[str, str, str, str], object] = {}
for _q in _QUANTS:
    for _family in ("gemv", "prefill"):
        for _a, _o in _DENSE_DTYPES:
            _fn = _make_dense(_q, _family, _a, _o)
            DENSE[(_q, _family, _a, _o)] = _fn
            globals()[_fn.__name__] = _fn
for _q in _QUANTS:       # hipEngine's rowtile names (gguf_q4_k_gemv.py:1517-1519,1552-1554): the same launch
    for _a, _o in (("f32", "f32"), ("bf16", "f32"), ("bf16", "bf16")):
        _fn = _make_dense(_q, "gemv_rowtile", _a, _o)
        DENSE[(_q, "gemv_rowtile", _a, _o)] = _fn
        globals()[_fn.__name__] = _fn
DENSE_DUAL = {(q, a, o): _make_dense_dual(q, a, o) for q in _QUANTS for a, o in (("f32", "f32"), ("bf16", "bf16"))}
for _fn in DENSE_DUAL.values():
    globals()[_fn.__name__] = _fn

def lean_fused(quant: str, act: str, out: str, library: ctypes.CDLL | None = None):
    """The C function behind ``FUSED[(quant, act, out)]`` with its argument types set: call it as
    ``fn(x_ptr, qweight_ptr, out_ptr, rows, in_features, out_features, threads, stream)`` and test the returned
    ``hipError_t``.  For loops that have validated their shapes once (one ctypes call per launch)."""
    return _launch.lean_entry(f"hipengine_gguf_{quant}_q8_1_fused_gemv_{act}_{out}_out", _FUSED_ARGS, library)


FUSED: dict[tuple[str, str, str], object] = {}
for _q in _QUANTS:
    for _a, _o in _FUSED_DTYPES:
        _fn = _make_fused(_q, _a, _o)
        FUSED[(_q, _a, _o)] = _fn
        globals()[_fn.__name__] = _fn

gguf_q4_k_q8_1_dp4a_vdr_bf16_f32_out = _make_q8_1(
    "gguf_q4_k_q8_1_dp4a_vdr_bf16_f32_out", "hipengine_gguf_q4_k_q8_1_dp4a_vdr_bf16_f32_out")
gguf_q4_k_q8_1_dp4a_vdr_bf16_bf16_out = _make_q8_1(
    "gguf_q4_k_q8_1_dp4a_vdr_bf16_bf16_out", "hipengine_gguf_q4_k_q8_1_dp4a_vdr_bf16_bf16_out")
gguf_q6_k_q8_1_dp4a_gemv_bf16_f32_out = _make_q8_1(
    "gguf_q6_k_q8_1_dp4a_gemv_bf16_f32_out", "hipengine_gguf_q6_k_q8_1_dp4a_gemv_bf16_f32_out")
gguf_q6_k_q8_1_dp4a_gemv_bf16_bf16_out = _make_q8_1(
    "gguf_q6_k_q8_1_dp4a_gemv_bf16_bf16_out", "hipengine_gguf_q6_k_q8_1_dp4a_gemv_bf16_bf16_out")
gguf_q4_k_q8_1_dp4a_ctl_bf16_f32_out = _make_q8_1(
    "gguf_q4_k_q8_1_dp4a_ctl_bf16_f32_out", "hipengine_gguf_q4_k_q8_1_dp4a_ctl_bf16_f32_out")
gguf_q4_k_q8_1_dp4a_ctl_bf16_bf16_out = _make_q8_1(
    "gguf_q4_k_q8_1_dp4a_ctl_bf16_bf16_out", "hipengine_gguf_q4_k_q8_1_dp4a_ctl_bf16_bf16_out")


def _make_q8_0_dp4a(name: str, count: int):
    """hipEngine's Q8_0 entries over q8_1 activations (``gguf_q8_0_dp4a_gemv.py:124-400``): ``count`` weights and
    outputs, then rows, in_features, one out_features per weight, a ``threads`` slot (passed as 0, as hipEngine's
    wrappers do) and the stream."""
    symbol = f"hipengine_{name}"
    argtypes = [VOID] * (1 + 2 * count) + [I64] * (2 + count) + [I64, VOID]

    def wrapper(xq_ptr: int, *args: int, stream: int = 0, library: ctypes.CDLL | None = None,
                runtime: HipRuntime | None = None) -> None:
        if len(args) != 3 * count + 2:
            raise TypeError(f"{name} takes xq_ptr, {count} weight and {count} output pointers, rows, in_features and "
                            f"{count} out_features")
        pointers, (rows, in_features, *out_features) = args[:2 * count], args[2 * count:]
        for n in out_features:
            validate_linear(rows, in_features, n, 128)
        validate_pointers(xq_ptr=xq_ptr, **{f"ptr_{i}": p for i, p in enumerate(pointers)})
        check_launch(entry(symbol, argtypes, library)(xq_ptr, *pointers, rows, in_features, *out_features, 0, stream),
                     runtime)

    wrapper.__name__ = name
    wrapper.__doc__ = (f"GGUF Q8_0 GEMV of {count} matri{'x' if count == 1 else 'ces'} over pre-quantized q8_1 "
                       f"activation blocks (C symbol ``{symbol}``).")
    return wrapper


Q8_0_DP4A: dict[str, object] = {}
for _shape, _count in (("", 1), ("rowtile4_", 1), ("dual_split_rowtile4_", 2), ("triple_split_rowtile4_", 3)):
    for _suffix in ("f32_f32_out", "bf16_bf16_out"):
        _fn = _make_q8_0_dp4a(f"gguf_q8_0_dp4a_{_shape}gemv_{_suffix}", _count)
        Q8_0_DP4A[f"q8_1_dp4a_{_shape}gemv_{_suffix}"] = _fn
        globals()[_fn.__name__] = _fn

_TUNED_ARGS = [I32, VOID, I32, VOID, VOID, I32, I64, I64, I64, I32, I32, I32, I32, VOID]


def gguf_q8_1_fused_gemv_tuned(quant_key: str, x_ptr: int, x_kind: str, qweight_ptr: int, out_ptr: int, out_kind: str,
                               rows: int, in_features: int, out_features: int, *, k_slices: int, row_groups: int,
                               blocks_per_wave: int, rows_per_lane: int, stream: int = 0,
                               library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """The fused GEMV with an explicit workgroup layout (tuning sweeps only)."""
    validate_linear(rows, in_features, out_features)
    fn = entry("hipengine_gfx950_gguf_q8_1_fused_gemv_tuned", _TUNED_ARGS, library)
    check_launch(fn(QUANT_KEY_TO_GGML[quant_key], x_ptr, _KINDS[x_kind], qweight_ptr, out_ptr, _KINDS[out_kind], rows,
                    in_features, out_features, k_slices, row_groups, blocks_per_wave, rows_per_lane, stream), runtime)


_RUN_TUNED_ARGS = [I32, VOID, I32, VOID, VOID, I32, I64, I64, I64, I32, I32, I32, VOID]


def gguf_q8_1_fused_gemv_run_tuned(quant_key: str, x_ptr: int, x_kind: str, qweight_ptr: int, out_ptr: int,
                                   out_kind: str, rows: int, in_features: int, out_features: int, *,
                                   rows_per_wave: int, loads_per_chunk: int, waves: int, stream: int = 0,
                                   library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """The run form of the fused GEMV with an explicit layout (tuning sweeps only)."""
    validate_linear(rows, in_features, out_features)
    fn = entry("hipengine_gfx950_gguf_q8_1_fused_gemv_run_tuned", _RUN_TUNED_ARGS, library)
    check_launch(fn(QUANT_KEY_TO_GGML[quant_key], x_ptr, _KINDS[x_kind], qweight_ptr, out_ptr, _KINDS[out_kind], rows,
                    in_features, out_features, rows_per_wave, loads_per_chunk, waves, stream), runtime)


def gguf_q8_1_fused_gemv_stream_tuned(quant_key: str, x_ptr: int, x_kind: str, qweight_ptr: int, out_ptr: int,
                                      out_kind: str, rows: int, in_features: int, out_features: int, *,
                                      loads_in_flight: int, waves: int, waves_total: int, stream: int = 0,
                                      library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """The stream form of the fused GEMV with an explicit layout (tuning sweeps only)."""
    validate_linear(rows, in_features, out_features)
    fn = entry("hipengine_gfx950_gguf_q8_1_fused_gemv_stream_tuned", _RUN_TUNED_ARGS, library)
    check_launch(fn(QUANT_KEY_TO_GGML[quant_key], x_ptr, _KINDS[x_kind], qweight_ptr, out_ptr, _KINDS[out_kind], rows,
                    in_features, out_features, loads_in_flight, waves, waves_total, stream), runtime)


class FusedFormUnavailable(ValueError):
    """The shape is outside the fused kernel's range; run the unfused sequence instead (hipEngine's
    ``launch_gguf_linear_pair_silu`` / ``launch_gguf_linear_residual`` return False in that case:
    ``runtime/qwen35_gguf_layer_ffn.py:519-538,619-630``)."""


def gguf_pair_silu_gemv(quant_key: str, x_ptr: int, x_kind: str, qweight_gate_ptr: int, qweight_up_ptr: int,
                        out_ptr: int, out_kind: str, rows: int, in_features: int, out_features: int, *,
                        round_mid: bool = True, stream: int = 0, library: ctypes.CDLL | None = None,
                        runtime: HipRuntime | None = None) -> None:
    """Dense FFN gate/up pair in one pass with SiLU*up fused: ``out = silu(gate x) * (up x)``.
    ``round_mid`` rounds gate and up to the output type first, as the unfused GEMV, GEMV, silu_mul sequence
    does through its stored intermediates.  Rows 1-2: one launch (Q4_K, stream form).  Rows 3-8: two launches on
    the MFMA forms, the gate projection stored to ``out`` and read back by the up projection's epilogue (any
    type; 16-bit outputs need ``round_mid``, which is what storing the gate does).  Raises
    :class:`FusedFormUnavailable` outside those ranges."""
    validate_linear(rows, in_features, out_features)
    validate_pointers(x_ptr=x_ptr, qweight_gate_ptr=qweight_gate_ptr, qweight_up_ptr=qweight_up_ptr, out_ptr=out_ptr)
    if rows > 8 or (rows <= 2 and (quant_key != "gguf_q4_k" or in_features < 4096)):
        raise FusedFormUnavailable("pair_silu: rows <= 2 need Q4_K and in_features >= 4096; rows <= 8")
    if rows > 2 and not round_mid and out_kind != "f32":
        raise FusedFormUnavailable("pair_silu: rows 3-8 with a 16-bit output round the gate (round_mid)")
    fn = entry("hipengine_gfx950_gguf_pair_silu_gemv",
               [I32, VOID, I32, VOID, VOID, VOID, I32, I64, I64, I64, I32, VOID], library)
    code = fn(QUANT_KEY_TO_GGML[quant_key], x_ptr, _KINDS[x_kind], qweight_gate_ptr, qweight_up_ptr, out_ptr,
              _KINDS[out_kind], rows, in_features, out_features, int(bool(round_mid)), stream)
    if code == 1:
        raise FusedFormUnavailable("pair_silu: shape outside the fused kernels' range")
    check_launch(code, runtime)


def gguf_gemv_residual(quant_key: str, x_ptr: int, x_kind: str, qweight_ptr: int, residual_ptr: int, out_ptr: int,
                       out_kind: str, rows: int, in_features: int, out_features: int, *, stream: int = 0,
                       library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """Projection with the residual add fused: ``out = round(W x) + residual`` in the output type
    (``residual_ptr`` may equal ``out_ptr``).  Raises :class:`FusedFormUnavailable` outside the fused range."""
    validate_linear(rows, in_features, out_features)
    validate_pointers(x_ptr=x_ptr, qweight_ptr=qweight_ptr, residual_ptr=residual_ptr, out_ptr=out_ptr)
    if quant_key not in ("gguf_q4_k", "gguf_q6_k") or rows > 8:
        raise FusedFormUnavailable("gemv_residual: Q4_K / Q6_K, rows <= 8 only")
    fn = entry("hipengine_gfx950_gguf_gemv_residual",
               [I32, VOID, I32, VOID, VOID, VOID, I32, I64, I64, I64, VOID], library)
    code = fn(QUANT_KEY_TO_GGML[quant_key], x_ptr, _KINDS[x_kind], qweight_ptr, residual_ptr, out_ptr,
              _KINDS[out_kind], rows, in_features, out_features, stream)
    if code == 1:
        raise FusedFormUnavailable("gemv_residual: shape outside the fused kernels' range")
    check_launch(code, runtime)


def gguf_multi_gemv(quant_keys, x_ptr: int, x_kind: str, qweight_ptrs, out_ptrs, out_kind: str, rows: int,
                    in_features: int, out_features, *, stream: int = 0, library: ctypes.CDLL | None = None,
                    runtime: HipRuntime | None = None) -> None:
    """Up to four matrices over one activation, ``out_i = W_i x`` (the q, k and v projections of an attention
    block), whatever their GGUF types and row counts.  Rows 1-2 with ``in_features >= 4096``: one launch, the
    workgroups divided between the matrices by their bytes; otherwise one launch per matrix.  Every output has
    the bits its own fused GEMV call gives (C symbol ``hipengine_gfx950_gguf_multi_gemv``)."""
    count = len(quant_keys)
    if not (1 <= count <= 4) or len(qweight_ptrs) != count or len(out_ptrs) != count or len(out_features) != count:
        raise ValueError("multi_gemv takes 1 to 4 matrices, with one weight, output and out_features each")
    for n in out_features:
        validate_linear(rows, in_features, n)
    validate_pointers(x_ptr=x_ptr, **{f"qweight_{i}": p for i, p in enumerate(qweight_ptrs)},
                      **{f"out_{i}": p for i, p in enumerate(out_ptrs)})
    types = (I32 * count)(*[QUANT_KEY_TO_GGML[q] for q in quant_keys])
    weights = (VOID * count)(*qweight_ptrs)
    outs = (VOID * count)(*out_ptrs)
    ns = (I64 * count)(*out_features)
    fn = entry("hipengine_gfx950_gguf_multi_gemv",
               [I32, ctypes.POINTER(I32), VOID, I32, ctypes.POINTER(VOID), ctypes.POINTER(VOID), I32, I64, I64,
                ctypes.POINTER(I64), VOID], library)
    check_launch(fn(count, types, x_ptr, _KINDS[x_kind], weights, outs, _KINDS[out_kind], rows, in_features, ns, stream),
                 runtime)


def _make_pair_silu(act: str, out: str):
    def wrapper(x_ptr: int, qweight_gate_ptr: int, qweight_up_ptr: int, out_ptr: int, rows: int, in_features: int,
                out_features: int, *, stream: int = 0, library: ctypes.CDLL | None = None,
                runtime: HipRuntime | None = None) -> None:
        gguf_pair_silu_gemv("gguf_q4_k", x_ptr, act, qweight_gate_ptr, qweight_up_ptr, out_ptr, out, rows, in_features,
                            out_features, round_mid=True, stream=stream, library=library, runtime=runtime)

    wrapper.__name__ = f"gguf_q4_k_dual_silu_gemv_{act}_{out}_out"
    wrapper.__doc__ = f"Q4_K gate/up pair with SiLU fused, {act} activations, {out} output (dual+SiLU operand order)."
    return wrapper


def _make_residual(quant: str, act: str, out: str):
    def wrapper(x_ptr: int, qweight_ptr: int, residual_ptr: int, out_ptr: int, rows: int, in_features: int,
                out_features: int, *, stream: int = 0, library: ctypes.CDLL | None = None,
                runtime: HipRuntime | None = None) -> None:
        gguf_gemv_residual(f"gguf_{quant}", x_ptr, act, qweight_ptr, residual_ptr, out_ptr, out, rows, in_features,
                           out_features, stream=stream, library=library, runtime=runtime)

    wrapper.__name__ = f"gguf_{quant}_gemv_{act}_residual_{out}_out"
    wrapper.__doc__ = (f"{quant.upper()} projection + residual, {act} activations, {out} residual and output "
                       "(operand order of hipEngine's pack8_gemv_bf16_residual_bf16_out).")
    return wrapper


PAIR_SILU = {(act, out): _make_pair_silu(act, out) for act, out in (("bf16", "bf16"), ("f32", "f32"))}
RESIDUAL = {(quant, act, out): _make_residual(quant, act, out)
            for quant in ("q4_k", "q6_k") for act, out in (("bf16", "bf16"), ("f32", "f32"))}


def gguf_q4_k_q8_1_fused_gemv_slab_tuned(x_ptr: int, x_kind: str, qweight_ptr: int, out_ptr: int, out_kind: str,
                                         rows: int, in_features: int, out_features: int, *,
                                         rows_per_workgroup: int = 0, stream: int = 0,
                                         library: ctypes.CDLL | None = None,
                                         runtime: HipRuntime | None = None) -> None:
    """The slab (int8 MFMA, K split over the waves of one workgroup per CU) form of the fused Q4_K GEMV with an
    explicit slab height; 0 takes the planner's (tuning sweeps only)."""
    validate_linear(rows, in_features, out_features)
    fn = entry("hipengine_gfx950_gguf_q4_k_q8_1_fused_gemv_slab_tuned",
               [VOID, I32, VOID, VOID, I32, I64, I64, I64, I32, VOID], library)
    check_launch(fn(x_ptr, _KINDS[x_kind], qweight_ptr, out_ptr, _KINDS[out_kind], rows, in_features, out_features,
                    rows_per_workgroup, stream), runtime)


def gguf_q8_1_fused_gemv_pslab_tuned(quant_key: str, x_ptr: int, x_kind: str, qweight_ptr: int, out_ptr: int,
                                     out_kind: str, rows: int, in_features: int, out_features: int, *,
                                     waves: int = 0, blocks_per_wave: int = 0, workgroups: int = 0, stream: int = 0,
                                     library: ctypes.CDLL | None = None,
                                     runtime: HipRuntime | None = None) -> None:
    """The phased slab (int8 MFMA, K blocks dealt to the waves phase by phase) form of the fused Q4_K / Q5_K / Q6_K / Q8_0
    GEMV with an explicit wave count, blocks per wave and phase (1, 2 or 4) and grid; 0 takes the
    planner's (tuning sweeps and tests only)."""
    validate_linear(rows, in_features, out_features)
    fn = entry("hipengine_gfx950_gguf_q8_1_fused_gemv_pslab_tuned",
               [I32, VOID, I32, VOID, VOID, I32, I64, I64, I64, I32, I32, I32, VOID], library)
    check_launch(fn(QUANT_KEY_TO_GGML[quant_key], x_ptr, _KINDS[x_kind], qweight_ptr, out_ptr, _KINDS[out_kind], rows,
                    in_features, out_features, waves, blocks_per_wave, workgroups, stream), runtime)


def gguf_q8_1_fused_gemv_dslab_tuned(quant_key: str, x_ptr: int, x_kind: str, qweight_ptr: int, out_ptr: int,
                                     out_kind: str, rows: int, in_features: int, out_features: int, *,
                                     waves: int = 0, ring: int = 0, workgroups: int = 0, k_parts: int = 0,
                                     stream: int = 0, library: ctypes.CDLL | None = None,
                                     runtime: HipRuntime | None = None) -> None:
    """The direct slab form (weights streamed straight into LDS, int8 MFMA) of the fused GEMV with an explicit
    wave count, ring depth (steps of 16 rows in flight per wave), grid and number of K parts (1, 2, 4); 0 takes
    the planner's (tuning sweeps and tests only)."""
    validate_linear(rows, in_features, out_features)
    fn = entry("hipengine_gfx950_gguf_q8_1_fused_gemv_dslab_tuned",
               [I32, VOID, I32, VOID, VOID, I32, I64, I64, I64, I32, I32, I32, I32, VOID], library)
    check_launch(fn(QUANT_KEY_TO_GGML[quant_key], x_ptr, _KINDS[x_kind], qweight_ptr, out_ptr, _KINDS[out_kind], rows,
                    in_features, out_features, waves, ring, workgroups, k_parts, stream), runtime)


def gguf_gemv_default_plan(quant_key: str, rows: int, in_features: int, out_features: int, *,
                           library: ctypes.CDLL | None = None) -> dict[str, int]:
    """The workgroup layout the library picks for a shape (host only)."""
    plan = (ctypes.c_int32 * 5)()
    fn = entry("hipengine_gfx950_gguf_gemv_default_plan", [I32, I64, I64, I64, ctypes.POINTER(ctypes.c_int32)], library)
    check_launch(fn(QUANT_KEY_TO_GGML[quant_key], rows, in_features, out_features, plan), None)
    return dict(zip(("batch_bucket", "rows_per_lane", "blocks_per_wave", "k_slices", "row_groups"), plan))


GEMV_FORMS = ("row_strided", "run", "stream", "slab", "phased_slab", "direct_slab")


def gguf_gemv_default_form(quant_key: str, rows: int, in_features: int, out_features: int, *,
                           library: ctypes.CDLL | None = None) -> tuple[str, int]:
    """The kernel form the default dispatch takes for a shape and the batch rows of its first launch (host only)."""
    form = (ctypes.c_int32 * 2)()
    fn = entry("hipengine_gfx950_gguf_gemv_default_form", [I32, I64, I64, I64, ctypes.POINTER(ctypes.c_int32)], library)
    check_launch(fn(QUANT_KEY_TO_GGML[quant_key], rows, in_features, out_features, form), None)
    return GEMV_FORMS[form[0]], int(form[1])


# hipEngine's per-shape tuning variants of the dense GEMV (gguf_k_gemv.py: rowbatch / coltile / wave32x2 / pipelined
# forms for Q5_K, Q6_K and Q8_0): the dense launch under those names.  (quant, variant) -> wrapper.
_DENSE_VARIANT_NAMES = (
    *((q, f"gemv_rowbatch{rb}_bf16_{o}_out") for q in ("q5_k", "q6_k") for rb in (8, 32) for o in ("bf16", "f32")),
    *((q, f"gemv_coltile{c}_rowbatch{r}_bf16_{o}_out") for q in ("q5_k", "q6_k") for c, r in ((2, 16), (4, 8))
      for o in ("bf16", "f32")),
    *(("q5_k", f"wave32x2{m}_gemv_decode_bf16_{o}_out") for m in ("", "_fixed_meta", "_swar_pair_fixed_meta")
      for o in ("bf16", "f32")),
    ("q6_k", "wave32x2_fixed_meta_gemv_decode_bf16_bf16_out"),
    ("q6_k", "gemv_dpp_wave_reduction_coltile4_rowbatch8_bf16_bf16_out"),
    ("q6_k", "gemv_dpp_wave_reduction_coltile2_rowbatch16_bf16_f32_out"),
    ("q6_k", "gemv_dpp_wave_reduction_full_group_compute_coltile4_rowbatch8_bf16_bf16_out"),
    ("q6_k", "gemv_dpp_wave_reduction_full_group_compute_coltile2_rowbatch16_bf16_f32_out"),
    ("q8_0", "gemv_coltile4_rowbatch8_pipelined_f32_f32_out"),
    ("q8_0", "gemv_coltile8_rowbatch4_pipelined_f32_f32_out"),
    ("q8_0", "gemv_coltile8_rowbatch4_wave_scale_f32_f32_out"),
    ("q8_0", "gemv_coltile8_rowbatch4_wave_scale_pipelined_f32_f32_out"),
    ("q8_0", "gemv_coltile8_rowbatch4_wave_scale_pipelined_dpp_f32_f32_out"),
    ("q8_0", "gemv_coltile8_rowbatch4_wave_scale_pipelined_dpp_checked_full_rows_f32_f32_out"),
)


def _make_dense_variant(quant: str, variant: str):
    symbol = f"hipengine_gguf_{quant}_{variant}"

    def wrapper(x_ptr: int, qweight_ptr: int, out_ptr: int, rows: int, in_features: int, out_features: int, *,
                threads: int = 128, stream: int = 0, library: ctypes.CDLL | None = None,
                runtime: HipRuntime | None = None) -> None:
        validate_linear(rows, in_features, out_features, threads)
        validate_pointers(x_ptr=x_ptr, qweight_ptr=qweight_ptr, out_ptr=out_ptr)
        check_launch(entry(symbol, _FUSED_ARGS, library)(x_ptr, qweight_ptr, out_ptr, rows, in_features, out_features,
                                                         threads, stream), runtime)

    wrapper.__name__ = f"gguf_{quant}_{variant}"
    wrapper.__doc__ = f"hipEngine's tuning variant ``{symbol}``: the dense GEMV launch (any shape)."
    return wrapper


DENSE_VARIANTS = {(q, v): _make_dense_variant(q, v) for q, v in _DENSE_VARIANT_NAMES}
_PAIR_ARGS = [VOID, VOID, VOID, VOID, VOID, I64, I64, I64, I64, I64, VOID]


def _make_q5_k_pair(variant: str):
    symbol = f"hipengine_gguf_q5_k_{variant}"

    def wrapper(x_ptr: int, qweight_a_ptr: int, qweight_b_ptr: int, out_a_ptr: int, out_b_ptr: int, rows: int,
                in_features: int, out_features_a: int, out_features_b: int, *, threads: int = 128, stream: int = 0,
                library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
        validate_linear(rows, in_features, out_features_a, threads)
        validate_linear(rows, in_features, out_features_b, threads)
        validate_pointers(x_ptr=x_ptr, qweight_a_ptr=qweight_a_ptr, qweight_b_ptr=qweight_b_ptr, out_a_ptr=out_a_ptr,
                          out_b_ptr=out_b_ptr)
        check_launch(entry(symbol, _PAIR_ARGS, library)(x_ptr, qweight_a_ptr, qweight_b_ptr, out_a_ptr, out_b_ptr, rows,
                                                        in_features, out_features_a, out_features_b, threads, stream),
                     runtime)

    wrapper.__name__ = f"gguf_q5_k_{variant}"
    wrapper.__doc__ = (f"hipEngine's Q5_K pair decode ``{symbol}``: two matrices of different heights over one bf16 "
                       "activation, one multi-matrix launch.")
    return wrapper


Q5_K_PAIR = {v: _make_q5_k_pair(v) for v in (
    "pair_wave32x2_gemv_decode_bf16_f32_out", "pair_wave32x2_fixed_meta_gemv_decode_bf16_bf16_out",
    "pair_wave32x2_fixed_meta_gemv_decode_bf16_f32_out", "pair_wave32x2_swar_pair_fixed_meta_gemv_decode_bf16_bf16_out",
    "pair_wave32x2_swar_pair_fixed_meta_gemv_decode_bf16_f32_out")}


def register_kernels(backend: str = "hip_gfx950", *, replace: bool = False) -> None:
    # the keys hipEngine's dispatcher resolves for raw-layout weights: gemv_* at one row, prefill_* above
    # (loading/qwen35_gguf_consumer_surface.py:134-144,527-530)
    for (quant, family, act, out), fn in DENSE.items():
        variant = family[len("gemv_"):] if family == "gemv_rowtile" else family     # "rowtile_<act>_<out>_out"
        register(KernelKey(backend, "linear", f"gguf_{quant}", f"{variant}_{act}_{out}_out"), fn, replace=replace)
    for (quant, act, out), fn in DENSE_DUAL.items():
        register(KernelKey(backend, "linear", f"gguf_{quant}", f"dual_gemv_{act}_{out}_out"), fn, replace=replace)
    for (act, out), fn in PAIR_SILU.items():
        register(KernelKey(backend, "linear", "gguf_q4_k", f"dual_silu_gemv_{act}_{out}_out"), fn, replace=replace)
    register(KernelKey(backend, "linear", "gguf", "multi_gemv"), gguf_multi_gemv, replace=replace)
    for (quant, variant), fn in DENSE_VARIANTS.items():
        register(KernelKey(backend, "linear", f"gguf_{quant}", variant), fn, replace=replace)
    for variant, fn in Q5_K_PAIR.items():
        register(KernelKey(backend, "linear", "gguf_q5_k", variant), fn, replace=replace)
    for (quant, act, out), fn in RESIDUAL.items():
        register(KernelKey(backend, "linear", f"gguf_{quant}", f"gemv_{act}_residual_{out}_out"), fn, replace=replace)
    for (quant, act, out), fn in FUSED.items():
        for prefix in ("q8_1_fused_gemv", "q8_1_fused_prefill"):
            register(KernelKey(backend, "linear", f"gguf_{quant}", f"{prefix}_{act}_{out}_out"), fn, replace=replace)
    for quant, variant, fn in (
        ("gguf_q4_k", "q8_1_dp4a_vdr_bf16_f32_out", gguf_q4_k_q8_1_dp4a_vdr_bf16_f32_out),
        ("gguf_q4_k", "q8_1_dp4a_vdr_bf16_bf16_out", gguf_q4_k_q8_1_dp4a_vdr_bf16_bf16_out),
        ("gguf_q6_k", "q8_1_dp4a_gemv_bf16_f32_out", gguf_q6_k_q8_1_dp4a_gemv_bf16_f32_out),
        ("gguf_q6_k", "q8_1_dp4a_gemv_bf16_bf16_out", gguf_q6_k_q8_1_dp4a_gemv_bf16_bf16_out),
        ("gguf_q4_k", "q8_1_dp4a_ctl_bf16_f32_out", gguf_q4_k_q8_1_dp4a_ctl_bf16_f32_out),
        ("gguf_q4_k", "q8_1_dp4a_ctl_bf16_bf16_out", gguf_q4_k_q8_1_dp4a_ctl_bf16_bf16_out),
        *(("gguf_q8_0", variant, fn) for variant, fn in Q8_0_DP4A.items()),
    ):
        register(KernelKey(backend, "linear", quant, variant), fn, replace=replace)
