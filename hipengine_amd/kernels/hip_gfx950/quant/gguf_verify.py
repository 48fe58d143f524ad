"""Verification exports: device-side block dequantization and the int32
sub-block dots of the q8_1 kernels, for bit-exact comparison with a CPU oracle."""

from __future__ import annotations

import ctypes

from hipengine_amd.core.hip import HipRuntime
from hipengine_amd.kernels.hip_gfx950._launch import (
    I32,
    I64,
    QUANT_KEY_TO_GGML,
    VOID,
    check_launch,
    entry,
    validate_pointers,
)


def gguf_dequantize_f32(quant_key: str, blocks_ptr: int, out_ptr: int, n_blocks: int, *, stream: int = 0,
                        library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """``n_blocks`` raw blocks -> float32 (256 values per Q4_K/Q6_K block, 32 per Q8_0 block)."""
    if n_blocks <= 0:
        raise ValueError("n_blocks must be positive")
    validate_pointers(blocks_ptr=blocks_ptr, out_ptr=out_ptr)
    fn = entry("hipengine_gfx950_gguf_dequantize_f32", [I32, VOID, VOID, I64, VOID], library)
    check_launch(fn(QUANT_KEY_TO_GGML[quant_key], blocks_ptr, out_ptr, n_blocks, stream), runtime)


def gguf_q8_1_block_dots_i32(quant_key: str, xq_ptr: int, qweight_ptr: int, dots_ptr: int, qsums_ptr: int, rows: int,
                             in_features: int, out_features: int, *, stream: int = 0,
                             library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """int32 sub-block dots ``[rows, out_features, K/32]`` (Q6_K: ``K/16``) and, when
    ``qsums_ptr`` is non-zero, the int32 q8 sums ``[rows, K/32]``."""
    if rows <= 0 or out_features <= 0 or in_features <= 0 or in_features % 256:
        raise ValueError("rows/out_features must be positive and in_features divisible by 256")
    validate_pointers(xq_ptr=xq_ptr, qweight_ptr=qweight_ptr, dots_ptr=dots_ptr)
    fn = entry("hipengine_gfx950_gguf_q8_1_block_dots_i32", [I32, VOID, VOID, VOID, VOID, I64, I64, I64, VOID], library)
    check_launch(fn(QUANT_KEY_TO_GGML[quant_key], xq_ptr, qweight_ptr, dots_ptr, qsums_ptr or None, rows, in_features,
                    out_features, stream), runtime)


FORM_SLAB, FORM_PSLAB, FORM_DSLAB = 3, 4, 5


def gguf_gemv_mfma_dots_i32(quant_key: str, form: int, xq_ptr: int, qweight_ptr: int, dots_ptr: int, out_ptr: int,
                            rows: int, in_features: int, out_features: int, *, stream: int = 0,
                            library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """The int32 sub-block dots of the decode GEMV's MFMA forms (``FORM_SLAB``: Q4_K; ``FORM_PSLAB``: all four
    types), written by the production kernel body: ``[rows, out_features, K/32]`` (Q6_K ``K/16``), and the
    kernel's float32 result ``[rows, out_features]``.  ``xq``: 36-byte q8_1 blocks, ``rows <= 8``."""
    if rows <= 0 or rows > 8 or out_features <= 0 or in_features <= 0 or in_features % 256:
        raise ValueError("rows must be in 1..8, out_features positive and in_features divisible by 256")
    if form not in (FORM_SLAB, FORM_PSLAB, FORM_DSLAB):
        raise ValueError("form must be FORM_SLAB, FORM_PSLAB or FORM_DSLAB")
    validate_pointers(xq_ptr=xq_ptr, qweight_ptr=qweight_ptr, dots_ptr=dots_ptr, out_ptr=out_ptr)
    fn = entry("hipengine_gfx950_gguf_gemv_mfma_dots_i32", [I32, I32, VOID, VOID, VOID, VOID, I64, I64, I64, VOID], library)
    check_launch(fn(QUANT_KEY_TO_GGML[quant_key], form, xq_ptr, qweight_ptr, dots_ptr, out_ptr, rows, in_features,
                    out_features, stream), runtime)


def gguf_mmq_dots_i32(quant_key: str, xq_ptr: int, qweight_ptr: int, dots_ptr: int, out_ptr: int, rows: int,
                      in_features: int, out_features: int, *, stream: int = 0, library: ctypes.CDLL | None = None,
                      runtime: HipRuntime | None = None) -> None:
    """The int32 dots of the MMQ prefill GEMM (Q4_K over DS4 blocks, Q5_K and Q8_0 over D4S4 blocks:
    ``[rows, N, K/32]``; Q6_K over D4S4 blocks: ``[rows, N, K/16]``, centred values) and its float32 result, from
    the production tile engine."""
    if quant_key not in ("gguf_q4_k", "gguf_q5_k", "gguf_q6_k", "gguf_q8_0"):
        raise ValueError("the MMQ takes gguf_q4_k, gguf_q5_k, gguf_q6_k or gguf_q8_0 weights")
    block = 128 if quant_key == "gguf_q8_0" else 256
    if rows <= 0 or out_features <= 0 or in_features <= 0 or in_features % block:
        raise ValueError(f"rows/out_features must be positive and in_features divisible by {block}")
    validate_pointers(xq_ptr=xq_ptr, qweight_ptr=qweight_ptr, dots_ptr=dots_ptr, out_ptr=out_ptr)
    fn = entry("hipengine_gfx950_gguf_mmq_dots_i32", [I32, VOID, VOID, VOID, VOID, I64, I64, I64, VOID], library)
    check_launch(fn(QUANT_KEY_TO_GGML[quant_key], xq_ptr, qweight_ptr, dots_ptr, out_ptr, rows, in_features,
                    out_features, stream), runtime)


def read_probe(src_ptr: int, nbytes: int, *, waves_per_workgroup: int = 8, loads_in_flight: int = 4, sink_ptr: int = 0,
               stream: int = 0, library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """Read-only pass over a device buffer with the streaming GEMV's load shape (the ceiling a launch that only
    reads reaches; C symbol ``hipengine_gfx950_read_probe``)."""
    if nbytes < 1024:
        raise ValueError("nbytes must be at least 1024")
    validate_pointers(src_ptr=src_ptr)
    fn = entry("hipengine_gfx950_read_probe", [VOID, I64, I32, I32, VOID, VOID], library)
    check_launch(fn(src_ptr, nbytes, waves_per_workgroup, loads_in_flight, sink_ptr or None, stream), runtime)


def read_probe_grid(src_ptr: int, nbytes: int, workgroups: int, *, waves_per_workgroup: int = 4, loads_in_flight: int = 1,
                    sink_ptr: int = 0, stream: int = 0, library: ctypes.CDLL | None = None,
                    runtime: HipRuntime | None = None) -> None:
    """The read-only pass over ``workgroups`` workgroups instead of one per CU (thousands of them: waves that read a
    piece or two and leave; C symbol ``hipengine_gfx950_read_probe_grid``)."""
    if nbytes < 1024 or workgroups < 1:
        raise ValueError("nbytes must be at least 1024 and workgroups positive")
    validate_pointers(src_ptr=src_ptr)
    fn = entry("hipengine_gfx950_read_probe_grid", [VOID, I64, I32, I32, I32, VOID, VOID], library)
    check_launch(fn(src_ptr, nbytes, waves_per_workgroup, loads_in_flight, workgroups, sink_ptr or None, stream), runtime)


def copy_bytes(src_ptr: int, dst_ptr: int, nbytes: int, *, stream: int = 0, library: ctypes.CDLL | None = None,
               runtime: HipRuntime | None = None) -> None:
    """Plain device copy kernel of a known size (calibration of HBM byte counters)."""
    if nbytes <= 0 or nbytes % 16:
        raise ValueError("nbytes must be a positive multiple of 16")
    validate_pointers(src_ptr=src_ptr, dst_ptr=dst_ptr)
    fn = entry("hipengine_gfx950_copy_bytes", [VOID, VOID, I64, VOID], library)
    check_launch(fn(src_ptr, dst_ptr, nbytes, stream), runtime)
