"""Row-wise arg-max of lm_head logits (greedy decode).

Signature, checks and registry key follow hipEngine's ``kernels/hip_gfx1100/linear/lm_head.py``
(``argmax_f32_rows_i32`` :329-377, ``_check_shape`` / ``_check_rows`` / ``_check_i32_vocab`` :612-628,
key ``("argmax", "w4_paro", "f32_rows_i32")`` :596-599; registered here under the quant-neutral
``("argmax", "f32", "rows_i32")`` as well).  The lm_head projection itself is the Q6_K / Q4_K GEMV.
"""

from __future__ import annotations

import ctypes

from hipengine_amd.core.hip import HipRuntime
from hipengine_amd.kernels.hip_gfx950._launch import I64, VOID, check_launch, entry, validate_pointers
from hipengine_amd.kernels.registry import KernelKey, register

_ALLOWED_THREADS = {128, 256, 512}


def argmax_scratch_entries(rows: int, vocab_size: int, threads: int = 256) -> int:
    """Entries of each scratch array (float32 values, int32 indices) a call needs."""
    return rows * ((vocab_size + threads * 4 - 1) // (threads * 4))


def argmax_f32_rows_i32(logits_f32_ptr: int, block_values_f32_ptr: int, block_indices_i32_ptr: int,
                        out_indices_i32_ptr: int, out_values_f32_ptr: int | None, rows: int, vocab_size: int, *,
                        threads: int = 256, stream: int = 0, library: ctypes.CDLL | None = None,
                        runtime: HipRuntime | None = None) -> None:
    """Write row-wise top-1 ids for ``logits[rows, vocab_size]`` without host logits."""
    if rows <= 0:
        raise ValueError("rows must be positive")
    if vocab_size <= 0:
        raise ValueError("vocab_size must be positive")
    if threads not in _ALLOWED_THREADS:
        raise ValueError("threads must be one of 128, 256, or 512")
    if vocab_size > 2**31 - 1:
        raise ValueError("vocab_size must fit int32 row-wise argmax outputs")
    validate_pointers(logits_f32_ptr=logits_f32_ptr, block_values_f32_ptr=block_values_f32_ptr,
                      block_indices_i32_ptr=block_indices_i32_ptr, out_indices_i32_ptr=out_indices_i32_ptr)
    fn = entry("hipengine_argmax_f32_rows_i32", [VOID, VOID, VOID, VOID, VOID, I64, I64, I64, VOID], library)
    check_launch(fn(logits_f32_ptr, block_values_f32_ptr, block_indices_i32_ptr, out_indices_i32_ptr,
                    out_values_f32_ptr or None, rows, vocab_size, threads, stream), runtime)


NOALLOC_MAX_ENTRIES = 65536   # HIPENGINE_GFX950_ARGMAX_NOALLOC_MAX_ENTRIES


def argmax_f32_rows_i32_noalloc(logits_f32_ptr: int, out_indices_i32_ptr: int, out_values_f32_ptr: int | None, rows: int,
                                vocab_size: int, *, threads: int = 256, stream: int = 0,
                                library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """``argmax_f32_rows_i32`` on scratch the library holds itself, for callers that cannot allocate
    (no counterpart in hipEngine).  ``rows * ceil(vocab_size / (threads * 4))`` may not exceed
    ``NOALLOC_MAX_ENTRIES``; calls that overlap on one device share the scratch and race."""
    if rows <= 0:
        raise ValueError("rows must be positive")
    if vocab_size <= 0:
        raise ValueError("vocab_size must be positive")
    if threads not in _ALLOWED_THREADS:
        raise ValueError("threads must be one of 128, 256, or 512")
    if vocab_size > 2**31 - 1:
        raise ValueError("vocab_size must fit int32 row-wise argmax outputs")
    if argmax_scratch_entries(rows, vocab_size, threads) > NOALLOC_MAX_ENTRIES:
        raise ValueError(f"rows * ceil(vocab_size / (threads * 4)) exceeds the library's scratch of {NOALLOC_MAX_ENTRIES} entries")
    validate_pointers(logits_f32_ptr=logits_f32_ptr, out_indices_i32_ptr=out_indices_i32_ptr)
    fn = entry("hipengine_gfx950_argmax_f32_rows_i32_noalloc", [VOID, VOID, VOID, I64, I64, I64, VOID], library)
    check_launch(fn(logits_f32_ptr, out_indices_i32_ptr, out_values_f32_ptr or None, rows, vocab_size, threads, stream),
                 runtime)


def register_kernels(backend: str = "hip_gfx950", *, replace: bool = False) -> None:
    register(KernelKey(backend, "argmax", "f32", "rows_i32"), argmax_f32_rows_i32, replace=replace)
    register(KernelKey(backend, "argmax", "w4_paro", "f32_rows_i32"), argmax_f32_rows_i32, replace=replace)
    register(KernelKey(backend, "argmax", "f32", "rows_i32_noalloc"), argmax_f32_rows_i32_noalloc, replace=replace)
