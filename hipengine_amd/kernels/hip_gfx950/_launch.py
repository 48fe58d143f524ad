"""Shared plumbing of the gfx950 raw-pointer wrappers: library lookup, typed
entry points configured once per symbol, and launch-status checking.

hipEngine measured ~88 us per launch when ``argtypes`` were set on every call
against ~1.4 us with them cached (``kernels/hip_gfx1100/quant/gguf_k_gemv.py:15-32``);
entry points are therefore configured once and kept in a dict.
"""

from __future__ import annotations

import ctypes

from hipengine_amd.core.build import load_library
from hipengine_amd.core.hip import HIP_SUCCESS, HipError, HipRuntime, get_hip_runtime

VOID = ctypes.c_void_p
I64 = ctypes.c_int64
I32 = ctypes.c_int32

ALLOWED_THREADS = frozenset({64, 128, 256})
KIND_F32, KIND_BF16, KIND_F16, KIND_Q8_1 = 0, 1, 2, 3
GGML_Q8_0, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K = 8, 12, 13, 14
# the four block types every kernel family here takes (decode GEMV, MMQ prefill, MoE, dequantization, embedding)
QUANT_KEY_TO_GGML = {"gguf_q8_0": GGML_Q8_0, "gguf_q4_k": GGML_Q4_K, "gguf_q5_k": GGML_Q5_K, "gguf_q6_k": GGML_Q6_K}

_entry_cache: dict[tuple[int, str], ctypes._CFuncPtr] = {}


def entry(symbol: str, argtypes: list, library: ctypes.CDLL | None = None):
    """The C function ``symbol`` with ``argtypes`` set, resolved once per library."""
    lib = library if library is not None else load_library()
    key = (id(lib), symbol)
    fn = _entry_cache.get(key)
    if fn is None:
        fn = getattr(lib, symbol)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
        _entry_cache[key] = fn
    return fn


# Argument validation in the Python wrappers (range and null-pointer checks that raise ValueError, as hipEngine's
# wrappers do).  A caller that has validated its shapes once and launches in a loop may switch it off: the C
# entry points check their arguments as well and return hipErrorInvalidValue.
VALIDATE = True


def set_validation(enabled: bool) -> None:
    global VALIDATE
    VALIDATE = bool(enabled)


def lean_entry(symbol: str, argtypes: list, library: ctypes.CDLL | None = None):
    """The configured C function itself (``argtypes`` set once, hipEngine's ``_cached_fn``:
    ``kernels/hip_gfx1100/quant/gguf_k_gemv.py:15-32``): called positionally with the C signature, it costs
    one ctypes call; the caller tests the returned ``hipError_t`` (0 is success)."""
    return entry(symbol, argtypes, library)


def check_launch(code: int, runtime: HipRuntime | None) -> None:
    if int(code) == HIP_SUCCESS:
        return
    if runtime is None:
        try:
            runtime = get_hip_runtime()
        except OSError:
            raise HipError(int(code), f"hipError {int(code)}") from None
    runtime.check(int(code))


def validate_linear(rows: int, in_features: int, out_features: int, threads: int = 128, *, block: int = 256) -> None:
    """Argument checks shared by the dense wrappers
    (hipEngine: ``gguf_q4_k_gemv.py:909-930``, ``gguf_k_gemv.py:1640-1662``)."""
    if rows <= 0:
        raise ValueError("rows must be positive")
    if in_features <= 0:
        raise ValueError("in_features must be positive")
    if out_features <= 0:
        raise ValueError("out_features must be positive")
    if in_features % block != 0:
        raise ValueError(f"in_features must be divisible by the GGUF block size {block}")
    if threads not in ALLOWED_THREADS:
        allowed = ", ".join(str(v) for v in sorted(ALLOWED_THREADS))
        raise ValueError(f"threads must be one of {allowed}")


def validate_pointers(**ptrs: int) -> None:
    for name, value in ptrs.items():
        if not isinstance(value, int) or value <= 0:
            raise ValueError(f"{name} must be a non-null device pointer")
