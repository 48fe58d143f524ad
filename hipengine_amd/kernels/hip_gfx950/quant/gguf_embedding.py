"""Token embedding lookup over raw GGUF rows (Q4_K, Q5_K, Q6_K, Q8_0) into bf16.

Signatures, checks and registry keys follow hipEngine's
``kernels/hip_gfx1100/quant/gguf_q6_k_embedding.py`` (wrappers :55-177, ``_validate`` :246-258,
keys ``("embedding", "gguf_q4_k", "lookup_bf16_out")`` ... :223-243).  Raw device pointers:
int64 token ids, uint8 block rows, bf16 bits out.
"""

from __future__ import annotations

import ctypes

from hipengine_amd.core.hip import HipRuntime
from hipengine_amd.kernels.hip_gfx950._launch import I64, VOID, check_launch, entry, validate_pointers
from hipengine_amd.kernels.registry import KernelKey, register

_ALLOWED_THREADS = frozenset({64, 128, 256, 512, 1024})
_ARGS = [VOID, VOID, VOID, I64, I64, I64, I64, VOID]


def _validate(quant: str, rows: int, hidden_size: int, vocab_size: int, threads: int) -> None:
    if rows <= 0:
        raise ValueError("rows must be positive")
    block_size = 32 if quant == "gguf_q8_0" else 256
    if hidden_size <= 0 or hidden_size % block_size != 0:
        raise ValueError(f"hidden_size must be positive and divisible by GGUF {quant} block size {block_size}")
    if vocab_size <= 0:
        raise ValueError("vocab_size must be positive")
    if threads not in _ALLOWED_THREADS:
        allowed = ", ".join(str(value) for value in sorted(_ALLOWED_THREADS))
        raise ValueError(f"threads must be one of {allowed}")


def _make(quant: str):
    symbol = f"hipengine_{quant}_embedding_bf16_out"

    def wrapper(token_ids_ptr: int, qweight_ptr: int, out_ptr: int, rows: int, hidden_size: int, vocab_size: int, *,
                threads: int = 256, stream: int = 0, library: ctypes.CDLL | None = None,
                runtime: HipRuntime | None = None) -> None:
        _validate(quant, rows, hidden_size, vocab_size, threads)
        validate_pointers(token_ids_ptr=token_ids_ptr, qweight_ptr=qweight_ptr, out_ptr=out_ptr)
        check_launch(entry(symbol, _ARGS, library)(token_ids_ptr, qweight_ptr, out_ptr, rows, hidden_size, vocab_size,
                                                   threads, stream), runtime)

    wrapper.__name__ = f"{quant}_embedding_bf16_out"
    wrapper.__doc__ = f"GGUF {quant[5:].upper()} embedding lookup into bf16 bits (C symbol ``{symbol}``)."
    return wrapper


gguf_q4_k_embedding_bf16_out = _make("gguf_q4_k")
gguf_q5_k_embedding_bf16_out = _make("gguf_q5_k")
gguf_q6_k_embedding_bf16_out = _make("gguf_q6_k")
gguf_q8_0_embedding_bf16_out = _make("gguf_q8_0")

EMBEDDING = {"gguf_q4_k": gguf_q4_k_embedding_bf16_out, "gguf_q5_k": gguf_q5_k_embedding_bf16_out,
             "gguf_q6_k": gguf_q6_k_embedding_bf16_out, "gguf_q8_0": gguf_q8_0_embedding_bf16_out}


def register_kernels(backend: str = "hip_gfx950", *, replace: bool = False) -> None:
    for quant, fn in EMBEDDING.items():
        register(KernelKey(backend, "embedding", quant, "lookup_bf16_out"), fn, replace=replace)
