"""ctypes view of ``libgguf_oracle.so`` (the C restatement).  TEST INFRASTRUCTURE ONLY.

``build()`` compiles ``gguf_oracle.c`` with the Makefile next to it; ``load()``
opens the result and declares argument types.  The wrappers take and return
NumPy arrays.
"""

from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "libgguf_oracle.so"
_lib: ctypes.CDLL | None = None

_VP = ctypes.c_void_p
_I64 = ctypes.c_int64
_I32 = ctypes.c_int

_SIGNATURES = {
    "oracle_f16_to_f32": ([ctypes.c_uint16], ctypes.c_float),
    "oracle_f32_to_f16": ([ctypes.c_float], ctypes.c_uint16),
    "oracle_f32_to_bf16": ([ctypes.c_float], ctypes.c_uint16),
    "oracle_q4_k_scale_min": ([_VP, _I64, _VP, _VP], None),
    "oracle_q4_k_unpack_int": ([_VP, _I64, _VP], None),
    "oracle_q6_k_unpack_int": ([_VP, _I64, _VP], None),
    "oracle_dequant_q4_k": ([_VP, _I64, _VP], None),
    "oracle_dequant_q6_k": ([_VP, _I64, _VP], None),
    "oracle_dequant_q8_0": ([_VP, _I64, _VP], None),
    "oracle_gemv_dequant": ([_VP, _VP, _I32, _VP, _I64, _I64, _I64], _I32),
    "oracle_quantize_q8_1_f32": ([_VP, _VP, _I64, _I64], None),
    "oracle_quantize_q8_1_bf16": ([_VP, _VP, _I64, _I64], None),
    "oracle_pack_ds4_bf16": ([_VP, _VP, _I64, _I64], None),
    "oracle_pack_d4s4_bf16": ([_VP, _VP, _I64, _I64], None),
    "oracle_q4_k_q8_1_block_dots": ([_VP, _VP, _VP, _VP, _I64, _I64, _I64], None),
    "oracle_q6_k_q8_1_block_dots": ([_VP, _VP, _VP, _I64, _I64, _I64], None),
    "oracle_q8_0_q8_1_block_dots": ([_VP, _VP, _VP, _I64, _I64, _I64], None),
    "oracle_q4_k_q8_1_gemv": ([_VP, _VP, _VP, _I64, _I64, _I64], None),
    "oracle_q6_k_q8_1_gemv": ([_VP, _VP, _VP, _I64, _I64, _I64], None),
    "oracle_q8_0_q8_1_gemv": ([_VP, _VP, _VP, _I64, _I64, _I64], None),
    "oracle_q4_k_ds4_mmq": ([_VP, _VP, _VP, _I64, _I64, _I64], None),
    "oracle_q6_k_d4s4_mmq": ([_VP, _VP, _VP, _I64, _I64, _I64], None),
    "oracle_num_threads": ([], _I32),
}

_TYPE_BYTES = {8: (32, 34), 12: (256, 144), 14: (256, 210)}


def build(force: bool = False) -> Path:
    src = _HERE / "gguf_oracle.c"
    if force or not _LIB_PATH.exists() or _LIB_PATH.stat().st_mtime < src.stat().st_mtime:
        subprocess.run(["make", "-C", str(_HERE), "-B", "libgguf_oracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            build()
        lib = ctypes.CDLL(str(_LIB_PATH))
        for name, (argtypes, restype) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = lib
    return _lib


def _p(a: np.ndarray) -> int:
    return a.ctypes.data


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(a).view(np.uint8)


def dequantize(qweight, qtype: int) -> np.ndarray:
    block, nbytes = _TYPE_BYTES[int(qtype)]
    raw = _u8(qweight)
    n_blocks = raw.size // nbytes
    out = np.empty(n_blocks * block, dtype=np.float32)
    name = {8: "oracle_dequant_q8_0", 12: "oracle_dequant_q4_k", 14: "oracle_dequant_q6_k"}[int(qtype)]
    getattr(load(), name)(_p(raw), n_blocks, _p(out))
    return out.reshape(*raw.shape[:-1], raw.shape[-1] // nbytes * block)


def q4_k_scale_min(scale_bytes) -> tuple[np.ndarray, np.ndarray]:
    raw = _u8(scale_bytes).reshape(-1, 12)
    sc = np.empty((raw.shape[0], 8), dtype=np.uint8)
    mn = np.empty_like(sc)
    load().oracle_q4_k_scale_min(_p(raw), raw.shape[0], _p(sc), _p(mn))
    return sc, mn


def unpack_int(qweight, qtype: int) -> np.ndarray:
    raw = _u8(qweight)
    if int(qtype) == 12:
        n = raw.size // 144
        out = np.empty(n * 256, dtype=np.uint8)
        load().oracle_q4_k_unpack_int(_p(raw), n, _p(out))
    else:
        n = raw.size // 210
        out = np.empty(n * 256, dtype=np.int8)
        load().oracle_q6_k_unpack_int(_p(raw), n, _p(out))
    return out.reshape(n, 256)


def gemv_dequant(x, qweight, qtype: int) -> np.ndarray:
    xa = np.ascontiguousarray(x, dtype=np.float32)
    raw = _u8(qweight)
    block, nbytes = _TYPE_BYTES[int(qtype)]
    rows, k = xa.shape
    n = raw.shape[0]
    assert raw.shape[1] == k // block * nbytes
    out = np.empty((rows, n), dtype=np.float32)
    rc = load().oracle_gemv_dequant(_p(xa), _p(raw), int(qtype), _p(out), rows, k, n)
    if rc:
        raise MemoryError("oracle_gemv_dequant")
    return out


def quantize_q8_1(x, bf16: bool = False) -> np.ndarray:
    xa = np.ascontiguousarray(x, dtype=np.uint16 if bf16 else np.float32)
    rows, k = xa.shape
    out = np.empty((rows, k // 32, 36), dtype=np.uint8)
    fn = load().oracle_quantize_q8_1_bf16 if bf16 else load().oracle_quantize_q8_1_f32
    fn(_p(xa), _p(out), rows, k)
    return out


def pack_ds4(x_bf16) -> np.ndarray:
    xa = np.ascontiguousarray(x_bf16, dtype=np.uint16)
    rows, k = xa.shape
    out = np.empty((rows, k // 128, 144), dtype=np.uint8)
    load().oracle_pack_ds4_bf16(_p(xa), _p(out), rows, k)
    return out


def pack_d4s4(x_bf16) -> np.ndarray:
    xa = np.ascontiguousarray(x_bf16, dtype=np.uint16)
    rows, k = xa.shape
    out = np.empty((rows, k // 128, 160), dtype=np.uint8)
    load().oracle_pack_d4s4_bf16(_p(xa), _p(out), rows, k)
    return out


def block_dots(xq, qweight, qtype: int):
    """int32 sub-block dots ``[rows, N, K/32]`` (Q6_K: ``K/16``); Q4_K also
    returns the int32 q8 sums ``[rows, K/32]``."""
    xa = _u8(xq)
    raw = _u8(qweight)
    rows = xa.shape[0]
    k = xa.reshape(rows, -1).shape[1] // 36 * 32
    n = raw.shape[0]
    lib = load()
    if int(qtype) == 12:
        dots = np.empty((rows, n, k // 32), dtype=np.int32)
        qsum = np.empty((rows, k // 32), dtype=np.int32)
        lib.oracle_q4_k_q8_1_block_dots(_p(xa), _p(raw), _p(dots), _p(qsum), rows, k, n)
        return dots, qsum
    if int(qtype) == 14:
        dots = np.empty((rows, n, k // 16), dtype=np.int32)
        lib.oracle_q6_k_q8_1_block_dots(_p(xa), _p(raw), _p(dots), rows, k, n)
        return dots
    dots = np.empty((rows, n, k // 32), dtype=np.int32)
    lib.oracle_q8_0_q8_1_block_dots(_p(xa), _p(raw), _p(dots), rows, k, n)
    return dots


def gemv_q8_1(xq, qweight, qtype: int) -> np.ndarray:
    xa = _u8(xq)
    raw = _u8(qweight)
    rows = xa.shape[0]
    k = xa.reshape(rows, -1).shape[1] // 36 * 32
    n = raw.shape[0]
    out = np.empty((rows, n), dtype=np.float32)
    name = {8: "oracle_q8_0_q8_1_gemv", 12: "oracle_q4_k_q8_1_gemv", 14: "oracle_q6_k_q8_1_gemv"}[int(qtype)]
    getattr(load(), name)(_p(xa), _p(raw), _p(out), rows, k, n)
    return out


def mmq_q4_k_ds4(xds4, qweight) -> np.ndarray:
    xa = _u8(xds4)
    raw = _u8(qweight)
    rows = xa.shape[0]
    k = xa.reshape(rows, -1).shape[1] // 144 * 128
    n = raw.shape[0]
    out = np.empty((rows, n), dtype=np.float32)
    load().oracle_q4_k_ds4_mmq(_p(xa), _p(raw), _p(out), rows, k, n)
    return out


def mmq_q6_k_d4s4(xq, qweight) -> np.ndarray:
    xa = _u8(xq)
    raw = _u8(qweight)
    rows = xa.shape[0]
    k = xa.reshape(rows, -1).shape[1] // 160 * 128
    n = raw.shape[0]
    out = np.empty((rows, n), dtype=np.float32)
    load().oracle_q6_k_d4s4_mmq(_p(xa), _p(raw), _p(out), rows, k, n)
    return out


def num_threads() -> int:
    return int(load().oracle_num_threads())
