"""Writes tests/golden/tiny_v3.gguf: the GGUF v3 container that hipEngine's reader test describes
(tests/test_unit_gguf_reader.py:54-110: three tensors -- F32 2x3, BF16 [2], one Q8_0 block -- and six metadata
entries, alignment 32), packed field by field from the published container layout with `struct` alone, so the
file does not depend on this package's own writer.

    python tests/golden/make_tiny_gguf.py
"""

from __future__ import annotations

import struct
from pathlib import Path

import numpy as np

# GGUF metadata value types and ggml tensor types (ggml's public numbering)
U32, F32V, STR, ARR = 4, 6, 8, 9
T_F32, T_Q8_0, T_BF16 = 0, 8, 30
ALIGN = 32


def s(text: str) -> bytes:
    raw = text.encode()
    return struct.pack("<Q", len(raw)) + raw


def pad(n: int) -> int:
    return -n % ALIGN


def main() -> None:
    payloads = [
        ("dense.weight", (3, 2), T_F32, np.arange(6, dtype="<f4").tobytes()),                       # ggml order: fastest first
        ("bf16.weight", (2,), T_BF16, np.array([0x3F80, 0xC020], dtype="<u2").tobytes()),           # 1.0, -2.5
        ("q8.weight", (32, 1), T_Q8_0, np.array([2.0], dtype="<f2").tobytes() + np.arange(-16, 16, dtype=np.int8).tobytes()),
    ]
    kv = b"".join([
        s("general.architecture") + struct.pack("<I", STR) + s("toy"),
        s("general.alignment") + struct.pack("<II", U32, ALIGN),
        s("general.file_type") + struct.pack("<II", U32, 7),
        s("toy.context_length") + struct.pack("<II", U32, 16),
        s("tokenizer.ggml.tokens") + struct.pack("<IIQ", ARR, STR, 2) + s("a") + s("b"),
        s("tokenizer.ggml.scores") + struct.pack("<IIQ", ARR, F32V, 2) + struct.pack("<ff", 0.25, -0.5),
    ])
    table, blob = b"", b""
    for name, dims, kind, data in payloads:
        blob += b"\0" * pad(len(blob))
        table += s(name) + struct.pack("<I", len(dims)) + struct.pack(f"<{len(dims)}Q", *dims) + struct.pack("<IQ", kind, len(blob))
        blob += data
    head = b"GGUF" + struct.pack("<IQQ", 3, len(payloads), 6) + kv + table
    out = Path(__file__).with_name("tiny_v3.gguf")
    out.write_bytes(head + b"\0" * pad(len(head)) + blob)
    print(out, out.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
