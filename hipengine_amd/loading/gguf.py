"""GGUF (v2 / v3) container intake: header, metadata and tensor table from a read-only memory map,
lazy NumPy views of tensor payloads in the raw block layout, and their upload to device memory.

Public names, fields and error behaviour follow hipEngine's ``hipengine/loading/gguf.py``
(``GGUFTensorInfo`` :56-73, ``GGUFModelInfo`` :76-131, ``GGUFReader`` :134-170, ``scan_gguf`` :185-268):
``shape`` is the row-major logical shape (the reverse of the on-disk ``ggml_shape``), block-quantized tensors are
exposed with their byte shape ``[..., bytes_per_row]`` - exactly the ``[N, K/256*144]`` uint8 rows the matmul
entry points take.  The container format itself is the published GGUF layout: magic ``GGUF``, u32 version,
u64 tensor count, u64 metadata count, key/value pairs, tensor infos, then the payload aligned to
``general.alignment`` (default 32).

``write_gguf`` writes the same container (synthetic models for tests and benches; there is no model file on
the machines this is developed on).
"""

from __future__ import annotations

import mmap
import struct
from dataclasses import dataclass
from math import prod
from pathlib import Path
from typing import Any, Iterable, Mapping, Sequence

import numpy as np

from hipengine_amd.quant.gguf import (
    GGMLQuantizationType,
    ggml_type,
    nbytes_for_shape,
    quant_layout,
    quant_shape_to_byte_shape,
)

GGUF_MAGIC = b"GGUF"
GGUF_DEFAULT_ALIGNMENT = 32
GGUF_SUPPORTED_VERSIONS = (2, 3)

# metadata value types of the container
_U8, _I8, _U16, _I16, _U32, _I32, _F32, _BOOL, _STRING, _ARRAY, _U64, _I64, _F64 = range(13)
_SCALAR_FORMAT = {_U8: "<B", _I8: "<b", _U16: "<H", _I16: "<h", _U32: "<I", _I32: "<i", _F32: "<f", _BOOL: "<?",
                  _U64: "<Q", _I64: "<q", _F64: "<d"}
_STORAGE_DTYPE = {"float32": np.float32, "float16": np.float16, "bf16": np.uint16, "uint8_blocks": np.uint8}


class GGUFFormatError(ValueError):
    pass


class MissingGGUFTensorError(KeyError):
    pass


@dataclass(frozen=True)
class GGUFTensorInfo:
    name: str
    shape: tuple[int, ...]          # row-major logical shape
    ggml_shape: tuple[int, ...]     # as stored: innermost dimension first
    ggml_type: int
    ggml_type_name: str
    n_elements: int
    nbytes: int
    offset: int                     # relative to the payload section
    data_offset: int                # absolute file offset
    byte_shape: tuple[int, ...]     # shape of the stored array (bytes per row for block types)


@dataclass(frozen=True)
class GGUFModelInfo:
    path: Path
    version: int
    alignment: int
    metadata: Mapping[str, Any]
    tensors: tuple[GGUFTensorInfo, ...]
    tensor_data_offset: int

    @property
    def tensor_count(self) -> int:
        return len(self.tensors)

    @property
    def total_tensor_nbytes(self) -> int:
        return sum(t.nbytes for t in self.tensors)

    @property
    def architecture(self) -> str | None:
        value = self.metadata.get("general.architecture")
        return None if value is None else str(value)

    @property
    def file_type(self) -> int | None:
        value = self.metadata.get("general.file_type")
        return None if value is None else int(value)

    def tensor(self, name: str) -> GGUFTensorInfo:
        for t in self.tensors:
            if t.name == name:
                return t
        raise MissingGGUFTensorError(f"missing GGUF tensor: {name}")

    def require(self, names: Iterable[str]) -> tuple[GGUFTensorInfo, ...]:
        table = {t.name: t for t in self.tensors}
        wanted = list(names)
        missing = [n for n in wanted if n not in table]
        if missing:
            more = "" if len(missing) <= 8 else f" (+{len(missing) - 8} more)"
            raise MissingGGUFTensorError(f"missing required GGUF tensors: {', '.join(missing[:8])}{more}")
        return tuple(table[n] for n in wanted)

    def names_with_prefix(self, prefix: str) -> tuple[str, ...]:
        return tuple(t.name for t in self.tensors if t.name.startswith(prefix))


class _Cursor:
    """Bounds-checked little-endian reads from a buffer."""

    def __init__(self, buf, size: int):
        self.buf, self.size, self.pos = buf, size, 0

    def take(self, n: int) -> bytes:
        if n < 0 or self.pos + n > self.size:
            raise EOFError(f"unexpected EOF while reading {n} bytes")
        out = bytes(self.buf[self.pos:self.pos + n])
        self.pos += n
        return out

    def scalar(self, kind: int):
        fmt = _SCALAR_FORMAT[kind]
        return struct.unpack(fmt, self.take(struct.calcsize(fmt)))[0]

    def string(self) -> str:
        return self.take(int(self.scalar(_U64))).decode("utf-8")

    def value(self, kind: int):
        if kind == _STRING:
            return self.string()
        if kind == _ARRAY:
            item = int(self.scalar(_U32))
            count = int(self.scalar(_U64))
            if item in (_STRING, _ARRAY):
                return [self.value(item) for _ in range(count)]
            if item not in _SCALAR_FORMAT:
                raise GGUFFormatError(f"unknown GGUF array item type {item}")
            fmt = _SCALAR_FORMAT[item]
            data = self.take(struct.calcsize(fmt) * count)
            return list(struct.unpack(f"<{count}{fmt[1]}", data)) if count else []
        if kind not in _SCALAR_FORMAT:
            raise GGUFFormatError(f"unknown GGUF metadata value type {kind}")
        return self.scalar(kind)


def _align_up(value: int, alignment: int) -> int:
    return (value + alignment - 1) // alignment * alignment


def scan_gguf(path: str | Path) -> GGUFModelInfo:
    """Parse the header, metadata and tensor table; no tensor payload is read."""
    resolved = Path(path).expanduser().resolve()
    file_size = resolved.stat().st_size
    with resolved.open("rb") as fh:
        if file_size < 4 or fh.read(4) != GGUF_MAGIC:
            raise GGUFFormatError(f"GGUF magic invalid: {resolved}")
        with mmap.mmap(fh.fileno(), 0, access=mmap.ACCESS_READ) as view:
            cur = _Cursor(view, file_size)
            cur.pos = 4
            version = int(cur.scalar(_U32))
            if version not in GGUF_SUPPORTED_VERSIONS:
                supported = ", ".join(str(v) for v in GGUF_SUPPORTED_VERSIONS)
                raise GGUFFormatError(f"unsupported GGUF version {version}; expected one of: {supported}")
            n_tensors, n_meta = int(cur.scalar(_U64)), int(cur.scalar(_U64))
            metadata: dict[str, Any] = {}
            for _ in range(n_meta):
                key = cur.string()
                kind = int(cur.scalar(_U32))
                if key in metadata:
                    raise GGUFFormatError(f"duplicate GGUF metadata key {key!r}")
                metadata[key] = cur.value(kind)
            raw = []
            seen: set[str] = set()
            for _ in range(n_tensors):
                name = cur.string()
                if name in seen:
                    raise GGUFFormatError(f"duplicate GGUF tensor name {name!r}")
                seen.add(name)
                n_dims = int(cur.scalar(_U32))
                dims = tuple(int(cur.scalar(_U64)) for _ in range(n_dims))
                raw.append((name, dims, int(cur.scalar(_U32)), int(cur.scalar(_U64))))
            alignment = int(metadata.get("general.alignment", GGUF_DEFAULT_ALIGNMENT))
            if alignment <= 0 or alignment & (alignment - 1):
                raise GGUFFormatError(f"invalid GGUF alignment {alignment}; expected non-zero power of two")
            payload = _align_up(cur.pos, alignment)

    tensors = []
    for name, dims, type_id, offset in raw:
        qtype = ggml_type(type_id)
        shape = tuple(reversed(dims))
        nbytes = nbytes_for_shape(shape, qtype)
        start = payload + offset
        if start < payload or start + nbytes > file_size:
            raise GGUFFormatError(
                f"tensor {name!r} byte range [{start}, {start + nbytes}) falls outside file size {file_size}")
        tensors.append(GGUFTensorInfo(name, shape, dims, int(qtype), qtype.name, int(prod(shape)), nbytes, offset, start,
                                      quant_shape_to_byte_shape(shape, qtype)))
    return GGUFModelInfo(resolved, version, alignment, metadata, tuple(tensors), payload)


load_gguf_index = scan_gguf


class GGUFReader:
    """Tensor table plus lazy read-only NumPy memory maps of the payloads."""

    def __init__(self, path: str | Path):
        self.info = scan_gguf(path)

    @property
    def path(self) -> Path:
        return self.info.path

    def tensor_info(self, name: str) -> GGUFTensorInfo:
        return self.info.tensor(name)

    def tensor_data(self, name: str) -> np.memmap:
        """The stored array: logical shape for F32 / F16 / BF16 (BF16 as uint16 bits), ``[..., bytes_per_row]``
        uint8 for block-quantized types."""
        t = self.tensor_info(name)
        dtype = _STORAGE_DTYPE[quant_layout(t.ggml_type).storage_dtype]
        return np.memmap(self.info.path, mode="r", dtype=dtype, offset=t.data_offset, shape=t.byte_shape)

    def to_device(self, name: str, *, runtime=None):
        """Upload a tensor's stored bytes unchanged (the raw layout the kernels take) and return the
        ``DeviceBuffer``; the caller owns and frees it."""
        from hipengine_amd.core import memory

        return memory.to_device(np.ascontiguousarray(self.tensor_data(name)), runtime=runtime)


# --------------------------------------------------------------------------------------------------------------
# writer (synthetic files)
# --------------------------------------------------------------------------------------------------------------

def _pack_string(text: str) -> bytes:
    data = text.encode("utf-8")
    return struct.pack("<Q", len(data)) + data


def _pack_value(value) -> bytes:
    if isinstance(value, bool):
        return struct.pack("<I?", _BOOL, value)
    if isinstance(value, int):
        return struct.pack("<Iq", _I64, value) if value < 0 else struct.pack("<II", _U32, value) if value < 2**32 \
            else struct.pack("<IQ", _U64, value)
    if isinstance(value, float):
        return struct.pack("<If", _F32, value)
    if isinstance(value, str):
        return struct.pack("<I", _STRING) + _pack_string(value)
    if isinstance(value, (list, tuple)):
        if all(isinstance(v, str) for v in value):
            return struct.pack("<IIQ", _ARRAY, _STRING, len(value)) + b"".join(_pack_string(v) for v in value)
        if all(isinstance(v, int) and not isinstance(v, bool) for v in value):
            return struct.pack("<IIQ", _ARRAY, _I32, len(value)) + struct.pack(f"<{len(value)}i", *value)
        if all(isinstance(v, float) for v in value):
            return struct.pack("<IIQ", _ARRAY, _F32, len(value)) + struct.pack(f"<{len(value)}f", *value)
    raise TypeError(f"unsupported GGUF metadata value {value!r}")


def write_gguf(path: str | Path, metadata: Mapping[str, Any],
               tensors: Sequence[tuple[str, int | GGMLQuantizationType, Sequence[int], np.ndarray]], *,
               version: int = 3, alignment: int = GGUF_DEFAULT_ALIGNMENT) -> Path:
    """Write a GGUF container.  ``tensors``: (name, ggml type, logical row-major shape, stored array) - for block
    types the stored array is the uint8 byte-shape array."""
    path = Path(path)
    meta = dict(metadata)
    if alignment != GGUF_DEFAULT_ALIGNMENT:
        meta["general.alignment"] = alignment
    head = bytearray(GGUF_MAGIC + struct.pack("<IQQ", version, len(tensors), len(meta)))
    for key, value in meta.items():
        head += _pack_string(key) + _pack_value(value)
    offset = 0
    blobs = []
    for name, type_id, shape, data in tensors:
        qtype = ggml_type(type_id)
        raw = np.ascontiguousarray(data)
        nbytes = nbytes_for_shape(tuple(shape), qtype)
        if raw.nbytes != nbytes:
            raise ValueError(f"tensor {name!r}: {raw.nbytes} stored bytes, expected {nbytes}")
        dims = tuple(reversed(tuple(int(d) for d in shape)))
        head += _pack_string(name) + struct.pack("<I", len(dims)) + struct.pack(f"<{len(dims)}Q", *dims)
        head += struct.pack("<IQ", int(qtype), offset)
        blobs.append((offset, raw))
        offset = _align_up(offset + nbytes, alignment)
    payload = _align_up(len(head), alignment)
    with path.open("wb") as fh:
        fh.write(head)
        fh.write(b"\0" * (payload - len(head)))
        for off, raw in blobs:
            fh.seek(payload + off)
            fh.write(raw.tobytes())
        fh.truncate(max(fh.tell(), payload + offset if blobs else payload))
    return path
