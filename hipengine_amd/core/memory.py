"""Device buffers as plain integer pointers (hipEngine: ``hipengine/core/memory.py:18-27,124-229``)."""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from hipengine_amd.core.hip import HipRuntime, MemcpyKind, get_hip_runtime


@dataclass
class DeviceBuffer:
    ptr: int
    nbytes: int
    runtime: HipRuntime | None = None


def malloc(nbytes: int, *, runtime: HipRuntime | None = None) -> DeviceBuffer:
    rt = runtime or get_hip_runtime()
    return DeviceBuffer(rt.malloc(max(int(nbytes), 1)), int(nbytes), rt)


def free(buf: DeviceBuffer) -> None:
    if buf.ptr:
        (buf.runtime or get_hip_runtime()).free(buf.ptr)
        buf.ptr = 0


def host_array_ptr(array: np.ndarray) -> int:
    if not array.flags["C_CONTIGUOUS"]:
        raise ValueError("host array must be C-contiguous")
    return int(array.ctypes.data)


def copy_host_to_device(buf: DeviceBuffer, host_ptr: int, nbytes: int | None = None) -> None:
    n = buf.nbytes if nbytes is None else int(nbytes)
    if n > buf.nbytes:
        raise ValueError("copy exceeds the device buffer")
    (buf.runtime or get_hip_runtime()).memcpy(buf.ptr, host_ptr, n, MemcpyKind.HOST_TO_DEVICE)


def copy_device_to_host(host_ptr: int, buf: DeviceBuffer, nbytes: int | None = None) -> None:
    n = buf.nbytes if nbytes is None else int(nbytes)
    if n > buf.nbytes:
        raise ValueError("copy exceeds the device buffer")
    (buf.runtime or get_hip_runtime()).memcpy(host_ptr, buf.ptr, n, MemcpyKind.DEVICE_TO_HOST)


def to_device(array: np.ndarray, *, runtime: HipRuntime | None = None) -> DeviceBuffer:
    """Allocate a device buffer and upload a host array into it (synchronous)."""
    host = np.ascontiguousarray(array)
    buf = malloc(host.nbytes, runtime=runtime)
    if host.nbytes:
        copy_host_to_device(buf, host_array_ptr(host), host.nbytes)
    return buf


def to_host(buf: DeviceBuffer, dtype, shape) -> np.ndarray:
    """Download a device buffer into a new host array (synchronous)."""
    out = np.empty(shape, dtype=dtype)
    if out.nbytes > buf.nbytes:
        raise ValueError("requested view exceeds the device buffer")
    if out.nbytes:
        copy_device_to_host(host_array_ptr(out), buf, out.nbytes)
    return out
