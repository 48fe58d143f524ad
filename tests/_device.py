"""Host-side helper for the GPU tests: moves NumPy arrays to and from device
buffers through the package's ctypes HIP binding (no torch) and keeps the
buffers alive for the duration of a test."""

from __future__ import annotations

import numpy as np

from hipengine_amd.core import memory
from hipengine_amd.core.build import load_library
from hipengine_amd.core.hip import get_hip_runtime


class Device:
    def __init__(self) -> None:
        self.runtime = get_hip_runtime()
        if self.runtime.device_count() < 1:
            raise RuntimeError("no HIP device visible: the gpu tests need one MI355X")
        self.runtime.set_device(0)
        self.library = load_library()   # raises when the library was not built

    def put(self, array: np.ndarray) -> memory.DeviceBuffer:
        return memory.to_device(np.ascontiguousarray(array), runtime=self.runtime)

    def empty(self, nbytes: int, fill: int | None = 0xA5) -> memory.DeviceBuffer:
        buf = memory.malloc(nbytes, runtime=self.runtime)
        if fill is not None and nbytes:
            self.runtime.memset(buf.ptr, fill, nbytes)
        return buf

    def get(self, buf: memory.DeviceBuffer, dtype, shape) -> np.ndarray:
        self.runtime.device_synchronize()
        return memory.to_host(buf, dtype, shape)

    def free(self, *bufs: memory.DeviceBuffer) -> None:
        for b in bufs:
            memory.free(b)

    def sync(self) -> None:
        self.runtime.device_synchronize()
