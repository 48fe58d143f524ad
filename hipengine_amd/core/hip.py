"""ctypes binding of the HIP runtime calls the GGUF kernels' host side needs.

Torch-free by contract, and lazy: importing this module neither opens
``libamdhip64.so`` nor touches a GPU; that happens on the first
``get_hip_runtime()``.  Mirrors the method names of hipEngine's
``hipengine/core/hip.py:102-610`` (``HipRuntime``) for the subset this path
uses: memory, streams, events, graph capture and error reporting.
"""

from __future__ import annotations

import ctypes
import enum
import os
from typing import Final

HIP_SUCCESS: Final[int] = 0
HIP_ERROR_INVALID_VALUE: Final[int] = 1
HIP_ERROR_NOT_READY: Final[int] = 600
_LIBRARY_CANDIDATES: Final[tuple[str, ...]] = (
    "/opt/rocm/lib/libamdhip64.so",
    "libamdhip64.so",
)


class MemcpyKind(enum.IntEnum):
    HOST_TO_HOST = 0
    HOST_TO_DEVICE = 1
    DEVICE_TO_HOST = 2
    DEVICE_TO_DEVICE = 3
    DEFAULT = 4


HipMemcpyKind = MemcpyKind


class HipError(RuntimeError):
    """A HIP runtime call or a kernel launcher returned a non-success code."""

    def __init__(self, code: int, message: str):
        self.code = int(code)
        super().__init__(f"HIP error {self.code}: {message}")


_VP = ctypes.c_void_p
_SZ = ctypes.c_size_t
_INT = ctypes.c_int
_UINT = ctypes.c_uint

# name -> (argtypes, restype); restype None means "int hipError_t"
_PROTOTYPES: Final[dict[str, list]] = {
    "hipMalloc": [ctypes.POINTER(_VP), _SZ],
    "hipFree": [_VP],
    "hipHostMalloc": [ctypes.POINTER(_VP), _SZ, _UINT],
    "hipHostFree": [_VP],
    "hipMemcpy": [_VP, _VP, _SZ, _INT],
    "hipMemcpyAsync": [_VP, _VP, _SZ, _INT, _VP],
    "hipMemset": [_VP, _INT, _SZ],
    "hipMemsetAsync": [_VP, _INT, _SZ, _VP],
    "hipMemGetInfo": [ctypes.POINTER(_SZ), ctypes.POINTER(_SZ)],
    "hipStreamCreateWithFlags": [ctypes.POINTER(_VP), _UINT],
    "hipStreamDestroy": [_VP],
    "hipStreamSynchronize": [_VP],
    "hipStreamWaitEvent": [_VP, _VP, _UINT],
    "hipStreamBeginCapture": [_VP, _INT],
    "hipStreamEndCapture": [_VP, ctypes.POINTER(_VP)],
    "hipGraphInstantiate": [ctypes.POINTER(_VP), _VP, _VP, _VP, _SZ],
    "hipGraphLaunch": [_VP, _VP],
    "hipGraphExecDestroy": [_VP],
    "hipGraphDestroy": [_VP],
    "hipEventCreateWithFlags": [ctypes.POINTER(_VP), _UINT],
    "hipEventDestroy": [_VP],
    "hipEventRecord": [_VP, _VP],
    "hipEventSynchronize": [_VP],
    "hipEventQuery": [_VP],
    "hipEventElapsedTime": [ctypes.POINTER(ctypes.c_float), _VP, _VP],
    "hipDeviceSynchronize": [],
    "hipGetDeviceCount": [ctypes.POINTER(_INT)],
    "hipSetDevice": [_INT],
    "hipGetDevice": [ctypes.POINTER(_INT)],
    "hipDeviceGetAttribute": [ctypes.POINTER(_INT), _INT, _INT],
    "hipGetLastError": [],
}

# hipDeviceAttribute_t values used below (hip_runtime_api.h)
ATTR_CLOCK_RATE_KHZ: Final[int] = 5
ATTR_MULTIPROCESSOR_COUNT: Final[int] = 63
ATTR_MEMORY_CLOCK_RATE_KHZ: Final[int] = 60
ATTR_MEMORY_BUS_WIDTH: Final[int] = 59


class HipRuntime:
    """A loaded HIP runtime library with typed entry points."""

    def __init__(self, library: ctypes.CDLL):
        self.library = library
        for name, argtypes in _PROTOTYPES.items():
            fn = getattr(library, name)
            fn.argtypes = argtypes
            fn.restype = _INT
        library.hipGetErrorString.argtypes = [_INT]
        library.hipGetErrorString.restype = ctypes.c_char_p

    @classmethod
    def load(cls, path: str | None = None) -> "HipRuntime":
        candidates = (path,) if path else _LIBRARY_CANDIDATES
        last: OSError | None = None
        for name in candidates:
            if os.path.isabs(name) and not os.path.exists(name):
                continue
            try:
                return cls(ctypes.CDLL(name, mode=ctypes.RTLD_GLOBAL))
            except OSError as exc:  # try the next candidate
                last = exc
        raise OSError(f"could not load the HIP runtime from {candidates}: {last}")

    # -- errors ---------------------------------------------------------
    def error_string(self, code: int) -> str:
        text = self.library.hipGetErrorString(int(code))
        return text.decode("utf-8", "replace") if text else f"hipError {int(code)}"

    def check(self, code: int) -> None:
        if int(code) != HIP_SUCCESS:
            raise HipError(int(code), self.error_string(int(code)))

    # -- devices ----------------------------------------------------------
    def device_count(self) -> int:
        n = _INT(0)
        code = self.library.hipGetDeviceCount(ctypes.byref(n))
        return int(n.value) if code == HIP_SUCCESS else 0

    def set_device(self, device: int) -> None:
        self.check(self.library.hipSetDevice(int(device)))

    def current_device(self) -> int:
        n = _INT(0)
        self.check(self.library.hipGetDevice(ctypes.byref(n)))
        return int(n.value)

    def device_attribute(self, attribute: int, device: int = 0) -> int:
        v = _INT(0)
        self.check(self.library.hipDeviceGetAttribute(ctypes.byref(v), int(attribute), int(device)))
        return int(v.value)

    def mem_get_info(self) -> tuple[int, int]:
        free, total = _SZ(0), _SZ(0)
        self.check(self.library.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)))
        return int(free.value), int(total.value)

    # -- memory -----------------------------------------------------------
    def malloc(self, nbytes: int) -> int:
        if nbytes < 0:
            raise ValueError("nbytes must be non-negative")
        ptr = _VP()
        self.check(self.library.hipMalloc(ctypes.byref(ptr), nbytes))
        return int(ptr.value or 0)

    def free(self, ptr: int) -> None:
        self.check(self.library.hipFree(_VP(ptr)))

    def host_malloc(self, nbytes: int, *, flags: int = 0) -> int:
        ptr = _VP()
        self.check(self.library.hipHostMalloc(ctypes.byref(ptr), nbytes, flags))
        return int(ptr.value or 0)

    def host_free(self, ptr: int) -> None:
        self.check(self.library.hipHostFree(_VP(ptr)))

    def memcpy(self, dst: int, src: int, nbytes: int, kind: MemcpyKind | int) -> None:
        self.check(self.library.hipMemcpy(_VP(dst), _VP(src), nbytes, int(kind)))

    def memcpy_async(self, dst: int, src: int, nbytes: int, kind: MemcpyKind | int, stream: int) -> None:
        self.check(self.library.hipMemcpyAsync(_VP(dst), _VP(src), nbytes, int(kind), _VP(stream)))

    def memset(self, dst: int, value: int, nbytes: int) -> None:
        self.check(self.library.hipMemset(_VP(dst), int(value), nbytes))

    def memset_async(self, dst: int, value: int, nbytes: int, stream: int) -> None:
        self.check(self.library.hipMemsetAsync(_VP(dst), int(value), nbytes, _VP(stream)))

    # -- streams, events, graphs ------------------------------------------
    def stream_create(self, *, flags: int = 0) -> int:
        """A stream at the default priority (other priorities are never used)."""
        s = _VP()
        self.check(self.library.hipStreamCreateWithFlags(ctypes.byref(s), flags))
        return int(s.value or 0)

    def stream_destroy(self, stream: int) -> None:
        self.check(self.library.hipStreamDestroy(_VP(stream)))

    def stream_synchronize(self, stream: int) -> None:
        self.check(self.library.hipStreamSynchronize(_VP(stream)))

    def stream_wait_event(self, stream: int, event: int, *, flags: int = 0) -> None:
        self.check(self.library.hipStreamWaitEvent(_VP(stream), _VP(event), flags))

    def stream_begin_capture(self, stream: int, mode: int = 2) -> None:
        self.check(self.library.hipStreamBeginCapture(_VP(stream), mode))

    def stream_end_capture(self, stream: int) -> int:
        g = _VP()
        self.check(self.library.hipStreamEndCapture(_VP(stream), ctypes.byref(g)))
        return int(g.value or 0)

    def graph_instantiate(self, graph: int) -> int:
        e = _VP()
        self.check(self.library.hipGraphInstantiate(ctypes.byref(e), _VP(graph), None, None, 0))
        return int(e.value or 0)

    def graph_launch(self, graph_exec: int, stream: int) -> None:
        self.check(self.library.hipGraphLaunch(_VP(graph_exec), _VP(stream)))

    def graph_exec_destroy(self, graph_exec: int) -> None:
        self.check(self.library.hipGraphExecDestroy(_VP(graph_exec)))

    def graph_destroy(self, graph: int) -> None:
        self.check(self.library.hipGraphDestroy(_VP(graph)))

    def event_create(self, *, flags: int = 0) -> int:
        e = _VP()
        self.check(self.library.hipEventCreateWithFlags(ctypes.byref(e), flags))
        return int(e.value or 0)

    def event_destroy(self, event: int) -> None:
        self.check(self.library.hipEventDestroy(_VP(event)))

    def event_record(self, event: int, stream: int = 0) -> None:
        self.check(self.library.hipEventRecord(_VP(event), _VP(stream)))

    def event_synchronize(self, event: int) -> None:
        self.check(self.library.hipEventSynchronize(_VP(event)))

    def event_query(self, event: int) -> bool:
        code = self.library.hipEventQuery(_VP(event))
        if code == HIP_ERROR_NOT_READY:
            return False
        self.check(code)
        return True

    def event_elapsed_time_ms(self, start: int, stop: int) -> float:
        ms = ctypes.c_float(0.0)
        self.check(self.library.hipEventElapsedTime(ctypes.byref(ms), _VP(start), _VP(stop)))
        return float(ms.value)

    def device_synchronize(self) -> None:
        self.check(self.library.hipDeviceSynchronize())


_default: HipRuntime | None = None


def get_hip_runtime(path: str | None = None) -> HipRuntime:
    """The process-wide runtime, loaded on first use."""
    global _default
    if _default is None:
        _default = HipRuntime.load(path)
    return _default


def is_default_runtime_loaded() -> bool:
    return _default is not None


def hip_device_available() -> bool:
    """True when the HIP runtime loads and reports at least one device."""
    try:
        return get_hip_runtime().device_count() > 0
    except OSError:
        return False
