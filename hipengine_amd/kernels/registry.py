"""Kernel registry keyed by ``(backend, layer, quant, variant)``.

Same public surface and lookup rules as hipEngine's
``hipengine/kernels/registry.py:17-203`` so that the dispatch layer can use it
unchanged: exact key first, then the same key without a variant, then the
``fp16`` quant on the same backend, then the same three on ``cpu_reference``.
This package registers nothing under ``cpu_reference``; the fallback exists
only so that a host application which does can keep relying on it.
"""

from __future__ import annotations

from collections.abc import Callable, Iterable, Mapping
from dataclasses import dataclass
from typing import Any, Literal

Kernel = Callable[..., Any]
MissingPolicy = Literal["error", "none"]

_FALLBACK_BACKEND = "cpu_reference"
_FALLBACK_QUANT = "fp16"


@dataclass(frozen=True, order=True)
class KernelKey:
    backend: str
    layer: str
    quant: str
    variant: str = ""

    def __post_init__(self) -> None:
        for name in ("backend", "layer", "quant"):
            if not getattr(self, name):
                raise ValueError(f"KernelKey.{name} must be non-empty")

    def display(self) -> str:
        text = f"backend={self.backend!r}, layer={self.layer!r}, quant={self.quant!r}"
        return text + (f", variant={self.variant!r}" if self.variant else "")


class DuplicateKernelError(ValueError):
    """A key was registered twice without ``replace=True``."""


class MissingKernelError(LookupError):
    """No registered kernel satisfies the request, fallbacks included."""

    def __init__(self, requested: KernelKey, attempted: Iterable[KernelKey]):
        self.requested = requested
        self.attempted = tuple(attempted)
        tried = "; ".join(k.display() for k in self.attempted)
        super().__init__(f"no kernel implementation for {requested.display()}; attempted: {tried}")


class _Table:
    """The process-wide table, a memo of resolved lookups and a mutation counter."""

    def __init__(self) -> None:
        self.kernels: dict[KernelKey, Kernel] = {}
        self.memo: dict[tuple[str, str, str, str], tuple[KernelKey, Kernel]] = {}
        self.generation = 0

    def touch(self) -> None:
        self.memo.clear()
        self.generation += 1


_T = _Table()


def generation() -> int:
    """Counter bumped by every mutation; callers memoizing ``resolve`` compare it."""
    return _T.generation


def register(key: KernelKey, kernel: Kernel, *, replace: bool = False) -> Kernel:
    if not replace and key in _T.kernels:
        raise DuplicateKernelError(f"kernel already registered for {key.display()}")
    _T.kernels[key] = kernel
    _T.touch()
    return kernel


def unregister(key: KernelKey) -> None:
    _T.kernels.pop(key, None)
    _T.touch()


def registered_keys() -> tuple[KernelKey, ...]:
    return tuple(sorted(_T.kernels))


def is_registered(key: KernelKey) -> bool:
    """Exact-key test, no fallbacks."""
    return _T.kernels.get(key) is not None


def _candidates(req: KernelKey) -> tuple[KernelKey, ...]:
    out: list[KernelKey] = []
    backends = (req.backend,) if req.backend == _FALLBACK_BACKEND else (req.backend, _FALLBACK_BACKEND)
    quants = (req.quant,) if req.quant == _FALLBACK_QUANT else (req.quant, _FALLBACK_QUANT)
    variants = (req.variant, "") if req.variant else ("",)
    for backend in backends:
        for quant in quants:
            for variant in variants:
                key = KernelKey(backend, req.layer, quant, variant)
                if key not in out:
                    out.append(key)
    return tuple(out)


def resolve(*, backend: str, layer: str, quant: str, variant: str = "", missing: MissingPolicy = "error") -> Kernel | None:
    ident = (backend, layer, quant, variant)
    hit = _T.memo.get(ident)
    if hit is not None:
        if _T.kernels.get(hit[0]) is hit[1]:
            return hit[1]
        del _T.memo[ident]
    requested = KernelKey(backend, layer, quant, variant)
    tried = _candidates(requested)
    for key in tried:
        fn = _T.kernels.get(key)
        if fn is not None:
            _T.memo[ident] = (key, fn)
            return fn
    if missing == "none":
        return None
    raise MissingKernelError(requested, tried)


def can_resolve(*, backend: str, layer: str, quant: str, variant: str = "") -> bool:
    return resolve(backend=backend, layer=layer, quant=quant, variant=variant, missing="none") is not None


def snapshot_registry_for_tests() -> dict[KernelKey, Kernel]:
    return dict(_T.kernels)


def clear_registry_for_tests() -> None:
    _T.kernels.clear()
    _T.touch()


def restore_registry_for_tests(kernels: Mapping[KernelKey, Kernel]) -> None:
    _T.kernels.clear()
    _T.kernels.update(kernels)
    _T.touch()
