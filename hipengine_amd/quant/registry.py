"""Quant plugin registry (hipEngine: ``hipengine/quant/registry.py:8-37``)."""

from __future__ import annotations

from hipengine_amd.quant.base import QuantPlugin


class DuplicateQuantError(ValueError):
    pass


class MissingQuantError(LookupError):
    pass


_PLUGINS: dict[str, QuantPlugin] = {}


def register_quant(plugin: QuantPlugin, *, replace: bool = False) -> QuantPlugin:
    name = plugin.name
    if not name:
        raise ValueError("quant plugin name must be non-empty")
    if name in _PLUGINS and not replace:
        raise DuplicateQuantError(f"quant plugin {name!r} already registered")
    _PLUGINS[name] = plugin
    return plugin


def resolve_quant(name: str) -> QuantPlugin:
    plugin = _PLUGINS.get(name)
    if plugin is None:
        known = ", ".join(sorted(_PLUGINS)) or "<none>"
        raise MissingQuantError(f"quant plugin {name!r} not registered; known: {known}")
    return plugin


def registered_quants() -> tuple[QuantPlugin, ...]:
    return tuple(_PLUGINS[n] for n in sorted(_PLUGINS))
