"""Registries: architecture name -> model, and part kind -> part class.

``config.json``'s ``architectures`` entry selects an ``Architecture``: a typed
configuration class and a function from that configuration to a ``ModelPlan``.
Each ``PartSpec.kind`` of a plan selects a class from the registry of its role
(mixer, feed-forward, norm, position encoding, block, embedding, head).

The reference has no registry: it checks the architecture string inside its
config reader and constructs its one model class directly
(qwen3_runtime/models/qwen3.py:35-37, qwen3_runtime/utils/loader.py:96-97).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Mapping

ROLES = ("mixer", "feed_forward", "norm", "position", "block", "embedding", "head")


@dataclass(frozen=True)
class Architecture:
    name: str
    read_config: Callable[[Mapping[str, Any]], Any]
    make_plan: Callable[[Any], Any]


_ARCHITECTURES: dict[str, Architecture] = {}
_PARTS: dict[str, dict[str, type]] = {role: {} for role in ROLES}
# named configurations: name -> (config.json as a dict, page size it is run with by default)
_PRESETS: dict[str, tuple[dict, int]] = {}


def register_architecture(name: str, read_config, make_plan) -> Architecture:
    arch = Architecture(name, read_config, make_plan)
    _ARCHITECTURES[name] = arch
    return arch


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def architecture_names() -> list[str]:
    _load_builtin()
    return sorted(_ARCHITECTURES)


def architecture_for(raw_config: Mapping[str, Any]) -> Architecture:
    """Pick the architecture a config.json names, or say which ones exist."""
    _load_builtin()
    names = raw_config.get("architectures") or []
    if isinstance(names, str):
        names = [names]
    for name in names:
        if name in _ARCHITECTURES:
            return _ARCHITECTURES[name]
    raise ValueError(
        f"no registered architecture among {list(names)}; registered: {sorted(_ARCHITECTURES)}"
    )


def register_preset(name: str, raw_config: Mapping[str, Any], page_size: int = 16) -> None:
    """A named configuration (a config.json as a dict, ``architectures`` included) that the
    entry points build with random weights: ``--preset NAME`` on the command line, and the
    model ``LLM(None)`` makes is the first one registered."""
    if not raw_config.get("architectures"):
        raise ValueError(f"preset {name!r}: the configuration names no architecture")
    _PRESETS[name] = (dict(raw_config), int(page_size))


def unregister_preset(name: str) -> None:
    _PRESETS.pop(name, None)


def preset_names() -> list[str]:
    _load_builtin()
    return list(_PRESETS)


def preset_config(name: str | None = None) -> dict:
    """The configuration registered under ``name`` (None: the first registered), as a fresh dict."""
    _load_builtin()
    if name is None:
        if not _PRESETS:
            raise ValueError("no preset is registered")
        name = next(iter(_PRESETS))
    try:
        return dict(_PRESETS[name][0])
    except KeyError:
        raise ValueError(f"unknown preset {name!r}; presets: {list(_PRESETS)}") from None


def preset_page_size(name: str) -> int:
    _load_builtin()
    return _PRESETS[name][1] if name in _PRESETS else 16


def register_part(role: str, kind: str, cls: type | None = None):
    """Register ``cls`` as the part ``kind`` of ``role``; usable as a decorator."""
    if role not in _PARTS:
        raise ValueError(f"unknown part role {role!r}; roles: {ROLES}")

    def _put(c: type) -> type:
        _PARTS[role][kind] = c
        return c

    return _put if cls is None else _put(cls)


def unregister_part(role: str, kind: str) -> None:
    _PARTS[role].pop(kind, None)


def part_class(role: str, kind: str) -> type:
    _load_builtin()
    try:
        return _PARTS[role][kind]
    except KeyError:
        raise ValueError(
            f"no {role} part of kind {kind!r}; registered: {sorted(_PARTS.get(role, {}))}"
        ) from None


_loaded = False


def _load_builtin() -> None:
    """Import the modules whose import registers the shipped parts and model."""
    global _loaded
    if _loaded:
        return
    _loaded = True
    from . import parts  # noqa: F401  (registers part kinds)
    from .models import qwen3  # noqa: F401  (registers Qwen3ForCausalLM)
