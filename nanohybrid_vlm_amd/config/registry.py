"""One registry from an architecture's name to the way its model is made.

The reference keys its registry by ``model_type`` and checks the checkpoint's
``architectures`` against the entry (nanovllm/models/registry.py:36-149); the same
two keys and the same kinds of error are kept here. An entry is not a model class
but a recipe: the typed configuration, a function from it to a ``ModelSpec`` (the
parts of every layer and the run order) and the names of the checkpoint's tensors.
"""
from __future__ import annotations

import importlib
from dataclasses import dataclass, field
from typing import Callable


class UnknownArchitecture(ValueError):
    pass


@dataclass(frozen=True)
class WeightSource:
    """Where one checkpoint tensor goes: into ``param`` (a name of the built model),
    whole or as rows [row_start, row_start + rows) of a packed parameter."""

    param: str
    row_start: int = 0
    rows: int | None = None        # None: the whole parameter
    # a second copy of what another checkpoint tensor already gives the same parameter (a tied head stored beside
    # the embedding): the file may leave it out; if it is there it must hold the same numbers as the first
    copy: bool = False


@dataclass(frozen=True)
class Architecture:
    name: str                                   # e.g. "Qwen3ForCausalLM"
    model_types: tuple[str, ...]                # values of config.json's model_type
    parse_config: Callable                      # raw dict -> typed configuration
    build_spec: Callable                        # typed configuration -> ModelSpec
    checkpoint_names: Callable                  # typed configuration -> {checkpoint tensor name: WeightSource}
    ignored_prefixes: tuple[str, ...] = ()      # checkpoint names under these are skipped (nanovllm/utils/loader.py:27-31)
    named_shapes: dict = field(default_factory=dict)   # name -> config.json contents, for measurements and examples


_ARCHITECTURES: dict[str, Architecture] = {}
# Modules that register architectures (and parts) when they are imported. The engine's own architectures are such a
# module like any other, and no name of an architecture stands here: the package ``architectures`` imports every
# module that lies in its folder. ``import_plugins`` adds to the list (the command line's ``--plugin``).
_PLUGINS: list[str] = [__name__.rsplit(".", 2)[0] + ".architectures"]
_imported: set[str] = set()


def import_plugins(names=()) -> None:
    """Imports modules that register architectures or parts of their own; each once."""
    for name in names or ():
        if name not in _PLUGINS:
            _PLUGINS.append(name)
    for name in list(_PLUGINS):
        if name not in _imported:
            _imported.add(name)
            importlib.import_module(name)


def register_architecture(arch: Architecture, replace: bool = False) -> None:
    if arch.name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture '{arch.name}' is already registered")
    _ARCHITECTURES[arch.name] = arch


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def _get(name: str) -> Architecture | None:
    import_plugins()
    return _ARCHITECTURES.get(name)


def registered_architectures() -> list[str]:
    import_plugins()
    return sorted(_ARCHITECTURES)


def named_shapes() -> dict[str, dict]:
    """Every registered architecture's named configurations (config.json contents by name)."""
    out: dict[str, dict] = {}
    for name in registered_architectures():
        arch = _get(name)
        if arch is not None:
            out.update(arch.named_shapes)
    return out


def resolve_architecture(raw_config: dict) -> Architecture:
    """Pick the architecture for a config.json: by ``architectures`` if it lists one
    that is registered, else by ``model_type``; a ``model_type`` whose entry is not
    among the listed architectures is an error (registry.py:69-95)."""
    listed = list(raw_config.get("architectures") or [])
    model_type = raw_config.get("model_type")
    for name in listed:
        arch = _get(name)
        if arch is not None:
            if model_type and arch.model_types and model_type not in arch.model_types:
                raise UnknownArchitecture(
                    f"config.json: architecture '{name}' does not go with model_type '{model_type}' "
                    f"(it is registered for {list(arch.model_types)})")
            return arch
    if model_type:
        import_plugins()
        by_type = [a for a in list(_ARCHITECTURES.values()) if model_type in a.model_types]
        if by_type:
            arch = by_type[0]
            if listed and arch.name not in listed:
                raise UnknownArchitecture(
                    f"config.json: model_type '{model_type}' is registered as '{arch.name}', "
                    f"but the checkpoint lists {listed}")
            return arch
    raise UnknownArchitecture(
        f"config.json names architectures {listed} and model_type {model_type!r}; "
        f"registered architectures: {registered_architectures()}")
