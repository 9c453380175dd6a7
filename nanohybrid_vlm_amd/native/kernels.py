"""The list of native libraries of the package, for the build entry point."""
from __future__ import annotations

from . import library, ops


def build_all(force: bool = False) -> list[str]:
    """Compiles every HIP library (always, when ``force``) and returns their paths."""
    return [library.build_library("nhv_core", ops.CORE_SOURCES, force=force)]
