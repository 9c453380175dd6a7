"""The list of native libraries of the package, for the build entry point."""
from __future__ import annotations

from concurrent.futures import ThreadPoolExecutor

from . import library, ops


def build_all(force: bool = False) -> list[str]:
    """Compiles every HIP library (always, when ``force``) and returns their paths: the core library, the
    wrapper of the vendor's matrix library, and the bfloat16 attention library for each of the usual head sizes (another head size is compiled when a model
    first needs it)."""
    jobs = [("nhv_core", ops.CORE_SOURCES, [], []), ("nhv_blas", ops.BLAS_SOURCES, [], ops.BLAS_LINK)]
    jobs += [(f"nhv_attention_d{d}", ops.ATTENTION_SOURCES, [f"-DNHV_HEAD_DIM={d}"], [])
             for d in ops.ATTENTION_HEAD_DIMS_BUILT_AHEAD]
    with ThreadPoolExecutor(max_workers=4) as pool:
        return list(pool.map(lambda j: library.build_library(j[0], j[1], j[2], force=force, link=j[3]), jobs))
