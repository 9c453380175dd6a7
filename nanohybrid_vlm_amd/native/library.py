"""Builds the HIP sources under ``csrc/`` with hipcc for gfx950 and loads them.

One shared library per set of sources and compile-time parameters; its file name
carries a hash of the sources and flags, so a library built from other sources is
never loaded by mistake. A library that is there is loaded; only when none fits
is hipcc run (a fresh checkout compiles at its first call and prints a line for
every file meanwhile). The library lands in ``native/_lib`` inside the package,
or in a per-user folder under the system's temporary folder when the package is
not writable.

There is no fallback: without hipcc and without a built library, loading raises.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import re
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor

ARCH = "gfx950"
CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_lib")

# -packed-fp32-ops is switched off: the compiler then makes no packed float instructions (v_pk_add_f32,
# v_pk_mul_f32, v_pk_fma_f32) out of ordinary float code; some of their forms have given wrong results on gfx950.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


class NativeBuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[nanohybrid_vlm_amd] {msg}", file=sys.stderr, flush=True)


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.isfile(exe):
        raise NativeBuildError("hipcc was not found (looked on PATH and in /opt/rocm/bin); "
                               "the HIP kernels cannot be built and there is no other path")
    return exe


def _sources(names: list[str]) -> list[str]:
    return [os.path.join(CSRC, n) for n in names]


def _digest(sources: list[str], defines: list[str], link: list[str] | None = None) -> str:
    h = hashlib.sha256()
    for path in sorted(sources) + sorted(
            os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")):
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS + defines + list(link or [])).encode())
    return h.hexdigest()[:16]


def _writable_dir() -> str:
    try:
        os.makedirs(LIB_DIR, exist_ok=True)
        fd, probe = tempfile.mkstemp(prefix=".probe", dir=LIB_DIR)
        os.close(fd)
        os.remove(probe)
        return LIB_DIR
    except OSError:
        d = os.path.join(tempfile.gettempdir(), f"nanohybrid_vlm_amd-{os.getuid()}")
        os.makedirs(d, exist_ok=True)
        return d


def _candidates(file_name: str) -> list[str]:
    return [os.path.join(LIB_DIR, file_name),
            os.path.join(tempfile.gettempdir(), f"nanohybrid_vlm_amd-{os.getuid()}", file_name)]


def _compile_one(src: str, obj: str, defines: list[str]) -> None:
    cmd = [_hipcc(), *HIPCC_FLAGS, *defines, "-I", CSRC, "-c", src, "-o", obj]
    t0 = time.time()
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise NativeBuildError(f"hipcc failed on {os.path.basename(src)}:\n{proc.stderr[-4000:]}")
    _say(f"compiled {os.path.basename(src)} {' '.join(defines)} in {time.time() - t0:.1f} s")


def build_library(stem: str, source_names: list[str], defines: list[str] | None = None, force: bool = False,
                  link: list[str] | None = None) -> str:
    """Compile ``source_names`` into ``lib<stem>_<hash>.so`` and return its path. ``link``: further arguments of the
    link step (libraries the sources call)."""
    defines = list(defines or [])
    link = list(link or [])
    sources = _sources(source_names)
    file_name = f"lib{stem}_{_digest(sources, defines, link)}.so"
    if not force:
        for path in _candidates(file_name):
            if os.path.isfile(path):
                return path
    out_dir = _writable_dir()
    target = os.path.join(out_dir, file_name)
    _say(f"building {file_name} from {len(sources)} HIP sources for {ARCH} ...")
    work = tempfile.mkdtemp(prefix="nhv_build_", dir=out_dir)
    try:
        objs = [os.path.join(work, os.path.basename(s) + ".o") for s in sources]
        with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
            list(pool.map(lambda so: _compile_one(so[0], so[1], defines), zip(sources, objs)))
        tmp_target = os.path.join(work, file_name)
        cmd = [_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-fno-gpu-rdc", *objs, *link, "-o", tmp_target]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise NativeBuildError(f"linking {file_name} failed:\n{proc.stderr[-4000:]}")
        os.replace(tmp_target, target)        # atomic: another process never sees half a file
        # libraries of older sources are of no use any more
        older = re.compile(re.escape(f"lib{stem}_") + r"[0-9a-f]{16}\.so")     # (not a library whose name begins with this one's)
        for f in os.listdir(out_dir):
            if older.fullmatch(f) and f != file_name:
                try:
                    os.remove(os.path.join(out_dir, f))
                except OSError:
                    pass
    finally:
        shutil.rmtree(work, ignore_errors=True)
    _say(f"built {target}")
    return target


_loaded: dict[str, ctypes.CDLL] = {}


def load_library(stem: str, source_names: list[str], defines: list[str] | None = None,
                 link: list[str] | None = None) -> ctypes.CDLL:
    key = stem + "|" + " ".join(defines or [])
    lib = _loaded.get(key)
    if lib is None:
        path = build_library(stem, source_names, defines, link=link)
        lib = ctypes.CDLL(path)
        _loaded[key] = lib
    return lib
