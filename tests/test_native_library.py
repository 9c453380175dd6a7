"""The layer that compiles and loads the HIP libraries (no GPU needed: hipcc cross-compiles, nothing is run).

What is checked here is how it fails and when it builds again: there is no other path than the compiled kernels, so a
missing compiler or a source that does not compile has to say so, at once and by name.
"""
import os

import pytest

from nanohybrid_vlm_amd.native import library


@pytest.fixture
def sandbox(tmp_path, monkeypatch):
    """Sources and libraries in a temporary folder of their own."""
    csrc, lib_dir = tmp_path / "csrc", tmp_path / "lib"
    csrc.mkdir()
    lib_dir.mkdir()
    (csrc / "common.h").write_text("#pragma once\n#define ANSWER 42\n")
    (csrc / "good.hip").write_text('#include "common.h"\nextern "C" int answer() { return ANSWER; }\n')
    monkeypatch.setattr(library, "CSRC", str(csrc))
    monkeypatch.setattr(library, "LIB_DIR", str(lib_dir))
    monkeypatch.setattr(library, "_loaded", {})
    return csrc, lib_dir


def test_a_missing_compiler_is_named(sandbox, monkeypatch):
    monkeypatch.setattr(library.shutil, "which", lambda name: None)
    monkeypatch.setattr(library.os.path, "isfile", lambda path: False if path.endswith("hipcc") else os.path.exists(path))
    with pytest.raises(library.NativeBuildError, match="hipcc was not found"):
        library.build_library("probe", ["good.hip"])


def test_a_source_that_does_not_compile_shows_the_compiler_s_words(sandbox):
    csrc, lib_dir = sandbox
    (csrc / "bad.hip").write_text('extern "C" int broken() { return no_such_name; }\n')
    with pytest.raises(library.NativeBuildError) as err:
        library.build_library("probe", ["good.hip", "bad.hip"])
    assert "bad.hip" in str(err.value) and "no_such_name" in str(err.value)
    assert not [f for f in os.listdir(lib_dir) if f.endswith(".so")], "nothing half-built is left behind"
    assert not [f for f in os.listdir(lib_dir) if f.startswith("nhv_build_")], "the work folder is gone"


def test_built_once_and_again_when_a_source_or_a_header_changes(sandbox):
    csrc, lib_dir = sandbox
    first = library.build_library("probe", ["good.hip"])
    assert os.path.dirname(first) == str(lib_dir) and os.path.isfile(first)
    stamp = os.stat(first).st_mtime_ns
    assert library.build_library("probe", ["good.hip"]) == first and os.stat(first).st_mtime_ns == stamp, "found, not built again"
    # the same sources under another name and with another define (the attention kernels: a library per head size)
    other = library.build_library("probe_d2", ["good.hip"], ["-DOTHER=1"])
    assert other != first and os.path.isfile(first) and os.path.isfile(other)
    # a changed header means new libraries, and those of the old sources are cleared away
    (csrc / "common.h").write_text("#pragma once\n#define ANSWER 43\n")
    second = library.build_library("probe", ["good.hip"])
    assert second != first and os.path.isfile(second) and not os.path.exists(first) and os.path.isfile(other)
    lib = library.load_library("probe", ["good.hip"])
    assert lib.answer() == 43                       # host code only: nothing here touches a GPU
    assert library.load_library("probe", ["good.hip"]) is lib
