"""The kernel library's bookkeeping (no GPU, no compiler): which sources it belongs to and where it may go."""
import os
import re

from llm_infrence_engine_amd.kernels import build


def test_source_hash_names_the_sources_and_the_flags(monkeypatch):
    h = build.source_hash()
    assert re.fullmatch(r"[0-9a-f]{12}", h) and h == build.source_hash()
    monkeypatch.setattr(build, "FLAGS", build.FLAGS + ["-DOTHER"])
    assert build.source_hash() != h


def test_fallback_folder_is_per_user_and_per_sources():
    d = build._fallback_dir()
    assert str(os.getuid()) in d.name and build.source_hash() in d.name


def test_stamp_lies_beside_the_library(tmp_path):
    assert build._stamp_of(tmp_path / build.LIB_NAME) == tmp_path / "libminiserve_gfx950.stamp"


def test_no_kernel_spills_registers_to_memory():
    """The compiler's own report for every kernel of the library: none keeps registers in scratch memory (a spill
    in a decode kernel has doubled its time before it was seen) and none asks for more static LDS than a block
    may have.  Compiles the device code of all sources (about 20 s); skipped where there is no hipcc."""
    import pytest

    try:
        build._hipcc()
    except build.KernelLibraryError:
        pytest.skip("no hipcc here")
    usage = build.resource_usage()
    assert len(usage) > 100
    spills = {k: v["scratch"] for k, v in usage.items() if v.get("scratch", 0) > 0}
    assert not spills, f"kernels that spill registers: {spills}"
    assert all(v.get("lds", 0) <= 64 * 1024 for v in usage.values())


def test_a_library_older_than_its_sources_is_built_again_not_loaded(tmp_path, monkeypatch):
    """``load()`` with a stamp that names other sources calls ``build()`` and loads what that returns."""
    import ctypes

    old = tmp_path / build.LIB_NAME
    old.write_bytes(b"not a library")
    build._stamp_of(old).write_text("0123456789ab\n")
    fresh = tmp_path / "fresh" / build.LIB_NAME
    calls, loaded = [], []

    def fake_build(verbose=True):
        calls.append(1)
        return fresh

    monkeypatch.setattr(build, "_lib", None)
    monkeypatch.setattr(build, "library_path", lambda: old)
    monkeypatch.setattr(build, "build", fake_build)
    monkeypatch.setattr(ctypes, "CDLL", lambda p: loaded.append(p) or object())
    build.load()
    assert calls == [1] and loaded == [str(fresh)]
    # a stamp that names these sources: loaded as it is
    build._stamp_of(old).write_text(build.source_hash() + "\n")
    monkeypatch.setattr(build, "_lib", None)
    build.load()
    assert calls == [1] and loaded[-1] == str(old)
    monkeypatch.setattr(build, "_lib", None)
