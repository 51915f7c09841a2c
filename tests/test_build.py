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
