"""The kernel build: library names carry a hash of sources and flags, and compiling one source
removes only that source's older libraries."""

import shutil

import pytest

from llmserve.ops import build


@pytest.mark.skipif(shutil.which("hipcc") is None and not build.Path("/opt/rocm/bin/hipcc").exists(),
                    reason="hipcc is needed to compile")
def test_compiling_one_source_leaves_the_libraries_of_others(tmp_path):
    old_own = tmp_path / "libllms_gemm_000000000000.so"
    other = tmp_path / "libllms_gemm_stream_0123456789ab.so"  # another source whose name starts the same
    unrelated = tmp_path / "libllms_gemm_notes.so"
    for f in (old_own, other, unrelated):
        f.write_bytes(b"x")
    messages = []
    final = build._compile("gemm", tmp_path, messages.append)
    assert final.exists() and final.name == f"libllms_gemm_{build._source_hash('gemm')}.so"
    assert not old_own.exists()
    assert other.exists() and unrelated.exists()
    assert any("gemm.hip ->" in m for m in messages)


def test_library_names_change_with_the_flags(monkeypatch):
    before = build._source_hash("gemm")
    monkeypatch.setattr(build, "HIPCC_FLAGS", build.HIPCC_FLAGS + ["-DX=1"])
    assert build._source_hash("gemm") != before


def test_library_names_follow_the_headers_a_source_includes(tmp_path, monkeypatch):
    """A header counts for the sources that include it, directly or through another header, and for no other: a
    change to one kernel's header must not make every built library stale."""
    (tmp_path / "common.h").write_text("#pragma once\n")
    (tmp_path / "wide.h").write_text('#include "deep.h"\n')
    (tmp_path / "deep.h").write_text("// deep\n")
    (tmp_path / "one.hip").write_text('#include "common.h"\n#include "wide.h"\n#include <vector>\n')
    (tmp_path / "two.hip").write_text('  #  include "common.h"\n')
    monkeypatch.setattr(build, "CSRC_DIR", tmp_path)
    assert [p.name for p in build._inputs("one")] == ["common.h", "deep.h", "one.hip", "wide.h"]
    assert [p.name for p in build._inputs("two")] == ["common.h", "two.hip"]
    one, two = build._source_hash("one"), build._source_hash("two")
    (tmp_path / "deep.h").write_text("// deeper\n")
    assert build._source_hash("one") != one and build._source_hash("two") == two
    (tmp_path / "common.h").write_text("#pragma once\n// more\n")
    assert build._source_hash("two") != two
