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
