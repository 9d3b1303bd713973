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


@pytest.mark.skipif(shutil.which("hipcc") is None and not build.Path("/opt/rocm/bin/hipcc").exists(),
                    reason="hipcc is needed to compile")
@pytest.mark.parametrize("name,kernels,most_bytes", [
    ("gemm_stream", ("gemm_stream_kernel", "gemm_slices_kernel"), 0),
    ("attention_mfma", ("attn_prompt_kernel", "attn_mfma_kernel"), 64),
    ("gemm_decode", ("gemm_decode_kernel", "gemm_decode_rows_kernel"), 128),
])
def test_streaming_kernels_hold_what_they_fetch_in_registers(tmp_path, name, kernels, most_bytes):
    """What a lane has fetched and not yet used must stay in registers.  The compiler may lower an array of a
    struct (uint4) that one place fills and another empties to copies through the lane's private memory, which puts
    a wait behind every load: twice the time, and no numerics test sees it.  The kernels' private segment (in the
    code object's metadata) is empty, or holds the few registers spilt by the kernels that are compiled for two
    workgroups per CU or that keep 64 rows of X in registers."""
    import re
    import subprocess

    flags = [f for f in build.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    out = tmp_path / f"{name}.s"
    subprocess.run([build._hipcc(), *flags, f"-I{build.CSRC_DIR}", "-S", "--cuda-device-only",
                    str(build.CSRC_DIR / f"{name}.hip"), "-o", str(out)], check=True, capture_output=True, timeout=600)
    text = out.read_text()
    sizes = {}
    for block in text.split("  - .agpr_count:")[1:]:  # one block of metadata per kernel
        kernel = re.search(r"\.name:\s+(\S+)", block).group(1)
        sizes[kernel] = int(re.search(r"\.private_segment_fixed_size:\s+(\d+)", block).group(1))
    checked = {k: v for k, v in sizes.items() if any(want in k for want in kernels)}
    assert checked, sorted(sizes)
    assert {k: v for k, v in checked.items() if v > most_bytes} == {}
