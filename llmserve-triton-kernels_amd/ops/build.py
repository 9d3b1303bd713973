"""Compiles the HIP sources under ``csrc/`` for gfx950 into shared libraries.

One source file becomes one library, named after the file and a hash of everything that
goes into it (the file, the headers of this folder it includes, the compiler flags).  A library whose hash
matches is loaded as it is; a missing or stale one is compiled at the first call that
needs it, so a fresh checkout works without a build step.  Libraries are written into
``lib/`` next to the sources; when that folder cannot be written, into a per-user folder
under the system's temporary directory (or ``LLMSERVE_BUILD_DIR``).
"""

from __future__ import annotations

import hashlib
import os
import re
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent.parent
CSRC_DIR = PACKAGE_DIR / "csrc"
LIB_DIR = PACKAGE_DIR / "lib"

ARCH = "gfx950"
# The target feature packed-fp32-ops is switched off for all device code.  Matrix instructions keep
# their accumulators in ordinary vector registers: the kernels here rescale and convert them between
# products, and the other register file would cost a copy each way.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "-shared", f"--offload-arch={ARCH}",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wno-unused-result", "-Wno-unknown-warning-option", "-Wno-pass-failed",
]

# Which libraries the step function of a model of a given dtype needs (the sampler's library is
# built when something is first sampled).
GROUPS = {
    "float32": ("elementwise", "gemm", "attention"),
    "bfloat16": ("elementwise", "gemm", "attention", "gemm_stream", "gemm_decode", "attention_mfma"),
}


class BuildError(RuntimeError):
    pass


def all_sources() -> list[str]:
    return sorted(p.stem for p in CSRC_DIR.glob("*.hip"))


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc); "
                     "the engine has no fallback without its compiled kernels")


_INCLUDE = re.compile(r'^\s*#\s*include\s+"([^"]+)"', re.MULTILINE)


def _inputs(name: str) -> list[Path]:
    """The source file and the headers of this folder it includes, directly or through one another."""
    found: dict[str, Path] = {}
    todo = [CSRC_DIR / f"{name}.hip"]
    while todo:
        path = todo.pop()
        if path.name in found or not path.exists():
            continue
        found[path.name] = path
        todo += [CSRC_DIR / inc for inc in _INCLUDE.findall(path.read_text(errors="replace"))]
    return [found[k] for k in sorted(found)]


def _source_hash(name: str) -> str:
    h = hashlib.sha256()
    h.update(" ".join(HIPCC_FLAGS).encode())
    for p in _inputs(name):
        h.update(p.name.encode())
        h.update(p.read_bytes())
    return h.hexdigest()[:12]


def _fallback_dir() -> Path:
    base = os.environ.get("LLMSERVE_BUILD_DIR")
    if base:
        return Path(base)
    return Path(tempfile.gettempdir()) / f"llmserve-build-{os.getuid()}"


def _writable_dir() -> Path:
    for d in (LIB_DIR, _fallback_dir()):
        try:
            d.mkdir(parents=True, exist_ok=True)
            probe = d / f".probe-{os.getpid()}"
            probe.write_bytes(b"")
            probe.unlink()
            return d
        except OSError:
            continue
    raise BuildError(f"no writable folder for compiled kernels (tried {LIB_DIR} and {_fallback_dir()})")


def library_path(name: str) -> Path | None:
    """Path of an up-to-date built library for source `name`, or None."""
    fname = f"libllms_{name}_{_source_hash(name)}.so"
    for d in (LIB_DIR, _fallback_dir()):
        p = d / fname
        if p.exists():
            return p
    return None


def _compile(name: str, out_dir: Path, log) -> Path:
    src = CSRC_DIR / f"{name}.hip"
    if not src.exists():
        raise BuildError(f"no kernel source {src}")
    final = out_dir / f"libllms_{name}_{_source_hash(name)}.so"
    tmp = out_dir / f".{final.name}.{os.getpid()}.{threading.get_ident()}.tmp"
    cmd = [_hipcc(), *HIPCC_FLAGS, f"-I{CSRC_DIR}", str(src), "-o", str(tmp)]
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    while True:
        try:
            output, _ = proc.communicate(timeout=20)
            break
        except subprocess.TimeoutExpired:
            log(f"[llmserve build] still compiling {name}.hip ({time.time() - t0:.0f} s)")
    if proc.returncode != 0:
        tmp.unlink(missing_ok=True)
        raise BuildError(f"hipcc failed on {src}:\n{output}")
    os.replace(tmp, final)  # atomic: a concurrent process sees either nothing or the whole file
    stale = re.compile(rf"libllms_{re.escape(name)}_[0-9a-f]{{12}}\.so")  # (not gemm_stream's when this is gemm)
    for old in out_dir.iterdir():
        if stale.fullmatch(old.name) and old != final:
            old.unlink(missing_ok=True)
    log(f"[llmserve build] {name}.hip -> {final.name} ({time.time() - t0:.0f} s)")
    return final


def build(names: list[str] | tuple[str, ...] | None = None, force: bool = False, verbose: bool = True) -> dict[str, Path]:
    """Make sure the libraries for `names` (default: all sources) exist; return their paths."""
    names = list(names) if names is not None else all_sources()

    def log(msg: str) -> None:
        if verbose:
            print(msg, file=sys.stderr, flush=True)

    result: dict[str, Path] = {}
    todo = []
    for n in names:
        p = None if force else library_path(n)
        if p is None:
            todo.append(n)
        else:
            result[n] = p
    if todo:
        out_dir = _writable_dir()
        log(f"[llmserve build] compiling {', '.join(todo)} for {ARCH} into {out_dir}")
        with ThreadPoolExecutor(max_workers=min(len(todo), 8)) as pool:
            for n, p in zip(todo, pool.map(lambda n: _compile(n, out_dir, log), todo)):
                result[n] = p
    return result
