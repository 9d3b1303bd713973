"""The installable face of the engine: setup.py names every subpackage of the source folder, and the console
scripts (the reference's `llmserve-gen`, pyproject.toml:35-36 there) point at functions that exist."""

import importlib
import os
import re

from conftest import ROOT

SOURCE = os.path.join(ROOT, "llmserve-triton-kernels_amd")


def test_setup_lists_every_subpackage():
    text = open(os.path.join(ROOT, "setup.py")).read()
    listed = set(re.search(r"SUBPACKAGES = \[(.*?)\]", text, re.S).group(1).replace('"', "").replace(" ", "").split(","))
    present = {name for name in os.listdir(SOURCE)
               if os.path.isfile(os.path.join(SOURCE, name, "__init__.py"))}
    assert listed == present


def test_console_scripts_point_at_callables():
    text = open(os.path.join(ROOT, "setup.py")).read()
    targets = re.findall(r'"([\w-]+) = ([\w.]+):(\w+)"', text)
    assert {name for name, _, _ in targets} == {"llmserve-gen", "llmserve-trace-run"}
    for _, module, function in targets:
        assert callable(getattr(importlib.import_module(module), function))


def test_top_level_names():
    import llmserve

    for name in ("LLM", "EngineConfig", "SamplingParams", "GenerationResult"):
        assert getattr(llmserve, name).__name__ == name


def test_bench_refuses_more_than_one_gpu_with_one_line():
    """The measurement program runs one GPU: asked for more it says so in one line and exits with 2, before it
    touches a device."""
    import subprocess
    import sys

    done = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                          capture_output=True, text=True, timeout=120)
    assert done.returncode == 2
    assert len(done.stdout.strip().splitlines()) == 1 and "--gpus 2" in done.stdout
