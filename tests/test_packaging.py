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
