"""Import name of the engine.

The sources live in the folder ``llmserve-triton-kernels_amd`` beside this one; that
folder's name is not a Python identifier, so this package maps its own submodule
search path onto it: ``import llmserve.engine`` loads
``llmserve-triton-kernels_amd/engine``, and ``python -m llmserve.cli`` is the command line.
"""

import os as _os

_SOURCE_DIR = _os.path.join(
    _os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))), "llmserve-triton-kernels_amd"
)
__path__ = [_SOURCE_DIR]

_EXPORTS = {
    "LLM": ("llmserve.engine.llm", "LLM"),
    "EngineConfig": ("llmserve.config", "EngineConfig"),
    "SamplingParams": ("llmserve.sampling", "SamplingParams"),
    "GenerationResult": ("llmserve.engine.request", "GenerationResult"),
}


def __getattr__(name):
    if name in _EXPORTS:
        import importlib

        module, attr = _EXPORTS[name]
        return getattr(importlib.import_module(module), attr)
    raise AttributeError(f"module 'llmserve' has no attribute {name!r}")
