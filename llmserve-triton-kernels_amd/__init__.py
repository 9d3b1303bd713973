"""The `llmserve` package: a Llama inference engine for one MI355X.

From a checkout it is imported through the small package `llmserve/` beside this folder (whose own name is
not a Python identifier); installed (`pip install .`), this folder is the package itself.  Either way the
names below are at the top: `from llmserve import LLM, EngineConfig, SamplingParams`.
"""

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
