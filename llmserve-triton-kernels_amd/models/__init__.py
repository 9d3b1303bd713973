"""Architectures: each module registers a name, a configuration class and a spec builder."""

from . import llama  # noqa: F401
