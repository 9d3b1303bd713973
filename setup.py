"""Packaging: the folder `llmserve-triton-kernels_amd/` (no Python identifier) is installed as the package
`llmserve`, with its kernel sources, which are compiled for gfx950 at first use (or beforehand:
`python -c "import __graft_entry__ as g; g.build()"` in a checkout)."""

from setuptools import setup

SUBPACKAGES = ["cache", "config", "engine", "models", "ops", "parts", "sampling", "weights"]

setup(
    name="llmserve-amd",
    version="0.2.0",
    description="A small, whole Llama inference engine for one MI355X: paged KV cache, continuous batching, "
                "hand-written HIP kernels.",
    python_requires=">=3.10",
    packages=["llmserve"] + [f"llmserve.{name}" for name in SUBPACKAGES],
    package_dir={"llmserve": "llmserve-triton-kernels_amd"},
    package_data={"llmserve": ["csrc/*.hip", "csrc/*.h"]},
    install_requires=["torch", "numpy", "safetensors"],
    extras_require={"text": ["transformers"], "dev": ["pytest", "hypothesis", "pytest-timeout"]},
    entry_points={"console_scripts": ["llmserve-gen = llmserve.cli:main",
                                      "llmserve-trace-run = llmserve.engine.replay:main"]},
)
