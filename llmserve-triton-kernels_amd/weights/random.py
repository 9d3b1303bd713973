"""Random weights from a configuration and a seed, as tensors or as a model folder
(config.json + model.safetensors).

The reference's `random_model` (src/llmserve/weights.py:60-79) fills matrices with
N(0, 0.05), norm weights with 1 and the rest with 0 from one generator in module order.
Here every tensor has a stream of its own, keyed by (seed, tensor name), so any single
tensor can be regenerated alone and large models can be filled on the device tensor by
tensor; matrices are N(0, std), norm weights 1 + N(0, norm_std) so that a norm's weight is
not a vacuous 1, biases 0.
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path
from typing import Callable

import torch

from ..parts.spec import ParamInfo

# How a tensor is filled, by the name a part puts into `ParamInfo.init`.  A filler is
#     fill(shape, generator, device, options) -> float32 tensor
# with the tensor's own seeded generator and `options` = {"std": ..., "norm_std": ...} (the scales the caller of
# `random_tensors` chose).  A part with another kind of tensor (a decay in (0, 1), the taps of a convolution)
# registers a filler of its own, or puts the function itself into `ParamInfo.init`; this file is not edited.
INITIALIZERS: dict[str, Callable] = {}


def register_initializer(name: str, fill: Callable | None = None):
    def put(fn):
        INITIALIZERS[name] = fn
        return fn

    return put if fill is None else put(fill)


@register_initializer("matrix")
def _fill_matrix(shape, generator, device, options):
    return options["std"] * torch.randn(shape, generator=generator, dtype=torch.float32, device=device)


@register_initializer("norm")
def _fill_norm(shape, generator, device, options):
    return 1.0 + options["norm_std"] * torch.randn(shape, generator=generator, dtype=torch.float32, device=device)


@register_initializer("zeros")
def _fill_zeros(shape, generator, device, options):
    return torch.zeros(shape, dtype=torch.float32, device=device)


def _generator(seed: int, name: str, device) -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    g = torch.Generator(device=device)
    g.manual_seed(int.from_bytes(digest[:8], "little") & (2**63 - 1))
    return g


def random_tensor(name: str, info: ParamInfo, seed: int, dtype: torch.dtype, device="cpu",
                  std: float = 0.02, norm_std: float = 0.01) -> torch.Tensor:
    shape = tuple(info.shape)
    fill = info.init if callable(info.init) else INITIALIZERS.get(info.init)
    if fill is None:
        raise ValueError(f"{name}: no initializer named {info.init!r}; registered: {sorted(INITIALIZERS)}")
    t = fill(shape, _generator(seed, name, device), device, {"std": std, "norm_std": norm_std})
    if tuple(t.shape) != shape:
        raise ValueError(f"{name}: its initializer made shape {tuple(t.shape)}, not {shape}")
    return t.to(dtype)


def random_tensors(infos: dict[str, ParamInfo], seed: int, dtype: torch.dtype, device="cpu",
                   std: float = 0.02, norm_std: float = 0.01) -> dict[str, torch.Tensor]:
    return {name: random_tensor(name, info, seed, dtype, device, std, norm_std) for name, info in infos.items()}


def write_random_model(model_dir: str | Path, config: dict, seed: int = 0, dtype: torch.dtype = torch.float32,
                       std: float = 0.02, norm_std: float = 0.01) -> Path:
    """Write `config` as config.json and seeded random tensors as model.safetensors."""
    from safetensors.torch import save_file

    from ..config.registry import architecture_of
    from ..parts.model import Model
    from ..parts.registry import BuildContext

    model_dir = Path(model_dir)
    model_dir.mkdir(parents=True, exist_ok=True)
    arch = architecture_of(config)
    cfg = arch.config_class.from_dict(config)
    model = Model(arch.build_spec(cfg), BuildContext(dtype, torch.device("cpu")))
    tensors = random_tensors(model.param_infos(), seed, dtype, "cpu", std, norm_std)
    written = dict(config)
    written.setdefault("architectures", [arch.name])
    (model_dir / "config.json").write_text(json.dumps(written, indent=2) + "\n")
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(model_dir / "model.safetensors"))
    return model_dir
