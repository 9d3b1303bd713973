"""Reads a model folder's tensors by name.

As the reference (src/llmserve/weights.py:24-57): every ``*.safetensors`` file of the
folder, sorted by name, forms one table of tensors; entries ending in
``rotary_emb.inv_freq`` are skipped; the names are the checkpoint's own, nothing is
renamed; a tied output head needs no tensor of its own.  Unlike the reference the folder
is first checked as a whole, from the file headers alone: one `WeightError` lists every
missing tensor, every unexpected tensor and every wrong shape; only then are the tensors
read, one at a time, and copied to the device.

Storage: a tensor whose `ParamInfo.dtype` is "model" is cast to the engine's dtype
(bfloat16 or float32); "stored" keeps what the file holds (a 32-bit tensor stays 32-bit,
an integer table becomes int32).
"""

from __future__ import annotations

import json
import struct
from pathlib import Path

import torch

from ..parts.spec import ParamInfo

_SKIP_SUFFIX = "rotary_emb.inv_freq"


class WeightError(RuntimeError):
    """The folder's tensors are not the model's: lists missing, unexpected and misshapen ones."""

    def __init__(self, message: str, missing=(), unexpected=(), wrong_shape=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)


def _read_header(path: Path) -> dict:
    """The JSON header of a safetensors file: 8 bytes little-endian length, then JSON
    name -> {dtype, shape, data_offsets}."""
    with open(path, "rb") as f:
        raw = f.read(8)
        if len(raw) != 8:
            raise WeightError(f"{path} is not a safetensors file (too short)")
        (n,) = struct.unpack("<Q", raw)
        if n > 100 * 2**20:
            raise WeightError(f"{path} is not a safetensors file (header of {n} bytes)")
        header = json.loads(f.read(n))
    header.pop("__metadata__", None)
    return header


def index_folder(model_dir: str | Path) -> dict[str, tuple[Path, tuple[int, ...], str]]:
    """name -> (file, shape, stored dtype) over all safetensors files of the folder."""
    model_dir = Path(model_dir)
    files = sorted(model_dir.glob("*.safetensors"))
    if not files:
        raise FileNotFoundError(f"no .safetensors files found in {model_dir}")
    index: dict[str, tuple[Path, tuple[int, ...], str]] = {}
    for f in files:
        for name, meta in _read_header(f).items():
            if name.endswith(_SKIP_SUFFIX):
                continue
            index[name] = (f, tuple(meta["shape"]), meta["dtype"])
    return index


def check_folder(index: dict, wanted: dict[str, ParamInfo], ignore: set[str] = frozenset()) -> None:
    missing = sorted(n for n in wanted if n not in index)
    unexpected = sorted(n for n in index if n not in wanted and n not in ignore)
    wrong = sorted((n, index[n][1], tuple(wanted[n].shape)) for n in wanted
                   if n in index and tuple(index[n][1]) != tuple(wanted[n].shape))
    if missing or unexpected or wrong:
        lines = ["checkpoint does not match the model:"]
        if missing:
            lines.append(f"  missing ({len(missing)}): {missing}")
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): {unexpected}")
        if wrong:
            lines.append(f"  wrong shape ({len(wrong)}): " +
                         ", ".join(f"{n}: file {list(a)} model {list(b)}" for n, a, b in wrong))
        raise WeightError("\n".join(lines), missing, unexpected, [w[0] for w in wrong])


def _storage_dtype(t: torch.Tensor, info: ParamInfo, model_dtype: torch.dtype) -> torch.dtype:
    if not t.dtype.is_floating_point:
        return torch.int32
    if info.dtype == "stored":
        return torch.float32 if t.dtype in (torch.float32, torch.float64) else t.dtype
    return model_dtype


def load_tensors(model_dir: str | Path, wanted: dict[str, ParamInfo], model_dtype: torch.dtype,
                 device: torch.device | str, ignore: set[str] = frozenset()) -> dict[str, torch.Tensor]:
    """The tensors `wanted` names, on `device`.  `ignore`: names that may be present without
    being used (the output head of a tied model)."""
    from safetensors import safe_open

    index = index_folder(model_dir)
    check_folder(index, wanted, ignore)
    by_file: dict[Path, list[str]] = {}
    for name in wanted:
        by_file.setdefault(index[name][0], []).append(name)
    out: dict[str, torch.Tensor] = {}
    for f, names in by_file.items():
        with safe_open(str(f), framework="pt", device="cpu") as sf:
            for name in names:
                t = sf.get_tensor(name)
                out[name] = t.to(device=device, dtype=_storage_dtype(t, wanted[name], model_dtype))
    return out
