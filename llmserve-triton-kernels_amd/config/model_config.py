"""Typed model configuration read from the architecture's own config.json keys.

Keys and defaults follow the reference's ``ModelConfig.from_hf_dict``
(src/llmserve/config.py:39-61): the five sizes are required, the rest default to
num_key_value_heads = heads, max_position_embeddings = 2048, rope_theta = 10000.0
(also read from rope_parameters.rope_theta), rms_norm_eps = 1e-5, attention_bias = False,
tie_word_embeddings = False; a non-default rope_scaling is rejected
(src/llmserve/config.py:41-46).  Options the reference silently ignores and this engine
does not implement (hidden_act other than silu, mlp_bias) are rejected by name.
"""

from __future__ import annotations

import json
from dataclasses import asdict, dataclass, field
from pathlib import Path


class ConfigError(ValueError):
    """config.json is missing a key, has an impossible value or asks for an unsupported option."""


_REQUIRED = ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads")


@dataclass(frozen=True)
class LlamaConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    attention_bias: bool
    tie_word_embeddings: bool
    architectures: tuple[str, ...] = field(default=("LlamaForCausalLM",))

    # -- reading ---------------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: dict) -> "LlamaConfig":
        missing = [k for k in _REQUIRED if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks required keys {missing}")
        rs = d.get("rope_scaling")
        if rs and rs.get("rope_type", rs.get("type")) not in (None, "default"):
            raise NotImplementedError(f"rope_scaling={rs!r} is not supported")
        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise NotImplementedError(f"hidden_act={act!r} is not supported (only 'silu')")
        if d.get("mlp_bias", False):
            raise NotImplementedError("mlp_bias=true is not supported")
        rope_theta = d.get("rope_theta") or (d.get("rope_parameters") or {}).get("rope_theta", 10000.0)
        heads = int(d["num_attention_heads"])
        hidden = int(d["hidden_size"])
        if heads <= 0:
            raise ConfigError(f"num_attention_heads={heads} must be positive")
        # src/llmserve/config.py:22-24: head_dim = hidden_size // num_heads, always; a config.json that names
        # another head_dim describes a model the reference cannot hold, and is refused rather than guessed at
        head_dim = hidden // heads
        if d.get("head_dim") is not None and int(d["head_dim"]) != head_dim:
            raise ConfigError(f"head_dim={d['head_dim']} differs from hidden_size // num_attention_heads = {head_dim}; "
                              "the Llama decoder here takes head_dim from those two")
        if hidden % heads:
            raise ConfigError(f"hidden_size={hidden} is not a multiple of num_attention_heads={heads}")
        cfg = cls(
            vocab_size=int(d["vocab_size"]),
            hidden_size=hidden,
            intermediate_size=int(d["intermediate_size"]),
            num_hidden_layers=int(d["num_hidden_layers"]),
            num_attention_heads=heads,
            num_key_value_heads=int(d.get("num_key_value_heads") or heads),
            head_dim=int(head_dim),
            max_position_embeddings=int(d.get("max_position_embeddings", 2048)),
            rope_theta=float(rope_theta),
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-5)),
            attention_bias=bool(d.get("attention_bias", False)),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            architectures=tuple(d.get("architectures") or ("LlamaForCausalLM",)),
        )
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, path: str | Path) -> "LlamaConfig":
        path = Path(path)
        if path.is_dir():
            path = path / "config.json"
        return cls.from_dict(json.loads(path.read_text()))

    def validate(self) -> None:
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                     "num_attention_heads", "num_key_value_heads", "head_dim", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name}={getattr(self, name)} must be positive")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads={self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads={self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim={self.head_dim} must be even for the rotary pairing")
        if self.rms_norm_eps <= 0 or self.rope_theta <= 0:
            raise ConfigError("rms_norm_eps and rope_theta must be positive")

    # -- writing ---------------------------------------------------------------------
    def to_dict(self) -> dict:
        """The config.json form (what `from_dict` reads back to the same object)."""
        d = asdict(self)
        d["architectures"] = list(self.architectures)
        d["model_type"] = "llama"
        d["hidden_act"] = "silu"
        return d


# Named sizes of the Llama architecture, as config.json dictionaries (models/llama.py registers them with the
# architecture; `config.preset(name)` finds them).  "tiny" is the reference's own test
# configuration (src/llmserve/config.py:26-37); the others are the shapes this engine
# is tested and measured on.
LLAMA_PRESETS: dict[str, dict] = {
    "tiny": dict(vocab_size=256, hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                 num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=512),
    "tiny-a": dict(vocab_size=256, hidden_size=64, intermediate_size=176, num_hidden_layers=2,
                   num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=128,
                   rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False),
    "tiny-b": dict(vocab_size=333, hidden_size=96, intermediate_size=256, num_hidden_layers=3,
                   num_attention_heads=3, num_key_value_heads=1, max_position_embeddings=256,
                   rope_theta=500000.0, rms_norm_eps=1e-6, tie_word_embeddings=True),
    "tinyllama-1.1b": dict(vocab_size=32000, hidden_size=2048, intermediate_size=5632,
                           num_hidden_layers=22, num_attention_heads=32, num_key_value_heads=4,
                           max_position_embeddings=2048, rope_theta=10000.0, rms_norm_eps=1e-5),
    "llama2-7b": dict(vocab_size=32000, hidden_size=4096, intermediate_size=11008,
                      num_hidden_layers=32, num_attention_heads=32, num_key_value_heads=32,
                      max_position_embeddings=4096, rope_theta=10000.0, rms_norm_eps=1e-5),
    "llama2-70b": dict(vocab_size=32000, hidden_size=8192, intermediate_size=28672,
                       num_hidden_layers=80, num_attention_heads=64, num_key_value_heads=8,
                       max_position_embeddings=4096, rope_theta=10000.0, rms_norm_eps=1e-5),
}

