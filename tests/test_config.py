import json

import pytest

from llmserve.config import (ARCHITECTURES, ConfigError, EngineConfig, LlamaConfig, architecture_of, preset,
                             read_config)
from conftest import TINY_A, TINY_B


def test_defaults_follow_the_reference():
    cfg = LlamaConfig.from_dict(dict(vocab_size=100, hidden_size=64, intermediate_size=128,
                                     num_hidden_layers=2, num_attention_heads=4))
    assert cfg.num_key_value_heads == 4 and cfg.head_dim == 16
    assert cfg.max_position_embeddings == 2048 and cfg.rope_theta == 10000.0 and cfg.rms_norm_eps == 1e-5
    assert cfg.attention_bias is False and cfg.tie_word_embeddings is False


def test_reads_every_key_it_is_given():
    for raw in (TINY_A, TINY_B):
        cfg = LlamaConfig.from_dict(raw)
        assert cfg.vocab_size == raw["vocab_size"] and cfg.hidden_size == raw["hidden_size"]
        assert cfg.intermediate_size == raw["intermediate_size"] and cfg.num_hidden_layers == raw["num_hidden_layers"]
        assert cfg.num_attention_heads == raw["num_attention_heads"]
        assert cfg.num_key_value_heads == raw["num_key_value_heads"]
        assert cfg.rope_theta == raw["rope_theta"] and cfg.rms_norm_eps == raw["rms_norm_eps"]
        assert cfg.max_position_embeddings == raw["max_position_embeddings"]
        assert cfg.tie_word_embeddings == raw["tie_word_embeddings"]
        assert LlamaConfig.from_dict(cfg.to_dict()) == cfg


def test_rope_theta_from_rope_parameters_and_head_dim_key():
    base = dict(vocab_size=10, hidden_size=64, intermediate_size=8, num_hidden_layers=1, num_attention_heads=4)
    assert LlamaConfig.from_dict(dict(base, rope_parameters={"rope_theta": 5e5})).rope_theta == 5e5
    assert LlamaConfig.from_dict(dict(base, head_dim=16)).head_dim == 16  # the key may be there if it says the same
    with pytest.raises(ConfigError, match="head_dim=32 differs"):
        LlamaConfig.from_dict(dict(base, head_dim=32))  # the reference always derives hidden // heads
    with pytest.raises(ConfigError, match="not a multiple of num_attention_heads"):
        LlamaConfig.from_dict(dict(base, hidden_size=66))


def test_missing_and_bad_values_are_named():
    with pytest.raises(ConfigError, match="intermediate_size"):
        LlamaConfig.from_dict(dict(vocab_size=10, hidden_size=64, num_hidden_layers=1, num_attention_heads=4))
    base = dict(vocab_size=10, hidden_size=64, intermediate_size=8, num_hidden_layers=1, num_attention_heads=4)
    with pytest.raises(ConfigError, match="multiple"):
        LlamaConfig.from_dict(dict(base, num_key_value_heads=3))
    with pytest.raises(ConfigError, match="even"):
        LlamaConfig.from_dict(dict(base, hidden_size=60, num_attention_heads=4, head_dim=15))
    with pytest.raises(NotImplementedError, match="rope_scaling"):
        LlamaConfig.from_dict(dict(base, rope_scaling={"rope_type": "llama3", "factor": 8.0}))
    LlamaConfig.from_dict(dict(base, rope_scaling={"rope_type": "default"}))
    with pytest.raises(NotImplementedError, match="hidden_act"):
        LlamaConfig.from_dict(dict(base, hidden_act="gelu"))
    with pytest.raises(NotImplementedError, match="mlp_bias"):
        LlamaConfig.from_dict(dict(base, mlp_bias=True))


def test_presets_have_the_published_sizes():
    from llmserve.parts.model import Model
    from llmserve.parts.registry import BuildContext
    import math
    import torch

    arch = architecture_of(preset("tinyllama-1.1b"))
    model = Model(arch.build_spec(LlamaConfig.from_dict(preset("tinyllama-1.1b"))),
                  BuildContext(torch.bfloat16, torch.device("cpu")))
    assert sum(math.prod(i.shape) for i in model.param_infos().values()) == 1_100_048_384
    assert LlamaConfig.from_dict(preset("llama2-70b")).head_dim == 128
    with pytest.raises(ConfigError, match="unknown preset"):
        preset("nope")


def test_presets_belong_to_the_architecture_that_registers_them():
    """Named sizes come with an architecture's registration; nothing in the framework lists them by hand."""
    from llmserve.config import is_preset, preset_names, register_architecture

    assert {"tiny", "tinyllama-1.1b", "llama2-7b", "llama2-70b"} <= set(preset_names())
    assert preset("TinyLlama_1.1B")["architectures"] == ["LlamaForCausalLM"] and preset("tiny")["model_type"] == "llama"
    register_architecture("PresetProbeForCausalLM", LlamaConfig, lambda cfg: None, model_type="preset_probe",
                          presets={"probe-small": dict(vocab_size=7, hidden_size=16)})
    try:
        assert is_preset("probe_small") and "probe-small" in preset_names()
        got = preset("probe-small")
        assert got == dict(vocab_size=7, hidden_size=16, architectures=["PresetProbeForCausalLM"], model_type="preset_probe")
        assert architecture_of(got).name == "PresetProbeForCausalLM"
    finally:
        ARCHITECTURES.pop("PresetProbeForCausalLM")
    assert not is_preset("probe-small")


def test_registry_picks_the_model_by_config(tmp_path):
    assert "LlamaForCausalLM" in ARCHITECTURES
    assert architecture_of({"architectures": ["LlamaForCausalLM"]}).name == "LlamaForCausalLM"
    assert architecture_of({"model_type": "llama"}).name == "LlamaForCausalLM"
    with pytest.raises(KeyError, match="registered"):
        architecture_of({"architectures": ["MambaForCausalLM"]})
    with pytest.raises(KeyError, match="names no architecture"):
        architecture_of({})
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    arch, cfg, raw = read_config(tmp_path)
    assert arch.name == "LlamaForCausalLM" and cfg.num_key_value_heads == 1 and raw == TINY_B
    with pytest.raises(FileNotFoundError):
        read_config(tmp_path / "missing")


def test_spec_is_data_per_layer():
    arch = architecture_of(TINY_B)
    spec = arch.build_spec(LlamaConfig.from_dict(TINY_B))
    assert len(spec.layers) == 3 and spec.schedule == (0, 1, 2)
    layer = spec.layers[1]
    assert layer.mixer.kind == "attention" and layer.mixer["num_kv_heads"] == 1 and layer.mixer["head_dim"] == 32
    assert layer.mixer["position"].kind == "rope" and layer.mixer["position"]["theta"] == 500000.0
    assert set(layer.parts) == set(layer.weights) == {"mixer", "feed_forward", "mixer_norm", "feed_forward_norm"}
    assert layer.parts["feed_forward"].kind == "swiglu" and layer.parts["feed_forward"]["intermediate"] == 256
    assert layer.parts["mixer_norm"]["eps"] == 1e-6 and layer.weights["mixer"] == "model.layers.1.self_attn."
    assert spec.head["tied"] is True


def test_engine_config_validation():
    EngineConfig().validate()
    for bad in (dict(dtype="float16"), dict(block_size=0), dict(num_blocks=0), dict(max_num_seqs=0)):
        with pytest.raises(ValueError):
            EngineConfig(**bad).validate()


def test_a_length_limit_beyond_the_models_positions_is_refused():
    """src/llmserve/utils.py:8-13 of the reference refuses it; so does the runner, before it takes any memory."""
    import torch

    from llmserve.engine.runner import ModelRunner
    from llmserve.parts.model import Model
    from llmserve.parts.registry import BuildContext

    arch = architecture_of(TINY_B)
    cfg = LlamaConfig.from_dict(TINY_B)
    model = Model(arch.build_spec(cfg), BuildContext(torch.float32, torch.device("cpu")))
    limit = TINY_B["max_position_embeddings"]
    with pytest.raises(ValueError, match=f"more than the model's {limit} positions"):
        ModelRunner(model, cfg, EngineConfig(dtype="float32", max_model_len=limit + 1, num_blocks=4), torch.device("cpu"))
