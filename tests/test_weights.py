import json

import pytest
import torch
from safetensors.torch import load_file, save_file

from llmserve.config import architecture_of
from llmserve.parts.model import Model
from llmserve.parts.registry import BuildContext
from llmserve.weights import WeightError, index_folder, load_tensors, random_tensor, write_random_model
from conftest import TINY_A, TINY_B


def _infos(cfg):
    arch = architecture_of(cfg)
    model = Model(arch.build_spec(arch.config_class.from_dict(cfg)), BuildContext(torch.float32, torch.device("cpu")))
    return model, model.param_infos()


def test_random_folder_round_trip(tmp_path):
    write_random_model(tmp_path, TINY_A, seed=3)
    assert json.loads((tmp_path / "config.json").read_text())["hidden_size"] == 64
    model, infos = _infos(TINY_A)
    names = set(index_folder(tmp_path))
    assert names == set(infos)
    assert "model.layers.1.self_attn.k_proj.weight" in names and "lm_head.weight" in names
    tensors = load_tensors(tmp_path, infos, torch.float32, "cpu")
    on_disk = load_file(str(tmp_path / "model.safetensors"))
    assert all(torch.equal(tensors[n], on_disk[n]) for n in infos)
    assert tensors["model.layers.0.mlp.gate_proj.weight"].shape == (176, 64)
    b16 = load_tensors(tmp_path, infos, torch.bfloat16, "cpu")
    assert all(t.dtype == torch.bfloat16 for t in b16.values())


def test_random_weights_are_seeded_per_tensor(tmp_path):
    _, infos = _infos(TINY_A)
    name = "model.layers.1.mlp.down_proj.weight"
    a = random_tensor(name, infos[name], 5, torch.float32)
    assert torch.equal(a, random_tensor(name, infos[name], 5, torch.float32))
    assert not torch.equal(a, random_tensor(name, infos[name], 6, torch.float32))
    assert not torch.equal(a[:, :64], random_tensor("model.layers.0.mlp.down_proj.weight", infos[name], 5, torch.float32)[:, :64])
    assert abs(float(a.std()) - 0.02) < 0.002
    norm = random_tensor("model.norm.weight", infos["model.norm.weight"], 5, torch.float32)
    assert abs(float(norm.mean()) - 1.0) < 0.01 and float(norm.std()) > 0


def test_a_part_brings_its_own_initializer():
    """A tensor that is neither a matrix nor a norm weight (a decay in (0.9, 1), say) is filled by a function
    the part registers under a name, or hands over itself: the weights package is not edited."""
    from llmserve.parts.spec import ParamInfo
    from llmserve.weights import INITIALIZERS, random_tensors, register_initializer

    @register_initializer("decay_probe")
    def decay(shape, generator, device, options):
        return 0.9 + 0.1 * torch.rand(shape, generator=generator, dtype=torch.float32, device=device)

    try:
        infos = {"a.decay": ParamInfo((5, 3), "decay_probe"),
                 "a.taps": ParamInfo((4,), lambda shape, g, dev, opt: torch.arange(4.0) * opt["std"]),
                 "a.proj": ParamInfo((3, 3))}
        t = random_tensors(infos, 9, torch.float32, std=0.5)
        assert (t["a.decay"] >= 0.9).all() and (t["a.decay"] < 1.0).all() and t["a.decay"].unique().numel() > 1
        assert torch.equal(t["a.taps"], torch.tensor([0.0, 0.5, 1.0, 1.5]))
        assert torch.equal(t["a.decay"], random_tensors(infos, 9, torch.float32)["a.decay"])  # seeded like the rest
    finally:
        INITIALIZERS.pop("decay_probe")
    with pytest.raises(ValueError, match="no initializer named 'decay_probe'"):
        random_tensors({"a.decay": ParamInfo((5, 3), "decay_probe")}, 9, torch.float32)
    with pytest.raises(ValueError, match="made shape"):
        random_tensors({"x": ParamInfo((2, 2), lambda shape, g, dev, opt: torch.zeros(3))}, 1, torch.float32)


def test_tied_model_has_no_head_tensor_and_ignores_one(tmp_path):
    write_random_model(tmp_path, TINY_B, seed=1)
    model, infos = _infos(TINY_B)
    assert "lm_head.weight" not in infos and "lm_head.weight" not in index_folder(tmp_path)
    t = load_file(str(tmp_path / "model.safetensors"))
    t["lm_head.weight"] = torch.zeros(333, 96)
    save_file(t, str(tmp_path / "model.safetensors"))
    load_tensors(tmp_path, infos, torch.float32, "cpu", ignore={"lm_head.weight"})
    with pytest.raises(WeightError, match="unexpected"):
        load_tensors(tmp_path, infos, torch.float32, "cpu")


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    write_random_model(tmp_path, TINY_A, seed=2)
    _, infos = _infos(TINY_A)
    t = load_file(str(tmp_path / "model.safetensors"))
    del t["model.layers.0.self_attn.q_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.qkv.weight"] = torch.zeros(2, 2)
    t["model.layers.1.mlp.up_proj.weight"] = torch.zeros(64, 176)
    t["model.layers.1.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)  # legacy buffer: skipped
    save_file(t, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightError) as e:
        load_tensors(tmp_path, infos, torch.float32, "cpu")
    assert e.value.missing == ["model.layers.0.self_attn.q_proj.weight", "model.norm.weight"]
    assert e.value.unexpected == ["model.layers.0.self_attn.qkv.weight"]
    assert e.value.wrong_shape == ["model.layers.1.mlp.up_proj.weight"]
    text = str(e.value)
    for part in ("missing (2)", "unexpected (1)", "wrong shape (1)", "file [64, 176] model [176, 64]"):
        assert part in text


def test_sharded_folder_and_missing_files(tmp_path):
    write_random_model(tmp_path, TINY_A, seed=4)
    _, infos = _infos(TINY_A)
    t = load_file(str(tmp_path / "model.safetensors"))
    names = sorted(t)
    (tmp_path / "model.safetensors").unlink()
    save_file({n: t[n] for n in names[:7]}, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file({n: t[n] for n in names[7:]}, str(tmp_path / "model-00002-of-00002.safetensors"))
    got = load_tensors(tmp_path, infos, torch.float32, "cpu")
    assert all(torch.equal(got[n], t[n]) for n in names)
    empty = tmp_path / "empty"
    empty.mkdir()
    with pytest.raises(FileNotFoundError, match="no .safetensors"):
        index_folder(empty)


def test_stored_dtype_rule(tmp_path):
    from llmserve.parts.spec import ParamInfo

    save_file({"a": torch.ones(2, 2), "b": torch.ones(2, 2), "t": torch.arange(4, dtype=torch.int64)},
              str(tmp_path / "model.safetensors"))
    wanted = {"a": ParamInfo((2, 2)), "b": ParamInfo((2, 2), dtype="stored"), "t": ParamInfo((4,), dtype="stored")}
    got = load_tensors(tmp_path, wanted, torch.bfloat16, "cpu")
    assert got["a"].dtype == torch.bfloat16 and got["b"].dtype == torch.float32 and got["t"].dtype == torch.int32
