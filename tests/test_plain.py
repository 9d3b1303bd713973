"""Pins of the plain implementation by what fixes it beside the reference's text: library
routines it must reduce to, invariants, and the vectors the reference's own tests hold."""

import math

import pytest
import torch
import torch.nn.functional as F

import plain_llama as pl
from conftest import TINY_A, TINY_B


def test_rms_norm_is_the_library_routine():
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(7, 96, generator=g), 1 + 0.1 * torch.randn(96, generator=g)
    for eps in (1e-5, 1e-6):
        assert torch.allclose(pl.rms_norm(x, w, eps), F.rms_norm(x, (96,), w, eps), atol=1e-6)


def test_rms_norm_scale_and_eps():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(3, 64, generator=g)
    one = torch.ones(64)
    y = pl.rms_norm(x, one, 1e-12)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(3), atol=1e-5)  # unit mean square
    assert torch.allclose(pl.rms_norm(5 * x, one, 1e-12), y, atol=1e-5)  # scale-free as eps -> 0
    tiny = 1e-3 * x
    assert not torch.allclose(pl.rms_norm(tiny, one, 1e-5), pl.rms_norm(tiny, one, 1e-6), atol=1e-3)  # eps counts


def test_rms_norm_weight_is_plain_not_one_plus():
    x = torch.randn(2, 8, generator=torch.Generator().manual_seed(2))
    assert torch.equal(pl.rms_norm(x, torch.zeros(8), 1e-5), torch.zeros(2, 8))


def test_rope_pairs_halves_with_the_right_sign():
    # D = 4, theta = 100: frequencies 1 and 0.1.  A unit vector along dimension 0 at position 1
    # turns into (cos 1, 0, sin 1, 0): dimension 0 pairs with 2 (not with 1), counter-clockwise.
    cos, sin = pl.rope_cos_sin(torch.tensor([1]), 4, 100.0)
    out = pl.apply_rope(torch.tensor([[[1.0, 0.0, 0.0, 0.0]]]), cos, sin)[0, 0]
    assert torch.allclose(out, torch.tensor([math.cos(1.0), 0.0, math.sin(1.0), 0.0]), atol=1e-6)
    out = pl.apply_rope(torch.tensor([[[0.0, 1.0, 0.0, 0.0]]]), cos, sin)[0, 0]
    assert torch.allclose(out, torch.tensor([0.0, math.cos(0.1), 0.0, math.sin(0.1)]), atol=1e-6)


def test_rope_is_complex_multiplication():
    g = torch.Generator().manual_seed(3)
    d, theta = 16, 500000.0
    x = torch.randn(2, 5, d, generator=g)
    pos = torch.tensor([0, 1, 7, 100, 250])
    cos, sin = pl.rope_cos_sin(pos, d, theta)
    out = pl.apply_rope(x, cos, sin)
    z = torch.complex(x[..., : d // 2].double(), x[..., d // 2:].double())
    freq = theta ** (-torch.arange(0, d, 2).double() / d)
    rot = torch.polar(torch.ones(5, d // 2, dtype=torch.float64), pos.double()[:, None] * freq)
    want = z * rot
    assert torch.allclose(out[..., : d // 2].double(), want.real, atol=1e-4)
    assert torch.allclose(out[..., d // 2:].double(), want.imag, atol=1e-4)
    assert torch.equal(out[:, 0], x[:, 0])  # position 0 is the identity


def test_rope_scores_depend_on_distance_only():
    g = torch.Generator().manual_seed(4)
    d = 32
    q, k = torch.randn(1, 1, d, generator=g), torch.randn(1, 1, d, generator=g)

    def score(m, n):
        cm, sm = pl.rope_cos_sin(torch.tensor([m]), d, 10000.0)
        cn, sn = pl.rope_cos_sin(torch.tensor([n]), d, 10000.0)
        return float((pl.apply_rope(q, cm, sm) * pl.apply_rope(k, cn, sn)).sum())

    assert abs(score(9, 4) - score(29, 24)) < 1e-4
    assert abs(score(9, 4) - score(9, 5)) > 1e-3


@pytest.mark.parametrize("nh,nkv", [(4, 2), (3, 1), (4, 4)])
def test_attention_is_library_sdpa(nh, nkv):
    g = torch.Generator().manual_seed(5)
    t, d = 11, 16
    q, k, v = (torch.randn(h, t, d, generator=g) for h in (nh, nkv, nkv))
    want = F.scaled_dot_product_attention(q[None], k.repeat_interleave(nh // nkv, 0)[None],
                                          v.repeat_interleave(nh // nkv, 0)[None], is_causal=True)[0]
    assert torch.allclose(pl.causal_attention(q, k, v), want, atol=1e-5)


def test_attention_special_cases():
    g = torch.Generator().manual_seed(6)
    q, v = torch.randn(2, 6, 8, generator=g), torch.randn(1, 6, 8, generator=g)
    k = torch.randn(1, 1, 8, generator=g).expand(1, 6, 8)  # all keys equal: uniform weights
    out = pl.causal_attention(q, k, v)
    assert torch.allclose(out[:, 0], v[:, 0].expand(2, 8), atol=1e-6)  # the first token sees itself only
    means = torch.cumsum(v[0], 0) / torch.arange(1, 7)[:, None]
    assert torch.allclose(out[0], means, atol=1e-5) and torch.allclose(out[1], means, atol=1e-5)


def test_attention_window_keeps_the_last_keys():
    g = torch.Generator().manual_seed(7)
    q, k, v = (torch.randn(1, 9, 8, generator=g) for _ in range(3))
    out = pl.causal_attention(q, k, v, window=3)
    for i in range(9):
        lo = max(0, i - 2)
        want = pl.causal_attention(q[:, lo:i + 1], k[:, lo:i + 1], v[:, lo:i + 1])[:, -1]
        assert torch.allclose(out[:, i], want, atol=1e-5)


def test_swiglu_is_silu_gate_times_up():
    g = torch.Generator().manual_seed(8)
    x = torch.randn(5, 12, generator=g)
    w = {"gate_proj.weight": torch.randn(20, 12, generator=g), "up_proj.weight": torch.randn(20, 12, generator=g),
         "down_proj.weight": torch.randn(12, 20, generator=g)}
    want = F.linear(F.silu(F.linear(x, w["gate_proj.weight"])) * F.linear(x, w["up_proj.weight"]), w["down_proj.weight"])
    assert torch.allclose(pl.swiglu(x, w, ""), want, atol=1e-5)
    w0 = dict(w, **{"gate_proj.weight": torch.zeros(20, 12)})
    assert torch.equal(pl.swiglu(x, w0, ""), torch.zeros(5, 12))  # silu(0) = 0 closes the gate


def _model(cfg, seed=0):
    from llmserve.parts.model import Model
    from llmserve.parts.registry import BuildContext
    from llmserve.config import architecture_of
    from llmserve.weights import random_tensors

    arch = architecture_of(cfg)
    model = Model(arch.build_spec(arch.config_class.from_dict(cfg)), BuildContext(torch.float32, torch.device("cpu")))
    return random_tensors(model.param_infos(), seed, torch.float32)


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_forward_is_causal_and_uses_the_tied_head(cfg):
    w = _model(cfg)
    ids = torch.randint(0, cfg["vocab_size"], (14,), generator=torch.Generator().manual_seed(9)).tolist()
    full = pl.forward(cfg, w, ids, torch.float32)
    assert full.shape == (14, cfg["vocab_size"])
    head = pl.forward(cfg, w, ids[:9], torch.float32)
    assert torch.allclose(full[:9], head, atol=1e-5)  # later tokens do not reach back
    assert ("lm_head.weight" in w) == (not cfg["tie_word_embeddings"])


# ------------------------------------------------------------------ the whole model, pinned without a second reading
def library_forward(cfg, w, ids):
    """The same model put together from the library's own routines only, batched and with complex numbers for
    the rotation: embedding, rms_norm, linear, scaled_dot_product_attention, silu.  It shares the layer order
    with the plain implementation (both follow src/llmserve/model/llama.py:131-135,171-185) and nothing else."""
    nh = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads", nh)
    hidden = cfg["hidden_size"]
    d = hidden // nh
    eps, theta = cfg["rms_norm_eps"], cfg["rope_theta"]
    t = len(ids)
    x = F.embedding(torch.tensor([ids]), w["model.embed_tokens.weight"])  # [1, T, H]
    turn = torch.polar(torch.ones(t, d // 2, dtype=torch.float64),
                       torch.arange(t, dtype=torch.float64)[:, None] * theta ** (-torch.arange(0, d, 2, dtype=torch.float64) / d))

    def rotate(v):  # [1, heads, T, D]; dimension i is the real part, i + D/2 the imaginary part
        z = torch.complex(v[..., : d // 2].double(), v[..., d // 2:].double()) * turn
        return torch.cat([z.real, z.imag], dim=-1).float()

    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = F.rms_norm(x, (hidden,), w[p + "input_layernorm.weight"], eps)
        q = F.linear(h, w[p + "self_attn.q_proj.weight"]).view(1, t, nh, d).transpose(1, 2)
        k = F.linear(h, w[p + "self_attn.k_proj.weight"]).view(1, t, nkv, d).transpose(1, 2)
        v = F.linear(h, w[p + "self_attn.v_proj.weight"]).view(1, t, nkv, d).transpose(1, 2)
        o = F.scaled_dot_product_attention(rotate(q), rotate(k), v, is_causal=True, enable_gqa=True)
        x = x + F.linear(o.transpose(1, 2).reshape(1, t, hidden), w[p + "self_attn.o_proj.weight"])
        h = F.rms_norm(x, (hidden,), w[p + "post_attention_layernorm.weight"], eps)
        x = x + F.linear(F.silu(F.linear(h, w[p + "mlp.gate_proj.weight"])) * F.linear(h, w[p + "mlp.up_proj.weight"]),
                         w[p + "mlp.down_proj.weight"])
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings") else w["lm_head.weight"]
    return F.linear(F.rms_norm(x, (hidden,), w["model.norm.weight"], eps), head)[0]


def _lively(w, seed=0):
    """Norm weights well away from 1 and matrices large enough that every branch matters."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, t in w.items():
        if name.endswith("norm.weight") or "layernorm" in name:
            out[name] = 1 + 0.5 * torch.randn(t.shape, generator=g)
        else:
            out[name] = t * 4
    return out


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_whole_model_from_library_routines(cfg):
    """atol 1e-4, the bound of the reference's own whole-model test (tests/test_model.py:85-105 there, which
    compares with an installed model class; no such class is used here)."""
    w = _lively(_model(cfg, seed=4))
    ids = torch.randint(0, cfg["vocab_size"], (23,), generator=torch.Generator().manual_seed(10)).tolist()
    got, want = pl.forward(cfg, w, ids, torch.float32), library_forward(cfg, w, ids)
    assert float(want.abs().max()) > 0.5
    assert (got - want).abs().max() <= 1e-4


def test_grouped_heads_read_the_kv_head_of_their_group():
    """A grouped model equals the ungrouped model whose K and V projections repeat each KV head for its group:
    query head h reads KV head h // group (a map like h % kv_heads fails here)."""
    cfg = dict(TINY_A, num_hidden_layers=1)
    w = _lively(_model(cfg, seed=5))
    nh, nkv, d = 4, 2, 16
    wide = dict(w)
    for name in ("k_proj", "v_proj"):
        key = f"model.layers.0.self_attn.{name}.weight"
        wide[key] = w[key].view(nkv, d, 64).repeat_interleave(nh // nkv, dim=0).reshape(nh * d, 64)
    ids = list(range(40, 57))
    got = pl.forward(cfg, w, ids, torch.float32)
    assert (got - pl.forward(dict(cfg, num_key_value_heads=nh), wide, ids, torch.float32)).abs().max() <= 1e-5
    tiled = dict(w)
    for name in ("k_proj", "v_proj"):
        key = f"model.layers.0.self_attn.{name}.weight"
        tiled[key] = w[key].view(nkv, d, 64).repeat(nh // nkv, 1, 1).reshape(nh * d, 64)
    assert (got - pl.forward(dict(cfg, num_key_value_heads=nh), tiled, ids, torch.float32)).abs().max() > 1e-3


def test_a_head_is_a_block_of_consecutive_rows():
    """Swapping two whole heads (rows h*D..(h+1)*D-1 of q, k, v and the same columns of o_proj) changes nothing;
    it would if heads were interleaved over the rows."""
    cfg = dict(TINY_A, num_hidden_layers=1, num_key_value_heads=4)
    w = _lively(_model(cfg, seed=6))
    order = torch.cat([torch.arange(32, 48), torch.arange(16, 32), torch.arange(0, 16), torch.arange(48, 64)])
    swapped = dict(w)
    for name in ("q_proj", "k_proj", "v_proj"):
        key = f"model.layers.0.self_attn.{name}.weight"
        swapped[key] = w[key][order]
    swapped["model.layers.0.self_attn.o_proj.weight"] = w["model.layers.0.self_attn.o_proj.weight"][:, order]
    ids = list(range(7, 30))
    assert (pl.forward(cfg, w, ids, torch.float32) - pl.forward(cfg, swapped, ids, torch.float32)).abs().max() <= 1e-5


def test_both_norms_sit_in_front_of_their_branch():
    """With a tiny eps a normed branch does not feel the scale of its input: layer(c x) - c x = layer(x) - x when
    the other branch is shut (its output projection zero).  A norm after the branch, or none, fails this."""
    cfg = TINY_B
    w = _lively(_model(cfg, seed=7))
    x = torch.randn(9, 96, generator=torch.Generator().manual_seed(11))
    args = dict(n_heads=3, n_kv_heads=1, head_dim=32, theta=5e5, eps=1e-12)
    for shut in ("mlp.down_proj.weight", "self_attn.o_proj.weight"):
        w1 = dict(w)
        w1["model.layers.0." + shut] = torch.zeros_like(w["model.layers.0." + shut])
        branch = pl.decoder_layer(x, w1, "model.layers.0.", **args) - x
        assert float(branch.abs().max()) > 1e-2
        assert ((pl.decoder_layer(3 * x, w1, "model.layers.0.", **args) - 3 * x) - branch).abs().max() <= 1e-4
    both = dict(w)
    for shut in ("mlp.down_proj.weight", "self_attn.o_proj.weight"):
        both["model.layers.0." + shut] = torch.zeros_like(w["model.layers.0." + shut])
    assert torch.equal(pl.decoder_layer(x, both, "model.layers.0.", **args), x)  # the stream itself is never normed


def test_the_second_branch_reads_the_stream_after_the_first():
    cfg = TINY_B
    w = _lively(_model(cfg, seed=8))
    x = torch.randn(6, 96, generator=torch.Generator().manual_seed(12))
    args = dict(n_heads=3, n_kv_heads=1, head_dim=32, theta=5e5, eps=1e-6)
    p = "model.layers.1."
    a = pl.attention_block(pl.rms_norm(x, w[p + "input_layernorm.weight"], 1e-6), w, p + "self_attn.", 3, 1, 32, 5e5)
    mid = x + a
    want = mid + pl.swiglu(pl.rms_norm(mid, w[p + "post_attention_layernorm.weight"], 1e-6), w, p + "mlp.")
    assert (pl.decoder_layer(x, w, p, **args) - want).abs().max() <= 1e-6
    parallel = mid + pl.swiglu(pl.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-6), w, p + "mlp.")
    assert (want - parallel).abs().max() > 1e-3  # (the test can tell the two arrangements apart)


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_final_norm_sits_between_the_last_layer_and_the_head(cfg):
    w = _lively(_model(cfg, seed=9))
    ids = list(range(11, 25))
    base = pl.forward(cfg, w, ids, torch.float32)
    scaled = dict(w, **{"model.norm.weight": 2.5 * w["model.norm.weight"]})
    assert (pl.forward(cfg, scaled, ids, torch.float32) - 2.5 * base).abs().max() <= 1e-4 * float(base.abs().max())
    off = dict(w, **{"model.norm.weight": torch.zeros_like(w["model.norm.weight"])})
    assert torch.equal(pl.forward(cfg, off, ids, torch.float32), torch.zeros_like(base))
    # with every branch shut the logits are head(norm(embedding)): no layer norms the stream on its way
    shut = {k: (torch.zeros_like(v) if k.endswith(("o_proj.weight", "down_proj.weight")) else v) for k, v in w.items()}
    table = w["model.embed_tokens.weight"]
    head = table if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    want = F.linear(F.rms_norm(table[torch.tensor(ids)], (cfg["hidden_size"],), w["model.norm.weight"], cfg["rms_norm_eps"]), head)
    assert (pl.forward(cfg, shut, ids, torch.float32) - want).abs().max() <= 1e-5


def test_forward_bfloat16_stays_near_float32():
    w = _model(TINY_A)
    ids = list(range(3, 40))
    f32 = pl.forward(TINY_A, w, ids, torch.float32)
    b16 = pl.forward(TINY_A, {k: v.bfloat16() for k, v in w.items()}, ids, torch.bfloat16)
    assert (f32 - b16).abs().max() < 0.05 * f32.abs().max()


LOGITS = torch.tensor([0.1, 3.0, 0.2, 2.9, -1.0])  # the reference's vector (tests/test_sampling.py:7-8)


def test_sampler_reference_vectors():
    assert pl.sample(LOGITS, 0.0, 0, 1.0, 0.5) == 1  # greedy is argmax
    us = [i / 20 for i in range(20)]
    assert all(pl.sample(LOGITS, 1.0, 1, 1.0, u) == 1 for u in us)  # top_k = 1
    assert all(pl.sample(LOGITS, 1.0, 0, 1e-6, u) == 1 for u in us)  # tiny top_p keeps the top token
    assert {pl.sample(LOGITS, 1.0, 2, 1.0, u) for u in [i / 200 for i in range(200)]} <= {1, 3}


def test_sampler_follows_the_distribution():
    probs = torch.softmax(LOGITS.double() / 0.7, -1)
    n = 4000
    counts = torch.zeros(5)
    for i in range(n):
        counts[pl.sample(LOGITS, 0.7, 0, 1.0, (i + 0.5) / n)] += 1
    assert torch.allclose(counts / n, probs.float(), atol=2e-3)


def test_generate_appends_eos_and_stops():
    w = _model(TINY_A)
    prompt = list(range(5, 15))
    first = pl.generate(TINY_A, w, prompt, 1, torch.float32)[0]
    assert pl.generate(TINY_A, w, prompt, 20, torch.float32, eos_token_id=first) == [first]
    assert len(pl.generate(TINY_A, w, prompt, 4, torch.float32)) == 4
