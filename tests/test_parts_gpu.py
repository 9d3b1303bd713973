"""Each part of a layer alone against its plain counterpart, and the generality of the
arrangement: a toy architecture, defined here and nowhere in the framework, whose layers
differ (rotary attention, windowed attention without position encoding and with biases, a
mixer with fixed-size state of its own, a layer that reads another layer's cache), one of
them run twice.  It is registered, written to a folder, loaded and stepped in portions."""

from dataclasses import dataclass

import pytest
import torch

import plain_llama as pl
import traces

pytestmark = pytest.mark.gpu

DEV = torch.device("cuda:0")
DTYPES = [torch.float32, torch.bfloat16]


def ctx(dtype):
    from llmserve.parts import BuildContext

    return BuildContext(dtype, DEV)


def rnd(*shape, seed=0, scale=1.0):
    return scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


def tol(dtype, ref):
    scale = max(1e-3, float(ref.abs().max()))
    return scale * (2.0 ** -6 if dtype == torch.bfloat16 else 1e-5)


def load_random(part, dtype, seed=0, scale=0.3):
    tensors = {}
    for i, (name, info) in enumerate(part.param_infos().items()):
        t = rnd(*info.shape, seed=seed + i, scale=scale)
        if info.init == "norm":
            t = 1 + 0.3 * t
        tensors[name] = t.to(dtype)
    part.load({k: v.to(DEV) for k, v in tensors.items()})
    return tensors


# ------------------------------------------------------------------ norm, position encoding, feed-forward
@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(dtype):
    from llmserve.parts import NORMS, PartSpec

    norm = NORMS.build(PartSpec("rmsnorm", {"hidden": 100, "eps": 1e-6}), ctx(dtype))
    w = load_random(norm, dtype)["weight"]
    x, d = rnd(6, 100, seed=1).to(dtype), rnd(6, 100, seed=2).to(dtype)
    ref = pl.rms_norm(x, w, 1e-6).float()
    assert (norm.forward(x.to(DEV)).float().cpu() - ref).abs().max() <= tol(dtype, ref)
    resid = x.clone().to(DEV)
    summed = (x.float() + d.float()).to(dtype)
    ref = pl.rms_norm(summed, w, 1e-6).float()
    assert (norm.add_norm(resid, d.to(DEV)).float().cpu() - ref).abs().max() <= tol(dtype, ref)
    assert torch.equal(resid.cpu(), summed)
    rows = torch.tensor([5, 1], dtype=torch.int32, device=DEV)
    got = norm.norm_rows(x.to(DEV), d.to(DEV), rows).float().cpu()
    assert (got - ref[[5, 1]]).abs().max() <= tol(dtype, ref)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rope_part(dtype):
    from llmserve.parts import POSITION_ENCODINGS, PartSpec

    nh, nkv, d = 3, 1, 32
    rope = POSITION_ENCODINGS.build(PartSpec("rope", {"head_dim": d, "theta": 500000.0}), ctx(dtype))
    rope.load({})
    qkv = rnd(5, (nh + 2 * nkv) * d, seed=3).to(dtype)
    pos = torch.tensor([0, 3, 100, 7, 255], dtype=torch.int32)
    dev = qkv.clone().to(DEV)
    rope.rotate(dev, pos.to(DEV), nh, nkv, d)
    cos, sin = pl.rope_cos_sin(pos, d, 500000.0)
    rot = pl.apply_rope(qkv[:, : (nh + nkv) * d].view(5, nh + nkv, d).transpose(0, 1), cos, sin).transpose(0, 1)
    got = dev.cpu()
    assert (got[:, : (nh + nkv) * d].float() - rot.reshape(5, -1).float()).abs().max() <= tol(dtype, rot.float()) * 4
    assert torch.equal(got[:, (nh + nkv) * d:], qkv[:, (nh + nkv) * d:])
    assert torch.equal(got[0], qkv[0])  # position 0 is the identity


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [3, 40])
def test_swiglu_part(dtype, rows):
    from llmserve.parts import FEED_FORWARDS, PartSpec

    ffn = FEED_FORWARDS.build(PartSpec("swiglu", {"hidden": 96, "intermediate": 176}), ctx(dtype))
    w = load_random(ffn, dtype, seed=4)
    x = rnd(rows, 96, seed=5).to(dtype)
    ref = pl.swiglu(x, w, "").float()
    assert (ffn.forward(x.to(DEV)).float().cpu() - ref).abs().max() <= tol(dtype, ref)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_tied_head(dtype):
    from llmserve.parts import EMBEDDINGS, HEADS, PartSpec

    emb = EMBEDDINGS.build(PartSpec("embedding", {"vocab": 333, "hidden": 96}), ctx(dtype))
    table = load_random(emb, dtype, seed=6)["weight"]
    ids = torch.tensor([0, 332, 17], dtype=torch.int32)
    assert torch.equal(emb.forward(ids.to(DEV)).cpu(), table[ids.long()])
    head = HEADS.build(PartSpec("lm_head", {"vocab": 333, "hidden": 96, "tied": True}), ctx(dtype))
    assert head.param_infos() == {}
    head.load({"weight": emb.weight})
    h = rnd(4, 96, seed=7).to(dtype)
    logits = head.forward(h.to(DEV))
    ref = h.float() @ table.float().t()
    assert logits.dtype == torch.float32 and (logits.cpu() - ref).abs().max() <= 1e-5 * float(ref.abs().max()) + 1e-6


# ------------------------------------------------------------------ attention alone
def attention_harness(dtype, params, lens, cuts, block_size=8, seed=10, xs=None):
    """Build an attention part with one layer of cache and run requests of `lens` tokens through it
    in the portions `cuts`; return its outputs and the plain result for the whole sequences."""
    from llmserve.cache import CacheManager, group_layers
    from llmserve.cache.storage import CacheStorage
    from llmserve.engine.batch import BatchUploader, build_batch
    from llmserve.parts import MIXERS, PartSpec

    att = MIXERS.build(PartSpec("attention", params), ctx(dtype))
    w = load_random(att, dtype, seed=seed, scale=0.25)
    hidden = params["hidden"]
    if xs is None:
        xs = [rnd(n, hidden, seed=seed + 50 + i) for i, n in enumerate(lens)]
    xs = [x.to(dtype) for x in xs]
    groups = group_layers([att.cache_spec()])
    manager = CacheManager(groups, num_blocks=sum(-(-n // block_size) for n in lens), block_size=block_size, max_seqs=4)
    storage = CacheStorage(groups, manager.num_blocks, block_size, 4, dtype, DEV, table_width=16)
    storage.poison()
    uploader = BatchUploader(DEV)
    outs = [[] for _ in lens]
    for b in range(len(lens)):
        manager.add_sequence(b)
    done = [0] * len(lens)
    for step in cuts:  # step: {request: tokens in this step}
        ids = sorted(step, key=lambda b: step[b] != 1)
        layout = manager.append(ids, [step[b] for b in ids])
        batch = build_batch(layout, [[0] * step[b] for b in ids], [], uploader, storage)
        x = torch.cat([xs[b][done[b]: done[b] + step[b]] for b in ids]).to(DEV)
        y = att.forward(x, batch, storage.layer_cache(0)).float().cpu()
        row = 0
        for b in ids:
            outs[b].append(y[row: row + step[b]])
            row += step[b]
            done[b] += step[b]
    refs = []
    for b, n in enumerate(lens):
        nh, nkv, d = params["num_heads"], params["num_kv_heads"], params["head_dim"]
        wp = {k: v for k, v in w.items()}
        if params["position"].kind == "rope":
            ref = pl.attention_block(xs[b], wp, "", nh, nkv, d, params["position"]["theta"], params.get("window"))
        else:  # no rotation: q, k as projected
            q = pl.linear(xs[b], wp["q_proj.weight"], wp.get("q_proj.bias")).view(n, nh, d).transpose(0, 1)
            k = pl.linear(xs[b], wp["k_proj.weight"], wp.get("k_proj.bias")).view(n, nkv, d).transpose(0, 1)
            v = pl.linear(xs[b], wp["v_proj.weight"], wp.get("v_proj.bias")).view(n, nkv, d).transpose(0, 1)
            o = pl.causal_attention(q, k, v, params.get("window")).transpose(0, 1).reshape(n, nh * d)
            ref = pl.linear(o, wp["o_proj.weight"])
        refs.append(ref.float())
    return [torch.cat(o) for o in outs], refs


def att_params(nh, nkv, d, hidden, position="rope", theta=10000.0, window=None, bias=False):
    from llmserve.parts import PartSpec

    pos = PartSpec("rope", {"head_dim": d, "theta": theta}) if position == "rope" else PartSpec("none", {})
    return {"hidden": hidden, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d, "bias": bias, "window": window,
            "position": pos}


ATT_PARTS = [
    (att_params(4, 2, 16, 64), 8),
    (att_params(3, 1, 32, 96, theta=5e5), 8),
    (att_params(2, 2, 48, 40, bias=True), 16),
    (att_params(4, 1, 16, 64, window=6), 8),
    (att_params(2, 1, 32, 64, position="none", window=11, bias=True), 8),
    (att_params(5, 5, 16, 80, position="none"), 4),  # pages of 4: the matrix-core kernel steps aside
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("params,block_size", ATT_PARTS)
def test_attention_part_whole_and_in_portions(dtype, params, block_size):
    lens = [37, 9]
    whole = [{0: 37, 1: 9}]
    pieces = [{0: 20}, {0: 1, 1: 4}, {0: 7, 1: 1}, {0: 1, 1: 1}, {0: 8, 1: 3}]
    for cuts in (whole, pieces):
        outs, refs = attention_harness(dtype, params, lens, cuts, block_size)
        for got, ref in zip(outs, refs):
            assert torch.isfinite(got).all()
            assert (got - ref).abs().max() <= tol(dtype, ref)


def test_attention_without_rotation_is_library_sdpa():
    """No position encoding, no window: the part must reduce to the library's causal attention."""
    import torch.nn.functional as F

    params = att_params(4, 2, 16, 64, position="none")
    outs, _ = attention_harness(torch.float32, params, [21], [{0: 21}], seed=33)
    from llmserve.parts import MIXERS, PartSpec

    att = MIXERS.build(PartSpec("attention", params), ctx(torch.float32))
    w = load_random(att, torch.float32, seed=33, scale=0.25)
    x = rnd(21, 64, seed=33 + 50)
    q = F.linear(x, w["q_proj.weight"]).view(21, 4, 16).transpose(0, 1)
    k = F.linear(x, w["k_proj.weight"]).view(21, 2, 16).transpose(0, 1).repeat_interleave(2, 0)
    v = F.linear(x, w["v_proj.weight"]).view(21, 2, 16).transpose(0, 1).repeat_interleave(2, 0)
    o = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    ref = F.linear(o.transpose(0, 1).reshape(21, 64), w["o_proj.weight"])
    assert (outs[0] - ref).abs().max() <= 1e-5


def test_attention_positions_only_count_as_distances():
    """Rotary attention depends on distances only: the last 9 inputs of a request of 30, placed at
    positions 0..8 of another request, give the same output at the last token when a window of 9
    hides everything earlier."""
    params = att_params(2, 1, 32, 64, window=9)
    x = rnd(30, 64, seed=44)
    outs, _ = attention_harness(torch.float32, params, [30, 9], [{0: 30, 1: 9}], seed=44, xs=[x, x[21:].clone()])
    assert (outs[0][-1] - outs[1][-1]).abs().max() <= 1e-5


# ------------------------------------------------------------------ a toy architecture, defined only here
@dataclass(frozen=True)
class ToyConfig:
    vocab_size: int
    hidden_size: int
    eps: float

    @classmethod
    def from_dict(cls, d):
        return cls(d["vocab_size"], d["hidden_size"], d["eps"])


def register_toy():
    from llmserve.config import register_architecture
    from llmserve.parts import (Block, FeedForward, LayerSpec, Mixer, ModelSpec, ParamInfo, PartSpec, PositionEncoding,
                                StateCacheSpec, register_block, register_feed_forward, register_mixer,
                                register_position_encoding)
    from llmserve.parts.linear import linear

    @register_position_encoding("interleaved")
    class InterleavedRotation(PositionEncoding):
        """Rotation of the pairs (2i, 2i+1) instead of (i, i + D/2): another position encoding, which the
        attention part takes through `rotate` alone (its fused kernels step aside)."""

        def __init__(self, spec, ctx):
            super().__init__(spec, ctx)
            self.theta = float(spec["theta"])

        def rotate(self, qkv, positions, n_heads, n_kv_heads, head_dim):
            n, half = qkv.shape[0], head_dim // 2
            inv = self.theta ** (-torch.arange(half, device=qkv.device, dtype=torch.float32) * 2 / head_dim)
            ang = positions.float()[:, None] * inv
            cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
            part = qkv[:, : (n_heads + n_kv_heads) * head_dim]
            x = part.float().view(n, n_heads + n_kv_heads, half, 2)
            even, odd = x[..., 0], x[..., 1]
            rot = torch.stack([even * cos - odd * sin, odd * cos + even * sin], dim=-1)
            part.copy_(rot.view(n, -1).to(qkv.dtype))

    @register_feed_forward("soft_experts")
    class SoftExperts(FeedForward):
        """y = sum_e softmax(router x)_e * down_e(gelu(up_e x)): a feed-forward with a router of its own
        (logits and softmax in 32-bit) and per-expert weights."""

        def __init__(self, spec, ctx):
            super().__init__(spec, ctx)
            self.hidden, self.inter, self.experts = spec["hidden"], spec["intermediate"], spec["experts"]

        def param_infos(self):
            infos = {"router.weight": ParamInfo((self.experts, self.hidden))}
            for e in range(self.experts):
                infos[f"experts.{e}.up.weight"] = ParamInfo((self.inter, self.hidden))
                infos[f"experts.{e}.down.weight"] = ParamInfo((self.hidden, self.inter))
            return infos

        def load(self, tensors):
            self.router = tensors["router.weight"].float()
            self.up = [tensors[f"experts.{e}.up.weight"].contiguous() for e in range(self.experts)]
            self.down = [tensors[f"experts.{e}.down.weight"].contiguous() for e in range(self.experts)]

        def forward(self, x):
            gates = torch.softmax(x.float() @ self.router.t(), dim=-1)
            y = torch.zeros_like(x, dtype=torch.float32)
            for e in range(self.experts):
                h = torch.nn.functional.gelu(linear(x, self.up[e]).float()).to(x.dtype)
                y += gates[:, e: e + 1] * linear(h, self.down[e]).float()
            return y.to(x.dtype)

    @register_mixer("running_mean")
    class RunningMean(Mixer):
        """y_t = W * mean(x_0 .. x_t): a mixer whose state per request is the running sum and the
        count, fixed in size whatever the length.  Plain torch on the device; it reads the batch's
        host fields, so steps through it are not captured as graphs."""

        def __init__(self, spec, ctx):
            super().__init__(spec, ctx)
            self.hidden = spec["hidden"]

        def cache_spec(self):
            return StateCacheSpec((self.hidden + 1,), "float32")

        def param_infos(self):
            return {"proj.weight": ParamInfo((self.hidden, self.hidden))}

        def load(self, tensors):
            self.weight = tensors["proj.weight"].contiguous()

        def forward(self, x, batch, cache):
            means = torch.empty_like(x, dtype=torch.float32)
            row = 0
            for slot, n in zip(batch.state_slot_list, batch.counts):
                state = cache.state[slot]
                sums = state[: self.hidden] + torch.cumsum(x[row: row + n].float(), 0)
                counts = state[self.hidden] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
                means[row: row + n] = sums / counts[:, None]
                state[: self.hidden] = sums[-1]
                state[self.hidden] = counts[-1]
                row += n
            return linear(means.to(x.dtype), self.weight)

    @register_block("sandwich")
    class SandwichBlock(Block):
        """x = x + post_norm(mixer(norm1(x))); x = x + feed_forward(norm2(x)): an arrangement with a third norm, a
        role the reference's layer does not have.  The model builds, loads and names the tensors of whatever
        roles an arrangement declares."""

        ROLES = dict(Block.ROLES, post_mixer_norm="norm")

        def forward(self, x, delta, batch, cache):
            h = self.mixer_norm.add_norm(x, delta)  # (x += delta in place)
            a = self.mixer.forward(h, batch, cache)
            a = self.post_mixer_norm.forward(a if isinstance(a, torch.Tensor) else a.total())
            h2 = self.feed_forward_norm.add_norm(x, a)
            return x, self.feed_forward.forward(h2)

    def toy_spec(cfg: ToyConfig) -> ModelSpec:
        h = cfg.hidden_size
        norm = PartSpec("rmsnorm", {"hidden": h, "eps": cfg.eps})
        interleaved = att_params(4, 2, 16, h)
        interleaved["position"] = PartSpec("interleaved", {"theta": 10000.0})
        mixers = [
            PartSpec("attention", interleaved),
            PartSpec("attention", att_params(2, 1, 32, h, position="none", window=5, bias=True)),
            PartSpec("running_mean", {"hidden": h}),
            PartSpec("attention", att_params(2, 2, 16, h, theta=777.0)),  # reads the cache of layer 0
        ]
        inters = [80, 48, 64, 32]
        layers = []
        for i, (mixer, inter) in enumerate(zip(mixers, inters)):
            p = f"toy.{i}."
            ffn = (PartSpec("soft_experts", {"hidden": h, "intermediate": inter, "experts": 3}) if i == 2
                   else PartSpec("swiglu", {"hidden": h, "intermediate": inter}))
            parts = {"mixer": mixer, "feed_forward": ffn, "mixer_norm": norm, "feed_forward_norm": norm}
            weights = {"mixer": p + "mix.", "feed_forward": p + "ffn.", "mixer_norm": p + "n1.", "feed_forward_norm": p + "n2."}
            if i == 1:  # the layer that runs twice has a third norm
                parts["post_mixer_norm"], weights["post_mixer_norm"] = norm, p + "n3."
            layers.append(LayerSpec(parts=parts, weights=weights, block="sandwich" if i == 1 else "prenorm",
                                    cache_from=0 if i == 3 else None))
        return ModelSpec(hidden_size=h, vocab_size=cfg.vocab_size, max_positions=128,
                         embedding=PartSpec("embedding", {"vocab": cfg.vocab_size, "hidden": h}),
                         layers=tuple(layers), schedule=(0, 1, 2, 3, 1), final_norm=norm,
                         head=PartSpec("lm_head", {"vocab": cfg.vocab_size, "hidden": h, "tied": False}),
                         weights={"embedding": "toy.emb.", "final_norm": "toy.norm.", "head": "toy.head."})

    register_architecture("ToyForCausalLM", ToyConfig, toy_spec)


TOY = {"architectures": ["ToyForCausalLM"], "vocab_size": 97, "hidden_size": 64, "eps": 1e-5}


def plain_toy_forward(w, ids, dtype):
    """The toy model from the plain parts, whole sequence, no cache."""
    t, h, eps = len(ids), 64, 1e-5
    x = w["toy.emb.weight"][torch.tensor(ids)].to(dtype)
    kv = {}

    def attention(i, hn, nh, nkv, d, theta, window, borrow=None, interleaved=False):
        p = f"toy.{i}.mix."
        q = pl.linear(hn, w[p + "q_proj.weight"], w.get(p + "q_proj.bias")).view(t, nh, d).transpose(0, 1)
        k = pl.linear(hn, w[p + "k_proj.weight"], w.get(p + "k_proj.bias")).view(t, nkv, d).transpose(0, 1)
        v = pl.linear(hn, w[p + "v_proj.weight"], w.get(p + "v_proj.bias")).view(t, nkv, d).transpose(0, 1)
        if theta is not None and interleaved:
            ang = torch.arange(t, dtype=torch.float32)[:, None] * theta ** (-torch.arange(d // 2, dtype=torch.float32) * 2 / d)

            def turn(x):  # [heads, t, d], pairs (2i, 2i+1)
                xf = x.float().view(x.shape[0], t, d // 2, 2)
                even, odd = xf[..., 0], xf[..., 1]
                return torch.stack([even * ang.cos() - odd * ang.sin(), odd * ang.cos() + even * ang.sin()], -1).view_as(x).to(x.dtype)

            q, k = turn(q.contiguous()), turn(k.contiguous())
        elif theta is not None:
            cos, sin = pl.rope_cos_sin(torch.arange(t), d, theta)
            q, k = pl.apply_rope(q, cos, sin), pl.apply_rope(k, cos, sin)
        if borrow is not None:
            k, v = kv[borrow]
        kv[i] = (k, v)
        o = pl.causal_attention(q, k, v, window).transpose(0, 1).reshape(t, nh * d)
        return pl.linear(o, w[p + "o_proj.weight"])

    for i in (0, 1, 2, 3, 1):
        p = f"toy.{i}."
        hn = pl.rms_norm(x, w[p + "n1.weight"], eps)
        if i == 0:
            a = attention(0, hn, 4, 2, 16, 10000.0, None, interleaved=True)
        elif i == 1:
            a = attention(1, hn, 2, 1, 32, None, 5)
        elif i == 2:
            means = torch.cumsum(hn.float(), 0) / torch.arange(1, t + 1)[:, None]
            a = pl.linear(means.to(dtype), w[p + "mix.proj.weight"])
        else:
            a = attention(3, hn, 2, 2, 16, 777.0, None, borrow=0)
        if i == 1:
            a = pl.rms_norm(a, w[p + "n3.weight"], eps)
        x = x + a
        hn2 = pl.rms_norm(x, w[p + "n2.weight"], eps)
        if i == 2:  # the routed feed-forward
            gates = torch.softmax(hn2.float() @ w[p + "ffn.router.weight"].float().t(), dim=-1)
            y = torch.zeros(t, h)
            for e in range(3):
                up = pl.linear(hn2, w[p + f"ffn.experts.{e}.up.weight"])
                y += gates[:, e: e + 1] * pl.linear(torch.nn.functional.gelu(up.float()).to(dtype),
                                                    w[p + f"ffn.experts.{e}.down.weight"]).float()
            x = x + y.to(dtype)
        else:
            x = x + pl.swiglu(hn2, w, p + "ffn.")
    return pl.rms_norm(x, w["toy.norm.weight"], eps).float() @ w["toy.head.weight"].float().t()


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_toy_architecture_is_registered_built_and_stepped(tmp_path, dtype_name):
    from safetensors.torch import load_file

    from llmserve.config import EngineConfig
    from llmserve.engine.replay import Replayer
    from llmserve.engine.runner import ModelRunner
    from llmserve.weights import write_random_model

    register_toy()
    # weights large enough for attention to have favourites, small enough that bfloat16's own noise
    # (plain bfloat16 against plain 32-bit) stays below the comparison's tolerance
    write_random_model(tmp_path, TOY, seed=5, std=0.06)
    dtype = getattr(torch, dtype_name)
    runner = ModelRunner.from_folder(tmp_path, EngineConfig(dtype=dtype_name, block_size=8, num_blocks=24, max_num_seqs=3))
    assert not runner.model.graph_safe()  # the toy mixer reads host fields
    kinds = [(g.paged, g.spec.window if g.paged else None, len(g.layers)) for g in runner.manager.groups]
    # rotary layer 0 alone (layer 3 borrows it), the windowed layer twice (it runs twice), one state group
    assert sorted(kinds, key=str) == sorted([(True, None, 1), (True, 5, 2), (False, None, 1)], key=str)
    runner.storage.poison()
    seqs = {f"t{i}": traces.random_ids(97, n, 900 + i) for i, n in enumerate([41, 23, 12, 30])}
    w = {k: v.to(dtype) for k, v in load_file(str(tmp_path / "model.safetensors")).items()}
    for mode in (traces.whole, traces.portions, lambda s: traces.mixed(s, seed=8, live_max=3)):
        steps = mode(seqs)
        rep = Replayer(runner)
        outputs = {}
        for rec in steps:
            out = rep.run(rec)
            runner.manager.check_invariants()
            if out.shape[0]:
                outputs[rec["step"]] = out.float().cpu()
        got = traces.collect(steps, outputs)
        for rid, ids in seqs.items():
            traces.assert_close(got[rid], plain_toy_forward(w, ids, dtype), dtype, f"toy {rid} {dtype_name}")
        assert runner.manager.num_free_slots == 3
        assert all(a.num_free == 24 for a in runner.manager.allocators.values())


def test_toy_architecture_generates_through_the_scheduler(tmp_path):
    """The toy mixer reads host fields, so no step of this model is replayed from a graph and the runner takes
    tokens from the host only: generation through the entry point must still feed every sampled id back."""
    from safetensors.torch import load_file

    from llmserve import LLM, EngineConfig, SamplingParams
    from llmserve.weights import write_random_model

    register_toy()
    write_random_model(tmp_path, TOY, seed=6, std=0.06)
    w = load_file(str(tmp_path / "model.safetensors"))
    llm = LLM(tmp_path, dtype="float32", engine=EngineConfig(block_size=8, num_blocks=48, max_num_seqs=3,
                                                              max_num_batched_tokens=16))
    assert not llm.runner.takes_device_tokens
    prompts = [traces.random_ids(97, n, 700 + i) for i, n in enumerate([9, 21, 4])]
    results = llm.generate(prompts, SamplingParams(max_new_tokens=10))
    for prompt, result in zip(prompts, results):
        ids = list(prompt)
        for _ in range(10):
            ids.append(int(plain_toy_forward(w, ids, torch.float32)[-1].argmax()))
        assert result.tokens == ids[len(prompt):]
    assert llm.runner.manager.num_free_slots == 3
