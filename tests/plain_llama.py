"""Plain, slow Llama: whole sequences, no cache, one function for each part.

Written from the formulas of the reference (the paths cited are relative to the reference's root);
it shares no code with the engine: weights come straight from the safetensors file
as a dict keyed by checkpoint name, the configuration is the raw config.json dict.

`dtype=torch.float32` evaluates the formulas exactly as written.  `dtype=torch.bfloat16`
keeps the reference's cast points (weights, activations and the residual stream are
rounded to bfloat16 after every operation) with the two exactness rules of this engine:
the rotation is done in 32-bit and rounded once, and scores, softmax and the value
sum are 32-bit with one rounding of the attention output.  Matrix products accumulate in
32-bit and round once, written out explicitly so the result does not depend on the
CPU library's bfloat16 mode.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


# --------------------------------------------------------------------------- parts


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """y = x W^T (+ b), weight stored [out, in] (src/llmserve/model/llama.py:64-67, nn.Linear)."""
    y = x.float() @ weight.float().t()
    if bias is not None:
        y = y + bias.float()
    return y.to(x.dtype)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """src/llmserve/model/llama.py:24-28: statistics in 32-bit, cast down, then times weight."""
    dtype = x.dtype
    xf = x.float()
    xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return weight * xf.to(dtype)


def rope_cos_sin(positions: torch.Tensor, head_dim: int, theta: float):
    """src/llmserve/model/llama.py:31-39: inv_freq_i = theta^(-2i/D); angles p*inv_freq,
    repeated for both halves; cos and sin in 32-bit."""
    exponent = torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim
    inv_freq = 1.0 / (theta**exponent)
    freqs = positions.float()[..., None] * inv_freq
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos(), emb.sin()


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """src/llmserve/model/llama.py:42-44: (x1, x2) -> (-x2, x1), halves not interleaved."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """src/llmserve/model/llama.py:47-54: x*cos + rotate_half(x)*sin; x is [heads, T, D],
    cos/sin [T, D].  Computed in 32-bit and rounded once to x's dtype."""
    xf = x.float()
    return (xf * cos[None] + rotate_half(xf) * sin[None]).to(x.dtype)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int | None = None):
    """q [nh, T, D], k/v [nkv, T, D] -> [nh, T, D].

    src/llmserve/model/llama.py:94-102: K and V heads are repeated nh/nkv times
    (query head h reads KV head h // (nh/nkv)), then scaled-dot-product attention with
    the default scale D^-1/2 and the causal mask `key j <= query i`
    (src/llmserve/kvcache/paged.py:105-110 states the same mask by positions).
    `window` (not in the reference) keeps only keys with i - j < window.
    """
    nh, T, D = q.shape
    rep = nh // k.shape[0]
    kf = k.float().repeat_interleave(rep, dim=0)
    vf = v.float().repeat_interleave(rep, dim=0)
    scores = (q.float() @ kf.transpose(1, 2)) * (1.0 / math.sqrt(D))
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    visible = j <= i
    if window is not None:
        visible = visible & (i - j < window)
    scores = scores.masked_fill(~visible[None], float("-inf"))
    probs = torch.softmax(scores, dim=-1)
    return (probs @ vf).to(q.dtype)


def attention_block(x, w, prefix, n_heads, n_kv_heads, head_dim, theta, window=None):
    """src/llmserve/model/llama.py:79-83,108-109: project, split heads (head h = output rows
    h*D..(h+1)*D-1), rotate q and k, attend, concatenate heads, o_proj (never a bias)."""
    T = x.shape[0]
    q = linear(x, w[prefix + "q_proj.weight"], w.get(prefix + "q_proj.bias"))
    k = linear(x, w[prefix + "k_proj.weight"], w.get(prefix + "k_proj.bias"))
    v = linear(x, w[prefix + "v_proj.weight"], w.get(prefix + "v_proj.bias"))
    q = q.view(T, n_heads, head_dim).transpose(0, 1)
    k = k.view(T, n_kv_heads, head_dim).transpose(0, 1)
    v = v.view(T, n_kv_heads, head_dim).transpose(0, 1)
    cos, sin = rope_cos_sin(torch.arange(T), head_dim, theta)
    q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    o = causal_attention(q, k, v, window)
    o = o.transpose(0, 1).reshape(T, n_heads * head_dim)
    return linear(o, w[prefix + "o_proj.weight"])


def silu(x: torch.Tensor) -> torch.Tensor:
    """z * sigmoid(z) (F.silu at src/llmserve/model/llama.py:120), rounded to x's dtype."""
    xf = x.float()
    return (xf * torch.sigmoid(xf)).to(x.dtype)


def swiglu(x, w, prefix):
    """src/llmserve/model/llama.py:112-120: down(silu(gate(x)) * up(x)), no biases."""
    g = linear(x, w[prefix + "gate_proj.weight"])
    u = linear(x, w[prefix + "up_proj.weight"])
    return linear(silu(g) * u, w[prefix + "down_proj.weight"])


def decoder_layer(x, w, prefix, n_heads, n_kv_heads, head_dim, theta, eps):
    """src/llmserve/model/llama.py:131-135: x = x + attn(norm1(x)); x = x + mlp(norm2(x)): both norms sit in front
    of their branch, and the second branch reads the stream after the first was added."""
    h = rms_norm(x, w[prefix + "input_layernorm.weight"], eps)
    x = x + attention_block(x=h, w=w, prefix=prefix + "self_attn.", n_heads=n_heads, n_kv_heads=n_kv_heads,
                            head_dim=head_dim, theta=theta)
    h = rms_norm(x, w[prefix + "post_attention_layernorm.weight"], eps)
    return x + swiglu(h, w, prefix + "mlp.")


# --------------------------------------------------------------------------- model


def read_model_dir(model_dir: str | Path, dtype: torch.dtype):
    """config.json as a dict and every tensor of model.safetensors by name, cast to dtype
    (src/llmserve/weights.py:31-43)."""
    from safetensors.torch import load_file

    model_dir = Path(model_dir)
    cfg = json.loads((model_dir / "config.json").read_text())
    weights = {k: v.to(dtype) for k, v in load_file(str(model_dir / "model.safetensors")).items()}
    return cfg, weights


def forward(cfg: dict, w: dict[str, torch.Tensor], ids: list[int], dtype: torch.dtype) -> torch.Tensor:
    """Logits [T, V] in 32-bit for the whole sequence `ids`.

    src/llmserve/model/llama.py:171-185 with src/llmserve/model/llama.py:131-135 per layer:
    x = E[ids]; x += attn(norm1(x)); x += mlp(norm2(x)); logits = lm_head(norm(x)).
    config.json keys and defaults as src/llmserve/config.py:47-60.
    """
    n_heads = cfg["num_attention_heads"]
    n_kv = cfg.get("num_key_value_heads", n_heads)
    head_dim = cfg["hidden_size"] // n_heads  # src/llmserve/config.py:22-24
    theta = float(cfg.get("rope_theta") or cfg.get("rope_parameters", {}).get("rope_theta", 10000.0))
    eps = cfg.get("rms_norm_eps", 1e-5)
    x = w["model.embed_tokens.weight"][torch.tensor(ids, dtype=torch.long)].to(dtype)
    for i in range(cfg["num_hidden_layers"]):
        x = decoder_layer(x, w, f"model.layers.{i}.", n_heads, n_kv, head_dim, theta, eps)
    x = rms_norm(x, w["model.norm.weight"], eps)
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return x.float() @ head.float().t()  # logits kept in 32-bit


# --------------------------------------------------------------------------- sampling


def filtered_probs(logits: torch.Tensor, temperature: float, top_k: int, top_p: float) -> torch.Tensor:
    """Distribution the reference draws from (src/llmserve/sampling/sampler.py:23-38), float64.

    z = logits/T; top-k keeps values >= the k-th largest (ties survive); top-p sorts
    descending, drops a token when the mass before it exceeds top_p; softmax of the rest.
    """
    z = logits.double() / temperature
    if top_k > 0:
        k = min(top_k, z.numel())
        kth = torch.topk(z, k).values[-1]
        z = z.masked_fill(z < kth, float("-inf"))
    if top_p < 1.0:
        sz, idx = torch.sort(z, descending=True)
        probs = torch.softmax(sz, dim=-1)
        remove = (probs.cumsum(-1) - probs) > top_p
        sz = sz.masked_fill(remove, float("-inf"))
        z = torch.full_like(z, float("-inf")).scatter(-1, idx, sz)
    return torch.softmax(z, dim=-1)


def sample(logits: torch.Tensor, temperature: float, top_k: int, top_p: float, u: float) -> int:
    """Greedy when temperature <= 0 (src/llmserve/sampling/sampler.py:20-21), else the inverse
    CDF of `filtered_probs` in vocabulary order at the uniform number u.  The reference draws
    with torch.multinomial; only reproducibility under a seed is promised there
    (tests/test_sampling.py:31-35), so the uniform number is an input here."""
    if temperature <= 0:
        return int(torch.argmax(logits).item())
    cdf = filtered_probs(logits, temperature, top_k, top_p).cumsum(-1)
    return int(min(int((cdf <= u * cdf[-1]).sum().item()), logits.numel() - 1))


def generate(cfg, w, prompt: list[int], max_new_tokens: int, dtype, eos_token_id=None) -> list[int]:
    """Greedy generation that re-runs the whole sequence for every token
    (src/llmserve/baseline/naive.py:33-47): the EOS token is appended before stopping."""
    ids = list(prompt)
    out: list[int] = []
    while len(out) < max_new_tokens:
        tok = int(torch.argmax(forward(cfg, w, ids, dtype)[-1]).item())
        out.append(tok)
        ids.append(tok)
        if eos_token_id is not None and tok == eos_token_id:
            break
    return out
