"""Builders of replay traces (lists of the JSON records `bin/trace_run` reads) and the
checks that compare what a replay wrote with the plain implementation."""

from __future__ import annotations

import random

import torch

import plain_llama

PORTIONS = [24, 7, 2, 16, 3, 11, 2, 5]


def random_ids(vocab: int, n: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def whole(seqs: dict[str, list[int]]) -> list[dict]:
    """Each request alone and whole: one step per request."""
    steps = []
    for i, (rid, ids) in enumerate(seqs.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": ids, "want": list(range(len(ids)))}],
                      "end": [rid]})
    return steps


def prefill_then_decode(seqs: dict[str, list[int]], tail: int = 32) -> list[dict]:
    """Most of a request in one step, its last `tail` tokens one by one (short requests: all
    but the first token one by one)."""
    steps = []
    for rid, ids in seqs.items():
        head = max(1, len(ids) - tail)
        cuts = [(0, head)] + [(p, p + 1) for p in range(head, len(ids))]
        for j, (a, b) in enumerate(cuts):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": ids[a:b], "want": list(range(b - a))}],
                          "end": [rid] if j == len(cuts) - 1 else []})
    return steps


def portions(seqs: dict[str, list[int]], sizes=PORTIONS) -> list[dict]:
    """In portions of changing size, down to two tokens."""
    steps = []
    for k, (rid, ids) in enumerate(seqs.items()):
        pos, j = 0, k  # start the size cycle at a different place for every request
        while pos < len(ids):
            n = min(sizes[j % len(sizes)], len(ids) - pos)
            j += 1
            done = pos + n == len(ids)
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": ids[pos:pos + n],
                                                           "want": list(range(n))}], "end": [rid] if done else []})
            pos += n
    return steps


def mixed(seqs: dict[str, list[int]], seed: int = 0, live_max: int = 4, tail: int = 6) -> list[dict]:
    """Up to `live_max` live requests; portions of some beside single tokens of others; a
    request is sometimes left out of a step; a finished request makes room for the next."""
    rng = random.Random(seed)
    waiting = list(seqs.items())
    live: list[list] = []  # [id, ids, pos]
    steps = []
    while waiting or live:
        while waiting and len(live) < live_max:
            rid, ids = waiting.pop(0)
            live.append([rid, ids, 0])
        entries, ended = [], []
        for item in live:
            rid, ids, pos = item
            if len(live) > 1 and rng.random() < 0.2 and entries:
                continue  # left out of this step
            remaining = len(ids) - pos
            if remaining <= tail:
                n = 1
            else:
                n = min(rng.choice([2, 3, 5, 8, 13, 24]), remaining - tail)
            entries.append({"id": rid, "tokens": ids[pos:pos + n], "want": list(range(n))})
            item[2] = pos + n
            if item[2] == len(ids):
                ended.append(rid)
        live = [it for it in live if it[0] not in ended]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def tokens_needed(steps: list[dict], round_to: int = 64) -> int:
    """--max-tokens for a trace: the most tokens live requests hold at any time, each
    request's count rounded up to a multiple of `round_to`."""
    length: dict[str, int] = {}
    most = 0
    for rec in steps:
        for e in rec["entries"]:
            length[e["id"]] = length.get(e["id"], 0) + len(e["tokens"])
        most = max(most, sum(-(-n // round_to) * round_to for n in length.values()))
        for rid in rec["end"]:
            length.pop(rid, None)
    return most


def collect(steps: list[dict], outputs: dict[int, torch.Tensor], partial: bool = False):
    """Per request the [len, vocab] logits, assembled from per-step outputs (`partial`: only some places
    were wanted; per request a dict from place to its logits)."""
    rows: dict[str, dict[int, torch.Tensor]] = {}
    length: dict[str, int] = {}
    for rec in steps:
        out = outputs.get(rec["step"])
        r = 0
        for e in rec["entries"]:
            start = length.get(e["id"], 0)
            for w in e["want"]:
                rows.setdefault(e["id"], {})[start + w] = out[r]
                r += 1
            length[e["id"]] = start + len(e["tokens"])
        assert out is None or r == out.shape[0]
    if partial:
        return rows
    return {rid: torch.stack([d[i] for i in sorted(d)]) for rid, d in rows.items()}


_PLAIN_CACHE: dict = {}


def plain_logits(model_dir, ids: list[int], dtype: torch.dtype) -> torch.Tensor:
    key = (str(model_dir), tuple(ids), dtype)
    if key not in _PLAIN_CACHE:
        cfg, w = plain_llama.read_model_dir(model_dir, dtype)
        _PLAIN_CACHE[key] = plain_llama.forward(cfg, w, ids, dtype)
    return _PLAIN_CACHE[key]


def tolerance(dtype: torch.dtype, ref: torch.Tensor) -> tuple[float, float]:
    """(max abs, mean abs) difference allowed between engine and plain logits.

    32-bit: only the order of summation differs: 2e-5 on logits of order 1 (the reference
    allows 1e-4, tests/test_model.py:10).  bfloat16: engine and plain implementation round
    at the same places, so they differ by single roundings (2^-8 relative) that flip with
    the order of summation and travel through the layers; the bound is a few such
    roundings of the largest logit, and the mean must stay near one rounding."""
    scale = max(1.0, float(ref.abs().max()))
    if dtype == torch.float32:
        return 2e-5 * scale, 5e-6 * scale
    return 2.0 ** -6 * scale, 2.0 ** -9 * scale


def assert_close(got: torch.Tensor, ref: torch.Tensor, dtype: torch.dtype, what: str) -> None:
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    diff = (got.double() - ref.double()).abs()
    max_tol, mean_tol = tolerance(dtype, ref)
    worst = int(diff.max(dim=-1).values.argmax())
    assert diff.max() <= max_tol, (f"{what}: max |diff| {diff.max():.3e} > {max_tol:.3e}; first bad position "
                                   f"{int((diff.max(dim=-1).values > max_tol).nonzero()[0])}, worst {worst}")
    assert diff.mean() <= mean_tol, f"{what}: mean |diff| {diff.mean():.3e} > {mean_tol:.3e}"
