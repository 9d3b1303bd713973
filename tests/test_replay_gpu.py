"""Replays on the GPU against the plain implementation: each request alone and whole; most
of it in one step and the last 32 tokens one by one; in portions of changing size; mixed,
with so few pages that they are used again.  32-bit and bfloat16, both tiny configurations."""

import json
import os
import subprocess

import numpy as np
import pytest
import torch

import traces
from conftest import ROOT, TINY

pytestmark = pytest.mark.gpu

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
LENGTHS = {"a": [5, 17, 33, 100, 128], "b": [1, 7, 40, 64, 100, 250]}


def sequences(name: str) -> dict[str, list[int]]:
    vocab = TINY[name][0]["vocab_size"]
    return {f"{name}{i}": traces.random_ids(vocab, n, 1000 + 17 * i) for i, n in enumerate(LENGTHS[name])}


def replay_in_process(model_dir, dtype_name, steps, block_size, num_blocks, use_graphs=True, max_seqs=4):
    from llmserve.config import EngineConfig
    from llmserve.engine.replay import Replayer
    from llmserve.engine.runner import ModelRunner

    runner = ModelRunner.from_folder(model_dir, EngineConfig(dtype=dtype_name, block_size=block_size,
                                                              num_blocks=num_blocks, max_num_seqs=max_seqs,
                                                              use_graphs=use_graphs))
    runner.storage.poison()  # a slot that was never written must never be read
    rep = Replayer(runner)
    outputs = {}
    for rec in steps:
        logits = rep.run(rec)
        runner.manager.check_invariants()
        if logits.shape[0]:
            outputs[rec["step"]] = logits.float().cpu()
    assert runner.manager.num_free_blocks == num_blocks, "pages were not all returned"
    assert runner.manager.num_free_slots == max_seqs, "state slots were not all returned"
    from llmserve.ops import library as ops
    assert ops.arrival_counters_are_zero(), "a decode attention left workgroups counted"
    return outputs


def check_against_plain(model_dir, dtype_name, seqs, steps, outputs):
    per_request = traces.collect(steps, outputs)
    dtype = DTYPES[dtype_name]
    for rid, ids in seqs.items():
        ref = traces.plain_logits(model_dir, ids, dtype)
        traces.assert_close(per_request[rid], ref, dtype, f"{rid} (len {len(ids)}, {dtype_name})")


MODES = {
    "whole": traces.whole,
    "decode_tail": traces.prefill_then_decode,
    "portions": traces.portions,
    "mixed": lambda seqs: traces.mixed(seqs, seed=3),
}


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("name", list(TINY))
def test_replay_matches_plain(model_dirs, name, dtype_name, mode):
    seqs = sequences(name)
    steps = MODES[mode](seqs)
    block_size = TINY[name][1]
    # exactly as many pages as the trace needs at its fullest: freed pages must be used again
    num_blocks = traces.tokens_needed(steps, round_to=block_size) // block_size
    outputs = replay_in_process(model_dirs[name], dtype_name, steps, block_size, num_blocks)
    check_against_plain(model_dirs[name], dtype_name, seqs, steps, outputs)


@pytest.mark.parametrize("mode", ["decode_tail", "mixed"])
@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_replay_without_graphs(model_dirs, dtype_name, mode):
    """Steps of single tokens are replayed from captured HIP graphs by default; the same steps launched
    kernel by kernel must give the same answers."""
    seqs = sequences("b")
    steps = MODES[mode](seqs)
    block_size = TINY["b"][1]
    num_blocks = traces.tokens_needed(steps, round_to=block_size) // block_size
    outputs = replay_in_process(model_dirs["b"], dtype_name, steps, block_size, num_blocks, use_graphs=False)
    check_against_plain(model_dirs["b"], dtype_name, seqs, steps, outputs)


@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_steps_with_portions_are_replayed_from_graphs(model_dirs, dtype_name):
    """A step with portions always runs at the sizes of its bucket, kernel by kernel the first time the bucket
    comes and from a captured graph from the second time on.  The mixed and the portioned trace, run twice
    through one runner, hit such graphs; both passes agree with the plain implementation, whatever the
    padding holds (the cache is poisoned) and whichever pages are used again, and they agree with each
    other to the bit: which kernels run is a function of the bucket, not of the way it is launched."""
    from llmserve.config import EngineConfig
    from llmserve.engine.replay import Replayer
    from llmserve.engine.runner import ModelRunner

    name = "a"
    seqs = sequences(name)
    block_size = TINY[name][1]
    for mode in ("mixed", "portions"):
        steps = MODES[mode](seqs)
        num_blocks = traces.tokens_needed(steps, round_to=block_size) // block_size
        runner = ModelRunner.from_folder(model_dirs[name], EngineConfig(dtype=dtype_name, block_size=block_size,
                                                                        num_blocks=num_blocks, max_num_seqs=4))
        runner.storage.poison()
        passes = []
        for _ in range(2):
            rep = Replayer(runner)
            outputs = {}
            for rec in steps:
                logits = rep.run(rec)
                runner.manager.check_invariants()
                if logits.shape[0]:
                    outputs[rec["step"]] = logits.float().cpu()
            check_against_plain(model_dirs[name], dtype_name, seqs, steps, outputs)
            assert runner.manager.num_free_blocks == num_blocks
            passes.append(outputs)
        assert runner._step_graphs, f"{mode}: no step with portions was replayed from a graph"
        assert len(runner._buckets) <= runner.MAX_STEP_GRAPHS
        assert all(b.graph is not None for b in runner._buckets.values() if b.uses >= runner.CAPTURE_AT_USE)
        for step, first in passes[0].items():
            assert torch.equal(first, passes[1][step]), f"{mode} step {step}: a replay differs from the first run"


def test_one_trace_gives_the_same_bits_in_fresh_runners(model_dirs):
    """The same mixed bfloat16 trace in two fresh runners: equal to the bit (no decision depends on a clock)."""
    seqs = sequences("b")
    steps = traces.mixed(seqs, seed=3)
    bs = TINY["b"][1]
    num_blocks = traces.tokens_needed(steps, round_to=bs) // bs
    first = replay_in_process(model_dirs["b"], "bfloat16", steps + steps_renumbered(steps), bs, num_blocks)
    second = replay_in_process(model_dirs["b"], "bfloat16", steps + steps_renumbered(steps), bs, num_blocks)
    assert first.keys() == second.keys() and len(first) > len(steps)
    for step in first:
        assert torch.equal(first[step], second[step]), f"step {step} differs between two runs"


def steps_renumbered(steps):
    """The same trace once more, as later steps (its requests ended, so their names are free again)."""
    return [dict(rec, step=rec["step"] + len(steps)) for rec in steps]


def test_returned_logits_survive_the_next_step(model_dirs):
    """Logits that `step` returns belong to the caller: a later step, replayed from the same graph, must not
    change them (the scheduler, which samples at once, borrows them instead)."""
    from llmserve.config import EngineConfig
    from llmserve.engine.runner import ModelRunner, StepEntry

    runner = ModelRunner.from_folder(model_dirs["a"], EngineConfig(dtype="float32", block_size=16, num_blocks=8,
                                                                   max_num_seqs=2))
    runner.add_sequence("s")
    ids = traces.random_ids(256, 12, 3)
    runner.step([StepEntry("s", ids[:8], [7])])
    kept, copies = [], []
    for t in ids[8:]:
        kept.append(runner.step([StepEntry("s", [t], [0])]))
        copies.append(kept[-1].cpu().clone())
    lent = runner.step([StepEntry("s", [ids[0]], [0])], borrow=True)
    assert all(torch.equal(k.cpu(), c) for k, c in zip(kept, copies))
    assert len({c.numpy().tobytes() for c in copies}) == len(copies)
    assert lent.shape == (1, 256)
    runner.free_sequence("s")


def test_padding_of_steps_is_bounded():
    from llmserve.engine.runner import ModelRunner

    for n in list(range(1, 700)) + [1000, 2047, 2048, 2049, 5000]:
        padded = ModelRunner._row_bucket(n)
        assert n <= padded and (padded - n < 16 or padded - n <= n / 8)


WIDE = {  # layer sizes of real models, few layers
    "tinyllama-1.1b": dict(num_hidden_layers=2),               # hidden 2048, 32 heads on 4 KV heads of 64, 5632, 32000
    "llama2-7b": dict(num_hidden_layers=1, vocab_size=4000),   # hidden 4096, 32 heads of 128, 11008 (no multiple of 512)
    "llama2-70b": dict(num_hidden_layers=1, vocab_size=2000),  # hidden 8192, 64 heads on 8 KV heads of 128, 28672
}


@pytest.fixture(scope="module", params=list(WIDE))
def wide_model_dir(request, tmp_path_factory):
    from llmserve.config import preset
    from llmserve.weights import write_random_model

    cfg = dict(preset(request.param), **WIDE[request.param])
    d = tmp_path_factory.mktemp("wide")
    write_random_model(d, cfg, seed=23)
    return d, cfg


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_replay_at_full_layer_sizes(wide_model_dir, dtype_name, mode, monkeypatch):
    """The tiny configurations never reach the paths that the sizes of a real model choose: products whose
    K is shared out to several workgroups and summed by the norm, the library's product for many rows, 8 waves
    per decoded token, a vocabulary of 2,000 tiles."""
    model_dir, cfg = wide_model_dir
    # (700 tokens: portions behind a prefix long enough for attention to share a block's keys out to workgroups)
    seqs = {f"w{i}": traces.random_ids(cfg["vocab_size"], n, 2000 + i) for i, n in enumerate([40, 150, 300, 700])}
    steps = MODES[mode](seqs)
    num_blocks = traces.tokens_needed(steps, round_to=16) // 16
    from llmserve.ops import library as ops
    shared_out = []
    original = ops.attention_mfma
    monkeypatch.setattr(ops, "attention_mfma", lambda *a, **kw: (shared_out.append((kw.get("split_waves", False),
                                                                                    kw.get("num_splits", 1))), original(*a, **kw))[1])
    outputs = replay_in_process(model_dir, dtype_name, steps, 16, num_blocks)
    check_against_plain(model_dir, dtype_name, seqs, steps, outputs)
    if dtype_name == "bfloat16" and mode == "portions":
        assert any(not waves and splits > 1 for waves, splits in shared_out), "no portion shared its keys out"


def many_live_trace(cfg, live):
    """Portions of some prompts beside decoded tokens of requests whose prompt is in, until every request has at most
    5 tokens to go; then all of them decode side by side."""
    import random

    rng = random.Random(live)
    seqs = {f"m{i}": traces.random_ids(cfg["vocab_size"], rng.randint(12, 70), 3000 + i) for i in range(live)}
    pos = {rid: 0 for rid in seqs}
    steps = []

    def step_of(entries):
        ended = [e["id"] for e in entries if pos[e["id"]] == len(seqs[e["id"]])]
        steps.append({"step": len(steps), "entries": entries, "end": ended})

    def bring(rid, n):
        ids = seqs[rid]
        entry = {"id": rid, "tokens": ids[pos[rid]:pos[rid] + n], "want": list(range(n))}
        pos[rid] += n
        return entry

    while any(len(ids) - pos[rid] > 5 for rid, ids in seqs.items()):
        entries = []
        for rid, ids in seqs.items():
            to_go = len(ids) - pos[rid]
            if to_go > 5 and rng.random() < 0.5:
                entries.append(bring(rid, min(rng.choice([2, 3, 5, 8, 13, 24]), to_go - 5)))
            elif 2 < to_go <= 5 and rng.random() < 0.2:
                entries.append(bring(rid, 1))
        if entries:
            step_of(entries)
    while any(pos[rid] < len(ids) for rid, ids in seqs.items()):
        step_of([bring(rid, 1) for rid, ids in seqs.items() if pos[rid] < len(ids)])
    assert any(len(rec["entries"]) == live and all(len(e["tokens"]) == 1 for e in rec["entries"]) for rec in steps)
    assert any(len(rec["entries"]) > 16 and any(len(e["tokens"]) > 1 for e in rec["entries"]) for rec in steps) or live <= 20
    return seqs, steps


@pytest.mark.parametrize("use_graphs", [True, False], ids=["graphs", "launches"])
@pytest.mark.parametrize("live", [20, 48])
@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_many_live_requests_at_full_layer_sizes(wide_model_dir, dtype_name, live, use_graphs):
    """17 to 64 rows at the widths of real models: the products for that many rows (the rows in registers, with the
    activation or the rotation and cache store behind them, K shared out where the sums go to a norm; the library's
    product and the activation kernel where K is too long for that), decode graphs for 32 and 64 requests.  Prompts
    come in portions beside decoded tokens of others; then all requests decode side by side."""
    model_dir, cfg = wide_model_dir
    if cfg["hidden_size"] > 4096:
        pytest.skip("the 1.1B and 7B widths cover the arrangement; the 70B width is replayed with four requests above")
    seqs, steps = many_live_trace(cfg, live)
    num_blocks = traces.tokens_needed(steps, round_to=16) // 16
    outputs = replay_in_process(model_dir, dtype_name, steps, 16, num_blocks, use_graphs=use_graphs, max_seqs=live)
    check_against_plain(model_dir, dtype_name, seqs, steps, outputs)


@pytest.mark.parametrize("live", [4, 20, 48])
def test_the_kernels_behind_the_switches_at_full_layer_sizes(wide_model_dir, live, monkeypatch):
    """The same replays with the decode product that has one workgroup per compute unit switched off
    (LLMSERVE_DECODE_GEMM=0: a workgroup per 16 weight rows, slices of K in LDS for 17 to 64 rows, norms as kernels of
    their own) and the shares of a split decode attention added up by the merge kernel (LLMSERVE_ATTN_MERGE=kernel)."""
    from llmserve.ops import library as ops
    from llmserve.parts import linear

    model_dir, cfg = wide_model_dir
    if cfg["hidden_size"] > 4096:
        pytest.skip("the 1.1B and 7B widths cover the arrangement")
    monkeypatch.setattr(linear, "DECODE_KERNEL", False)
    monkeypatch.setattr(ops, "MERGE_BY_KERNEL", True)
    used = set()
    for name in ("gemm_stream", "gemm_slices", "gemm_decode"):
        original = getattr(ops, name)
        monkeypatch.setattr(ops, name, (lambda name, original: lambda *a, **kw: (used.add(name), original(*a, **kw))[1])(name, original))
    seqs, steps = many_live_trace(cfg, live) if live > 4 else (None, None)
    if live <= 4:
        seqs = {f"s{i}": traces.random_ids(cfg["vocab_size"], 40 + 9 * i, 4100 + i) for i in range(live)}
        steps = traces.mixed(seqs, seed=5, live_max=4, tail=6)
    num_blocks = traces.tokens_needed(steps, round_to=16) // 16
    outputs = replay_in_process(model_dir, "bfloat16", steps, 16, num_blocks, max_seqs=max(live, 4))
    check_against_plain(model_dir, "bfloat16", seqs, steps, outputs)
    assert "gemm_stream" in used and "gemm_decode" not in used
    assert live <= 16 or cfg["hidden_size"] > 2048 or "gemm_slices" in used  # (it takes weights of up to 24 MB)


@pytest.mark.parametrize("seed", [1, 2, 3, 4])
@pytest.mark.parametrize("name", list(TINY))
def test_random_mixed_traces(model_dirs, name, seed):
    """Random numbers of requests of random lengths (up to the model's limit), mixed with random cuts, in a pool
    of exactly the pages the trace needs: both precisions against the plain implementation."""
    import random

    cfg, bs = TINY[name]
    rng = random.Random(1000 * seed + len(name))
    seqs = {f"r{i}": traces.random_ids(cfg["vocab_size"], rng.randint(1, cfg["max_position_embeddings"] - 2), 100 * seed + i)
            for i in range(rng.randint(2, 7))}
    steps = traces.mixed(seqs, seed=seed, live_max=4, tail=rng.randint(1, 8))
    num_blocks = traces.tokens_needed(steps, round_to=bs) // bs
    for dtype_name in DTYPES:
        outputs = replay_in_process(model_dirs[name], dtype_name, steps, bs, num_blocks)
        check_against_plain(model_dirs[name], dtype_name, seqs, steps, outputs)


@pytest.mark.parametrize("seed", range(10))
def test_random_configurations(tmp_path, seed):
    """Configurations drawn at random from what config.json allows (head sizes in steps of 16 up to 256, 1 to 5 KV
    heads with 1 to 32 query heads each, widths and vocabularies that are no power of two, bias or none, tied or
    untied head, one to three layers, pages of 4 to 32 tokens): a mixed trace on exactly the pages it needs, in both
    precisions, with and without graphs, against the plain implementation."""
    import random

    from llmserve.weights import write_random_model

    rng = random.Random(4000 + seed)
    head_dim = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 256])
    group = rng.choice([1, 2, 3, 4, 6, 8, 12, 16, 24, 32])
    kv_heads = rng.randint(1, max(1, min(5, 2048 // (head_dim * group))))
    heads = kv_heads * group
    cfg = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=rng.choice([97, 256, 333, 1000, 2053, 5003]),
               hidden_size=heads * head_dim, intermediate_size=8 * rng.randint(3, 60), num_hidden_layers=rng.randint(1, 3),
               num_attention_heads=heads, num_key_value_heads=kv_heads, max_position_embeddings=rng.choice([96, 160, 300]),
               rope_theta=rng.choice([1e4, 5e5, 1e6]), rms_norm_eps=rng.choice([1e-5, 1e-6]),
               tie_word_embeddings=rng.random() < 0.4, attention_bias=rng.random() < 0.3)
    block_size = rng.choice([4, 8, 16, 32])
    write_random_model(tmp_path, cfg, seed=seed)
    longest = cfg["max_position_embeddings"] - 2
    seqs = {f"s{i}": traces.random_ids(cfg["vocab_size"], rng.randint(1, longest), 100 * seed + i) for i in range(rng.randint(2, 5))}
    steps = traces.mixed(seqs, seed=seed, live_max=4, tail=rng.randint(1, 6))
    num_blocks = traces.tokens_needed(steps, round_to=block_size) // block_size
    for dtype_name in DTYPES:
        outputs = replay_in_process(tmp_path, dtype_name, steps, block_size, num_blocks, use_graphs=rng.random() < 0.7)
        check_against_plain(tmp_path, dtype_name, seqs, steps, outputs)


def test_mixed_trace_reuses_pages(model_dirs):
    """The mixed trace is only a test of reuse if it hands out more pages than the pool has."""
    seqs = sequences("a")
    steps = traces.mixed(seqs, seed=3)
    bs = TINY["a"][1]
    pool = traces.tokens_needed(steps, round_to=bs) // bs
    handed_out = sum(-(-len(ids) // bs) for ids in seqs.values())
    assert handed_out > pool


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_trace_run_program(model_dirs, tmp_path, dtype_name):
    """bin/trace_run as a user runs it: records on stdin, `done <step>` after each, files of
    little-endian floats, exit code 0 at the end of the input."""
    name = "b"
    seqs = sequences(name)
    steps = traces.mixed(seqs, seed=5)
    out = tmp_path / "out"
    cmd = [os.path.join(ROOT, "bin", "trace_run"), "--model", str(model_dirs[name]), "--dtype", dtype_name,
           "--out", str(out), "--max-tokens", str(traces.tokens_needed(steps, 64))]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for rec in steps:
        proc.stdin.write(json.dumps(rec) + "\n")
        proc.stdin.flush()
        assert proc.stdout.readline().strip() == f"done {rec['step']}"
    proc.stdin.close()
    assert proc.wait(timeout=60) == 0
    vocab = TINY[name][0]["vocab_size"]
    outputs = {}
    for rec in steps:
        wanted = sum(len(e["want"]) for e in rec["entries"])
        path = out / f"{rec['step']}.f32"
        assert path.exists() == (wanted > 0)
        if wanted:
            outputs[rec["step"]] = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(wanted, vocab).copy())
    check_against_plain(model_dirs[name], dtype_name, seqs, steps, outputs)


@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_long_decoding(model_dirs, dtype_name):
    """A short prompt, then more than two hundred tokens one by one: every page edge is crossed by a
    single token, and the replayed graphs see contexts far beyond the one they were captured at."""
    ids = traces.random_ids(TINY["b"][0]["vocab_size"], 250, 4242)
    seqs = {"long": ids}
    steps = traces.prefill_then_decode(seqs, tail=230)
    outputs = replay_in_process(model_dirs["b"], dtype_name, steps, 8, 32)
    check_against_plain(model_dirs["b"], dtype_name, seqs, steps, outputs)


@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_contexts_of_many_pages(tmp_path_factory, dtype_name):
    """1,300 tokens in pages of 8 (163 pages: the attention kernels hold 64 page ids at a time): the prompt in
    portions of 512, 300 and what is left, then tokens one by one, beside a second request that is decoding
    all the while; wanted are the last rows of each portion and every decoded token."""
    from llmserve.weights import write_random_model

    cfg = dict(TINY["a"][0], max_position_embeddings=2048)
    model_dir = tmp_path_factory.mktemp(f"long_{dtype_name}")
    write_random_model(model_dir, cfg, seed=77)
    vocab = cfg["vocab_size"]
    seqs = {"long": traces.random_ids(vocab, 1300, 5), "side": traces.random_ids(vocab, 29, 6)}
    long_ids, side_ids = seqs["long"], seqs["side"]
    steps, pos, side = [], 0, 8
    steps.append({"step": 0, "entries": [{"id": "side", "tokens": side_ids[:side], "want": list(range(side))}], "end": []})
    for n in (512, 300, 470):
        entries = [{"id": "long", "tokens": long_ids[pos:pos + n], "want": list(range(n - 4, n))},
                   {"id": "side", "tokens": [side_ids[side]], "want": [0]}]
        steps.append({"step": len(steps), "entries": entries, "end": []})
        pos, side = pos + n, side + 1
    while pos < len(long_ids):
        entries = [{"id": "long", "tokens": [long_ids[pos]], "want": [0]}]
        if side < len(side_ids):
            entries.append({"id": "side", "tokens": [side_ids[side]], "want": [0]})
            side += 1
        pos += 1
        steps.append({"step": len(steps), "entries": entries,
                      "end": (["long"] if pos == len(long_ids) else []) + (["side"] if side == len(side_ids) and "side" in
                              [e["id"] for e in entries] else [])})
    assert side == len(side_ids)
    outputs = replay_in_process(model_dir, dtype_name, steps, 8, 163 + 5)
    per_request = traces.collect(steps, outputs, partial=True)
    dtype = DTYPES[dtype_name]
    for rid, ids in seqs.items():
        ref = traces.plain_logits(model_dir, ids, dtype)
        places = sorted(per_request[rid])
        got = torch.stack([per_request[rid][p] for p in places])
        traces.assert_close(got, ref[places], dtype, f"{rid} ({dtype_name})")
    assert len(per_request["long"]) == 12 + 18 and len(per_request["side"]) == 29


@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("name", list(TINY))
def test_first_tokens(model_dirs, name, dtype_name):
    """The first tokens of a sequence: prompts of one, two and three tokens, whole and token by token
    (position 0 attends to itself only; a one-token prompt is prefill and decode at once)."""
    vocab = TINY[name][0]["vocab_size"]
    seqs = {f"s{n}": traces.random_ids(vocab, n, 70 + n) for n in (1, 2, 3, 4)}
    for steps in (traces.whole(seqs), traces.prefill_then_decode(seqs, tail=8)):
        outputs = replay_in_process(model_dirs[name], dtype_name, steps, TINY[name][1], 4)
        check_against_plain(model_dirs[name], dtype_name, seqs, steps, outputs)
    # all four at once, one token each per step
    steps, pos = [], 0
    while any(pos < len(ids) for ids in seqs.values()):
        entries = [{"id": r, "tokens": [ids[pos]], "want": [0]} for r, ids in seqs.items() if pos < len(ids)]
        steps.append({"step": pos, "entries": entries, "end": [r for r, ids in seqs.items() if pos == len(ids) - 1]})
        pos += 1
    outputs = replay_in_process(model_dirs[name], dtype_name, steps, TINY[name][1], 4)
    check_against_plain(model_dirs[name], dtype_name, seqs, steps, outputs)


@pytest.fixture(scope="module")
def sharp_dir(model_dirs, tmp_path_factory):
    """Tiny B with query and key projections scaled up, so that attention has favourites among the
    keys instead of the near-uniform weights that small random matrices give: a key that is missed,
    or read from the wrong page, then changes the logits by much more than the tolerance."""
    import shutil

    from safetensors.torch import load_file, save_file

    d = tmp_path_factory.mktemp("tiny_b_sharp")
    shutil.copy(model_dirs["b"] / "config.json", d / "config.json")
    w = load_file(str(model_dirs["b"] / "model.safetensors"))
    for k in w:
        if k.endswith("q_proj.weight") or k.endswith("k_proj.weight"):
            w[k] = w[k] * 6.0
    save_file(w, str(d / "model.safetensors"))
    return d


@pytest.mark.parametrize("mode", ["portions", "mixed"])
@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_replay_with_sharp_attention(sharp_dir, dtype_name, mode):
    seqs = sequences("b")
    ref = traces.plain_logits(sharp_dir, seqs["b5"], torch.float32)
    flat = traces.plain_logits(TINY_DIRS["b"], seqs["b5"], torch.float32) if "b" in TINY_DIRS else None
    steps = MODES[mode](seqs)
    num_blocks = traces.tokens_needed(steps, round_to=8) // 8
    outputs = replay_in_process(sharp_dir, dtype_name, steps, 8, num_blocks)
    check_against_plain(sharp_dir, dtype_name, seqs, steps, outputs)
    assert flat is None or (ref - flat).abs().max() > 1e-3


TINY_DIRS: dict = {}


@pytest.fixture(autouse=True)
def _remember_dirs(model_dirs):
    TINY_DIRS.update(model_dirs)
