"""Replays on the GPU against the plain implementation: each request alone and whole; most
of it in one step and the last 32 tokens one by one; in portions of changing size; mixed,
with so few pages that they are used again.  32-bit and bfloat16, both tiny configurations."""

import json
import os
import subprocess
import sys

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


def replay_in_process(model_dir, dtype_name, steps, block_size, num_blocks, use_graphs=True):
    from llmserve.config import EngineConfig
    from llmserve.engine.replay import Replayer
    from llmserve.engine.runner import ModelRunner

    runner = ModelRunner.from_folder(model_dir, EngineConfig(dtype=dtype_name, block_size=block_size,
                                                              num_blocks=num_blocks, max_num_seqs=4,
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
    assert runner.manager.num_free_slots == 4, "state slots were not all returned"
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
