"""Generation through the Python entry point and the command line, on the GPU."""

import os
import subprocess
import sys

import pytest
import torch

import plain_llama
import traces
from conftest import ROOT, TINY

pytestmark = pytest.mark.gpu


def _llm(model_dir, name, dtype, **kw):
    from llmserve import LLM, EngineConfig

    opts = dict(block_size=TINY[name][1], num_blocks=64, max_num_seqs=4, max_num_batched_tokens=24)
    opts.update(kw)
    return LLM(model_dir, dtype=dtype, engine=EngineConfig(**opts))


@pytest.mark.parametrize("name,lengths,new", [("a", [5, 17, 33], 16), ("b", [1, 7, 40, 64, 100], 24)])
def test_greedy_generation_matches_plain(model_dirs, name, lengths, new):
    from llmserve import SamplingParams

    vocab = TINY[name][0]["vocab_size"]
    prompts = [traces.random_ids(vocab, n, 300 + i) for i, n in enumerate(lengths)]
    cfg, w = plain_llama.read_model_dir(model_dirs[name], torch.float32)
    want = [plain_llama.generate(cfg, w, p, new, torch.float32) for p in prompts]
    llm = _llm(model_dirs[name], name, "float32")
    results = llm.generate(prompts, SamplingParams(max_new_tokens=new))
    assert [r.tokens for r in results] == want
    assert all(r.finish_reason == "length" and len(r.step_latencies_s) == new - 1 and r.ttft_s > 0 for r in results)
    assert llm.engine.manager.num_free_blocks == 64
    # the baseline without a cache between tokens gives the same tokens
    assert llm.generate_naive(prompts[1], SamplingParams(max_new_tokens=6)).tokens == want[1][:6]


@pytest.mark.parametrize("name,lengths,new", [("a", [5, 17, 33], 16), ("b", [1, 7, 40, 64, 100], 24)])
def test_generation_without_graphs_feeds_the_sampled_ids(model_dirs, name, lengths, new):
    """With graphs off every decode step is launched kernel by kernel and takes its tokens from the host:
    the scheduler must then wait for the ids instead of starting the next step on placeholders."""
    from llmserve import SamplingParams

    vocab = TINY[name][0]["vocab_size"]
    prompts = [traces.random_ids(vocab, n, 300 + i) for i, n in enumerate(lengths)]
    cfg, w = plain_llama.read_model_dir(model_dirs[name], torch.float32)
    want = [plain_llama.generate(cfg, w, p, new, torch.float32) for p in prompts]
    llm = _llm(model_dirs[name], name, "float32", use_graphs=False)
    assert llm.runner.takes_device_tokens is False
    assert [r.tokens for r in llm.generate(prompts, SamplingParams(max_new_tokens=new))] == want
    from llmserve.engine.runner import StepEntry

    llm.runner.add_sequence("x")
    with pytest.raises(ValueError, match="from the host only"):
        llm.runner.step([StepEntry("x", [0], [0])], device_tokens=torch.zeros(1, dtype=torch.int32, device="cuda"))
    llm.runner.free_sequence("x")
    # seeded temperature sampling: the same tokens as with graphs, whatever launches the steps
    params = [SamplingParams(temperature=0.8, seed=40 + i, max_new_tokens=new) for i in range(len(prompts))]
    eager = [r.tokens for r in llm.generate(prompts, params)]
    replayed = [r.tokens for r in _llm(model_dirs[name], name, "float32").generate(prompts, params)]
    assert eager == replayed and len({tuple(t) for t in eager}) == len(prompts)


@pytest.mark.parametrize("name", ["a", "b"])
def test_preemption_by_recompute_keeps_greedy_tokens(model_dirs, name):
    """14 pages of 4 tokens and four requests of 6 + 14 tokens cannot all grow: some are thrown
    out and recomputed (the reference's case, tests/test_scheduler.py:69-82 there)."""
    from llmserve import SamplingParams

    vocab = TINY[name][0]["vocab_size"]
    prompts = [traces.random_ids(vocab, 6, 50 + i) for i in range(4)]
    cfg, w = plain_llama.read_model_dir(model_dirs[name], torch.float32)
    want = [plain_llama.generate(cfg, w, p, 14, torch.float32) for p in prompts]
    tight = _llm(model_dirs[name], name, "float32", block_size=4, num_blocks=14)
    assert [r.tokens for r in tight.generate(prompts, SamplingParams(max_new_tokens=14))] == want
    assert tight.engine.stats.preemptions > 0
    assert tight.engine.manager.num_free_blocks == 14


@pytest.mark.parametrize("name,seed", [("a", 1), ("a", 2), ("b", 3), ("b", 4)])
def test_random_serving_workloads_keep_greedy_tokens(model_dirs, name, seed):
    """Requests that arrive while others run, a pool so small that some are thrown out and recomputed, a token
    budget that cuts prompts anywhere, and requests stopped from outside in the middle: every request that runs to
    its end has the tokens of the plain implementation, and every page comes back."""
    import random

    from llmserve import EngineConfig, SamplingParams
    from llmserve.engine.runner import ModelRunner
    from llmserve.engine.scheduler import ContinuousBatchingEngine
    from llmserve.sampling import Sampler

    rng = random.Random(seed)
    vocab = TINY[name][0]["vocab_size"]
    cfg, w = plain_llama.read_model_dir(model_dirs[name], torch.float32)
    block_size = rng.choice([4, 8])
    jobs = []
    for i in range(10):
        prompt = traces.random_ids(vocab, rng.randint(1, 48), 900 + 16 * seed + i)
        jobs.append(dict(prompt=prompt, new=rng.randint(1, 18), arrive=rng.randint(0, 25), abort_at=None))
    for job in rng.sample(jobs, 2):
        job["abort_at"] = job["arrive"] + rng.randint(1, 8)
    longest = max(len(j["prompt"]) + j["new"] for j in jobs)
    pages = -(-longest // block_size) + rng.randint(2, 10)  # the longest request fits; several at once do not
    runner = ModelRunner.from_folder(model_dirs[name], EngineConfig(dtype="float32", block_size=block_size, num_blocks=pages,
                                                                   max_num_seqs=4, max_num_batched_tokens=rng.choice([8, 24, 64])))
    engine = ContinuousBatchingEngine(runner, Sampler(runner.device), max_num_seqs=4,
                                      max_num_batched_tokens=runner.engine_config.max_num_batched_tokens)
    ids, step = {}, 0
    while step < 400 and (engine.has_unfinished() or len(ids) < len(jobs)):
        for i, job in enumerate(jobs):
            if job["arrive"] == step:
                ids[i] = engine.add_request(job["prompt"], SamplingParams(max_new_tokens=job["new"]))
            if job["abort_at"] == step and i in ids:
                engine.abort(ids[i])
        engine.step()
        step += 1
    assert not engine.has_unfinished() and len(ids) == len(jobs)
    finished = 0
    for i, job in enumerate(jobs):
        request = engine.finished[ids[i]]
        want = plain_llama.generate(cfg, w, job["prompt"], job["new"], torch.float32)
        if request.finish_reason == "abort":
            assert job["abort_at"] is not None and request.generated == want[: len(request.generated)]
        else:
            assert request.finish_reason == "length" and request.generated == want, (i, job)
            finished += 1
    assert finished >= len(jobs) - 2
    assert engine.manager.num_free_blocks == pages
    engine.manager.check_invariants()


def test_bfloat16_generation_follows_plain_logits(model_dirs):
    """In bfloat16 greedy ties can fall either way, so the check is on the logits: every token the
    engine picks must be (nearly) the best one under the plain bfloat16 implementation."""
    from llmserve import SamplingParams

    name = "b"
    vocab = TINY[name][0]["vocab_size"]
    prompt = traces.random_ids(vocab, 40, 77)
    llm = _llm(model_dirs[name], name, "bfloat16")
    tokens = llm.generate([prompt], SamplingParams(max_new_tokens=12))[0].tokens
    ref = traces.plain_logits(model_dirs[name], prompt + tokens, torch.bfloat16)
    max_tol, _ = traces.tolerance(torch.bfloat16, ref)
    for i, tok in enumerate(tokens):
        row = ref[len(prompt) - 1 + i]
        assert row.max() - row[tok] <= 2 * max_tol, f"token {i} = {tok} is not near the top of the plain logits"


@pytest.mark.parametrize("name", ["a", "b"])
def test_bfloat16_generation_of_many_requests_at_once(model_dirs, name):
    """48 requests decoding in one step: from 17 and from 33 rows on the products of a step take other kernels
    (a slice of all rows in LDS, partial sums added up by the norm and by the rotation), replayed from a graph."""
    from llmserve import SamplingParams

    vocab = TINY[name][0]["vocab_size"]
    prompts = [traces.random_ids(vocab, 3 + (5 * i) % 18, 500 + i) for i in range(48)]
    llm = _llm(model_dirs[name], name, "bfloat16", num_blocks=48 * 8, max_num_seqs=48, max_num_batched_tokens=256)
    results = llm.generate(prompts, SamplingParams(max_new_tokens=10))
    assert llm.engine.stats.preemptions == 0
    for prompt, result in zip(prompts, results):
        ref = traces.plain_logits(model_dirs[name], prompt + result.tokens, torch.bfloat16)
        max_tol, _ = traces.tolerance(torch.bfloat16, ref)
        for i, tok in enumerate(result.tokens):
            row = ref[len(prompt) - 1 + i]
            assert row.max() - row[tok] <= 2 * max_tol, f"token {i} = {tok} is not near the top of the plain logits"


def test_temperature_sampling_is_seeded_and_matches_plain_sampler(model_dirs):
    from llmserve import SamplingParams
    from llmserve.sampling import uniform

    name = "b"
    vocab = TINY[name][0]["vocab_size"]
    prompts = [traces.random_ids(vocab, n, 500 + i) for i, n in enumerate([1, 7, 40, 64, 100])]
    params = [SamplingParams(temperature=0.8, seed=40 + i, max_new_tokens=24) for i in range(5)]
    llm = _llm(model_dirs[name], name, "float32")
    first = [r.tokens for r in llm.generate(prompts, params)]
    assert first == [r.tokens for r in _llm(model_dirs[name], name, "float32", max_num_batched_tokens=64)
                     .generate(prompts, params)]
    assert len({tuple(t) for t in first}) == 5
    # each sampled token is what the plain sampler picks from the plain logits with the same uniform number
    cfg, w = plain_llama.read_model_dir(model_dirs[name], torch.float32)
    for p, sp, toks in list(zip(prompts, params, first))[:3]:
        logits = plain_llama.forward(cfg, w, p + toks, torch.float32)
        for i, tok in enumerate(toks):
            row = logits[len(p) - 1 + i]
            u = uniform(sp.seed, i)
            cdf = plain_llama.filtered_probs(row, 0.8, 0, 1.0).cumsum(-1)
            lo = float(cdf[tok - 1]) if tok > 0 else 0.0
            assert lo - 1e-5 <= u < float(cdf[tok]) + 1e-5, (i, tok, u, lo, float(cdf[tok]))


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_requests_with_their_own_sampling_options_share_a_batch(model_dirs, dtype_name):
    """Greedy requests beside requests with temperature, top-k, top-p and seeds of their own, in one batch through
    the scheduler and the device sampler (ids read a step late; the reference's engine test runs top_k=20:
    tests/test_scheduler.py:122-131 there).  Every token is what the plain sampler picks from the plain logits
    with the same uniform number: exactly in 32-bit; in bfloat16 within what the logits' rounding moves the
    distribution, and never a token that the filters of the plain logits exclude by more than that rounding."""
    from llmserve import SamplingParams
    from llmserve.sampling import uniform

    name = "b"
    vocab = TINY[name][0]["vocab_size"]
    dtype = getattr(torch, dtype_name)
    prompts = [traces.random_ids(vocab, n, 800 + i) for i, n in enumerate([3, 30, 11, 64, 7, 19])]
    params = [SamplingParams(max_new_tokens=14),
              SamplingParams(temperature=0.9, top_k=20, seed=11, max_new_tokens=14),
              SamplingParams(temperature=1.3, top_p=0.9, seed=12, max_new_tokens=14),
              SamplingParams(max_new_tokens=9),
              SamplingParams(temperature=0.7, top_k=5, top_p=0.8, seed=13, max_new_tokens=14),
              SamplingParams(temperature=1.0, seed=14, max_new_tokens=14)]
    llm = _llm(model_dirs[name], name, dtype_name, max_num_batched_tokens=48)
    results = [r.tokens for r in llm.generate(prompts, params)]
    assert llm.engine.stats.steps > 14 and [len(t) for t in results] == [p.max_new_tokens for p in params]
    if dtype_name == "float32":  # another way of cutting the same work: the same tokens
        again = _llm(model_dirs[name], name, dtype_name, max_num_batched_tokens=2048, use_graphs=False)
        assert [r.tokens for r in again.generate(prompts, params)] == results
    cfg, w = plain_llama.read_model_dir(model_dirs[name], dtype)
    for p, sp, toks in zip(prompts, params, results):
        logits = plain_llama.forward(cfg, w, p + toks, dtype).float()
        max_tol, _ = traces.tolerance(dtype, logits)
        for i, tok in enumerate(toks):
            row = logits[len(p) - 1 + i]
            if sp.temperature == 0:
                slack = 0.0 if dtype_name == "float32" else 2 * max_tol
                assert row.max() - row[tok] <= slack, (i, tok)
                continue
            probs = plain_llama.filtered_probs(row, sp.temperature, sp.top_k, sp.top_p)
            cdf = probs.cumsum(-1)
            u = uniform(sp.seed, i)
            lo = float(cdf[tok - 1]) if tok > 0 else 0.0
            # the logits' rounding moves every probability by about that much relative to itself, so a cumulated sum
            # by no more than that in all
            slack = 1e-5 if dtype_name == "float32" else 4 * max_tol / sp.temperature
            assert lo - slack <= u < float(cdf[tok]) + slack, (i, tok, u, lo, float(cdf[tok]))
            if sp.top_k:  # inside the plain top-k, or tied with its last member within the rounding
                kth = row.topk(sp.top_k).values[-1]
                assert row[tok] >= kth - (0.0 if dtype_name == "float32" else 2 * max_tol), (i, tok)


def test_warm_up_captures_the_decode_graphs_ahead(model_dirs):
    """After `warm_up` no decode step has to capture anything, and the tokens are the same as without it."""
    from llmserve import SamplingParams

    name = "a"
    prompts = [traces.random_ids(TINY[name][0]["vocab_size"], n, 300 + i) for i, n in enumerate([5, 17, 33])]
    cold = _llm(model_dirs[name], name, "bfloat16")
    want = [r.tokens for r in cold.generate(prompts, SamplingParams(max_new_tokens=12))]
    warm = _llm(model_dirs[name], name, "bfloat16")
    made = warm.warm_up()
    assert made == 3 * 1 and warm.warm_up() == 0  # capacities 1, 2, 4 at the one reach that 128 positions need
    before = set(warm.runner._graphs)
    assert [r.tokens for r in warm.generate(prompts, SamplingParams(max_new_tokens=12))] == want
    assert set(warm.runner._graphs) == before
    assert _llm(model_dirs[name], name, "float32", use_graphs=False).warm_up() == 0


def test_eos_stops_generation(model_dirs):
    from llmserve import SamplingParams

    prompt = traces.random_ids(256, 10, 9)
    llm = _llm(model_dirs["a"], "a", "float32")
    first = llm.generate([prompt], SamplingParams(max_new_tokens=1))[0].tokens[0]
    r = llm.generate([prompt], SamplingParams(max_new_tokens=50, eos_token_id=first))[0]
    assert r.tokens == [first] and r.finish_reason == "stop"
    with pytest.raises(ValueError):
        llm.generate([[1] * 128], SamplingParams(max_new_tokens=5))  # beyond max_position_embeddings


def test_command_line(model_dirs):
    env = dict(os.environ, PYTHONPATH=ROOT)
    out = subprocess.run([sys.executable, "-m", "llmserve.cli", "--model", "tiny", "--max-new-tokens", "8",
                          "--dtype", "float32"], capture_output=True, text=True, env=env, timeout=120)
    assert out.returncode == 0, out.stderr
    lines = out.stdout.strip().splitlines()
    assert len(eval(lines[0])) == 8 and lines[-1].startswith("[kv_cache] ttft=") and "peak mem=" in lines[-1]
    naive = subprocess.run([sys.executable, "-m", "llmserve.cli", "--model", "tiny", "--max-new-tokens", "8",
                            "--dtype", "float32", "--mode", "naive"], capture_output=True, text=True, env=env, timeout=120)
    assert naive.returncode == 0, naive.stderr
    assert naive.stdout.strip().splitlines()[0] == lines[0]  # same tokens with and without the cache
    folder = subprocess.run([sys.executable, "-m", "llmserve.cli", "--model", str(model_dirs["a"]), "--prompt-ids",
                             "5,6,7,8", "--max-new-tokens", "4", "--block-size", "16", "--num-blocks", "8"],
                            capture_output=True, text=True, env=env, timeout=120)
    assert folder.returncode == 0, folder.stderr
    assert len(eval(folder.stdout.strip().splitlines()[0])) == 4


def test_generation_without_the_library_product(model_dirs):
    """LLMSERVE_GEMM=own: every matrix product on this repository's kernels, same tokens."""
    code = ("import sys; sys.path[:0] = [%r, %r]\n"
            "import torch, plain_llama, traces\n"
            "from llmserve import LLM, EngineConfig, SamplingParams\n"
            "from llmserve.parts import linear\n"
            "assert linear.OWN_KERNELS_ONLY\n"
            "d = %r\n"
            "prompts = [traces.random_ids(333, n, 300 + i) for i, n in enumerate([7, 100])]\n"
            "llm = LLM(d, dtype='bfloat16', engine=EngineConfig(block_size=8, num_blocks=64, max_num_seqs=4, max_num_batched_tokens=128))\n"
            "toks = [r.tokens for r in llm.generate(prompts, SamplingParams(max_new_tokens=8))]\n"
            "for p, t in zip(prompts, toks):\n"
            "    ref = traces.plain_logits(d, p + t, torch.bfloat16)\n"
            "    tol = traces.tolerance(torch.bfloat16, ref)[0]\n"
            "    assert all(ref[len(p) - 1 + i].max() - ref[len(p) - 1 + i][x] <= 2 * tol for i, x in enumerate(t))\n"
            "print('ok')\n") % (ROOT, os.path.join(ROOT, "tests"), str(model_dirs["b"]))
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120,
                         env=dict(os.environ, LLMSERVE_GEMM="own"))
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stderr[-2000:]
