"""Decode and prefill throughput of the engine on one MI355X, TinyLlama-1.1B shape, random
weights, bfloat16.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 512] [--layers L]

Prints one JSON line.  `value` is decoded tokens per second at the default batch: K timed
scheduler steps (step function + sampling + the read-back of the token ids) after W untimed
ones, with synchronisation on both sides.  `prefill` is one request of 2,048 tokens in one
step (`chunked`: the same prompt in portions of 512 tokens, the scheduler cutting it);
`roofline` prices the decode step against HBM bandwidth (every weight it uses read once, plus
the keys and values of the live requests); `points` holds decode at further batch sizes
(1, 16, 24, 32, 64: the step grows with the blocks of 16 rows) and, at the default batch, behind
contexts of 2,048 and 4,096 tokens, and with temperature, top-k and top-p for every request
instead of greedy (`decode_b8_sampled`); `serve` is a short continuous-batching run on the same model
(requests with random prompt lengths arriving at once: tokens a second, time to first token,
inter-token latency); `peak_mib` is the most device memory the process held; `measured_peaks` is
what this box delivers to a plain device copy and to a large library matrix product, the
practical ceilings beside the published ones.

    python bench.py --workload serve [--model llama2-7b] [--requests 64] [--new-tokens 256]
                    [--prompt-min 128] [--prompt-max 2048] [--pages-fraction 1.0]

runs the other workload: continuous batching of requests with seeded random prompt lengths,
all arriving at once; `value` is generated tokens per second over the whole run, with time to
first token, inter-token latency percentiles and the number of preemptions beside it.
`--pages-fraction` shrinks the cache pool below what the whole workload needs, so that
requests wait and are preempted.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # bytes/s, MI355X
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}  # dense matrix-core peaks, MI355X
PREFILL_TOKENS = 2048
PREFILL_CHUNK = 512  # the portion size of the chunked prefill measurement
MODEL_NAMES = {"tinyllama-1.1b": "TinyLlama 1.1B", "llama2-7b": "Llama-2-7B", "llama2-70b": "Llama-2-70B"}


def measured_peaks(torch) -> dict:
    """What the box delivers: a device-to-device copy of 1 GiB (read + write counted) and a
    bfloat16 library product of 8192^3."""
    def timed(fn, reps):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps

    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    copy_s = timed(lambda: dst.copy_(src), 10)
    a = torch.randn(8192, 8192, device="cuda").bfloat16()
    b = torch.randn(8192, 8192, device="cuda").bfloat16()
    mm_s = timed(lambda: torch.mm(a, b.t()), 10)
    return {"copy_GBps": round(2 * src.numel() / copy_s / 1e9, 1), "gemm_bf16_TFLOPs": round(2 * 8192 ** 3 / mm_s / 1e12, 1)}


def percentile(values, q):
    values = sorted(values)
    if not values:
        return 0.0
    return values[min(len(values) - 1, int(q * len(values)))]


def serve_summary(torch, runner, sampler, vocab: int, budget: int, max_seqs: int, requests: int = 32,
                  new_tokens: int = 64) -> dict:
    """A short continuous-batching run on a runner that is already there: `requests` requests with seeded random
    prompt lengths of 64 to 1,024 tokens that all arrive at once, `new_tokens` each (the figures of the reference's
    benchmarks/run_benchmark.py:85-91: tokens a second, time to first token, inter-token latency, peak memory)."""
    from llmserve import SamplingParams
    from llmserve.engine.scheduler import ContinuousBatchingEngine

    gen = torch.Generator().manual_seed(7)
    requests = min(requests, max_seqs)
    lengths = torch.randint(64, 1025, (requests,), generator=gen).tolist()
    lo = min(100, vocab // 4)
    texts = [torch.randint(lo, vocab, (n,), generator=gen).tolist() for n in lengths]
    need = sum(-(-(n + new_tokens + 1) // runner.block_size) + 1 for n in lengths)
    if need > runner.manager.num_blocks:
        return {}
    runner.warm_up(requests, max(lengths) + new_tokens + 1)  # a server captures its decode graphs after loading
    eng = ContinuousBatchingEngine(runner, sampler, max_num_seqs=requests, max_num_batched_tokens=budget)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ids = [eng.add_request(p, SamplingParams(max_new_tokens=new_tokens), arrival_time=t0) for p in texts]
    while eng.has_unfinished():
        eng.step()
    torch.cuda.synchronize()
    total_s = time.perf_counter() - t0
    reqs = [eng.finished[i] for i in ids]
    ttft = [r.token_times[0] - r.arrival_time for r in reqs]
    itl = [b - a for r in reqs for a, b in zip(r.token_times, r.token_times[1:])]
    return {"requests": requests, "prompt_tokens": sum(lengths), "new_tokens": new_tokens,
            "value": round(sum(len(r.generated) for r in reqs) / total_s, 1),
            "ttft_p50_ms": round(percentile(ttft, 0.5) * 1e3, 2), "itl_p50_ms": round(percentile(itl, 0.5) * 1e3, 3),
            "itl_p99_ms": round(percentile(itl, 0.99) * 1e3, 3), "preemptions": eng.stats.preemptions}


def serve(args) -> int:
    """Continuous batching of --requests requests that all arrive at time 0."""
    import torch

    from llmserve import EngineConfig, SamplingParams
    from llmserve.config import preset
    from llmserve.engine.runner import ModelRunner
    from llmserve.engine.scheduler import ContinuousBatchingEngine
    from llmserve.sampling import Sampler

    cfg = preset(args.model)
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    layers = cfg["num_hidden_layers"]
    vocab = cfg["vocab_size"]
    block_size = 16
    gen = torch.Generator().manual_seed(0)
    lengths = torch.randint(args.prompt_min, args.prompt_max + 1, (args.requests,), generator=gen).tolist()
    lo = min(100, vocab // 4)
    prompts = [torch.randint(lo, vocab, (n,), generator=gen).tolist() for n in lengths]
    longest = max(lengths) + args.new_tokens + 1
    cfg["max_position_embeddings"] = max(cfg["max_position_embeddings"], longest)
    need = sum(-(-(n + args.new_tokens + 1) // block_size) + 1 for n in lengths)
    pages = max(int(need * args.pages_fraction), -(-longest // block_size) + 2) + 1
    engine_cfg = EngineConfig(dtype=args.dtype, block_size=block_size, num_blocks=pages, max_num_seqs=args.requests,
                              max_num_batched_tokens=args.budget, seed=0)
    runner = ModelRunner.from_random(cfg, seed=0, engine_config=engine_cfg)
    sampler = Sampler(runner.device)

    def run(n_requests, new_tokens):
        eng = ContinuousBatchingEngine(runner, sampler, max_num_seqs=args.requests, max_num_batched_tokens=args.budget)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ids = [eng.add_request(p, SamplingParams(max_new_tokens=new_tokens), arrival_time=t0) for p in prompts[:n_requests]]
        steps = 0
        while eng.has_unfinished():
            eng.step()
            steps += 1
        torch.cuda.synchronize()
        return eng, [eng.finished[i] for i in ids], time.perf_counter() - t0, steps

    run(min(4, args.requests), 8)  # warm-up: kernels loaded
    runner.warm_up(args.requests, longest)  # the decode graphs of every batch size, as a server does after loading
    runner.rows_asked = runner.rows_run = 0
    eng, reqs, total_s, steps = run(args.requests, args.new_tokens)
    generated = sum(len(r.generated) for r in reqs)
    ttft = [r.token_times[0] - r.arrival_time for r in reqs]
    itl = [b - a for r in reqs for a, b in zip(r.token_times, r.token_times[1:])]
    line = {
        "metric": "continuous batching: generated tok/s over the whole run",
        "value": round(generated / total_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": 0,
        "ms_per_step": round(total_s / steps * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": args.model, "requests": args.requests, "prompt_min": args.prompt_min,
                   "prompt_max": args.prompt_max, "prompt_tokens": sum(lengths), "new_tokens": args.new_tokens,
                   "parallelism": "single-gpu", "layers": layers, "layers_full": full_layers, "budget": args.budget,
                   "pages": pages, "pages_needed": need, "block_size": block_size, "weights": "random"},
        "total_s": round(total_s, 3),
        "ttft_ms": {"p50": round(percentile(ttft, 0.5) * 1e3, 2), "p90": round(percentile(ttft, 0.9) * 1e3, 2),
                    "max": round(max(ttft) * 1e3, 2)},
        "itl_ms": {"p50": round(percentile(itl, 0.5) * 1e3, 3), "p90": round(percentile(itl, 0.9) * 1e3, 3),
                   "p99": round(percentile(itl, 0.99) * 1e3, 3), "max": round(max(itl) * 1e3, 3)},
        "preemptions": eng.stats.preemptions,
        "peak_mib": round(torch.cuda.max_memory_allocated() / 2 ** 20, 1),
        # rows the steps held, rows that ran with the padding of buckets and graphs, and the padded fraction
        "rows": {"asked": runner.rows_asked, "run": runner.rows_run,
                 "padding": round(runner.rows_run / max(runner.rows_asked, 1) - 1, 4)},
    }
    print(json.dumps(line))
    return 0


def gemv(args) -> int:
    """The decode step's matrix products one by one, as the step's parts launch them (the kernel, the epilogue and
    the prologue they choose for the row count), at 1, 8, 32 and 64 rows.  Every launch of a chain takes the next of
    several copies of its weight, a gigabyte in all, so that nothing is left in the 256 MB memory-side cache from the
    launch before (the convention of the reference's benchmarks/bench_decode_matmul.py:28,78-81); the chain is
    captured as a graph, so the figure is device time per launch, start and drain included."""
    import torch

    from llmserve.config import preset
    from llmserve.ops import library as ops
    from llmserve.parts import linear as lin

    cfg = preset(args.model)
    h, inter, vocab = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = h // nh
    block_size = 16
    ops.ensure_built("bfloat16")
    dev = torch.device("cuda:0")
    shapes = {"qkv": ((nh + 2 * nkv) * d, h), "o_proj": (h, nh * d), "gate_up": (2 * inter, h), "down_proj": (h, inter),
              "lm_head": (vocab, h)}
    inv_freq = (1.0 / (cfg.get("rope_theta", 10000.0) ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).to(dev)
    results = {}
    for name, (n, k) in shapes.items():
        copies = max(2, -(-(1 << 30) // (n * k * 2)))
        weights = [torch.randn(n, k, device=dev, dtype=torch.bfloat16) * 0.02 for _ in range(copies)]
        norm_weight = torch.ones(k, device=dev, dtype=torch.bfloat16)
        for m in (1, 8, 32, 64):
            x = torch.randn(m, k, device=dev, dtype=torch.bfloat16)
            decode = lin.decode_product(x, weights[0])
            norm = (norm_weight, 1e-5) if decode and m <= ops.GEMM_DECODE_NORM_ROWS else None
            how = "gemm_decode" if decode else "gemm_stream" if lin.few_rows(m, weights[0]) else "library"
            if name == "gate_up":
                out = torch.empty(m, inter, device=dev, dtype=torch.bfloat16)
                if decode:
                    run = lambda w: ops.gemm_decode(out, x, w, swiglu=True, norm=norm)  # noqa: E731
                elif lin.few_rows(m, weights[0]):
                    run = lambda w: ops.gemm_stream(out, x, w, swiglu=True)  # noqa: E731
                else:
                    wide = torch.empty(m, n, device=dev, dtype=torch.bfloat16)
                    run = lambda w: ops.silu_mul(out, torch.mm(x, w.t(), out=wide))  # noqa: E731
                    how = "library + silu_mul"
            elif name == "qkv":
                positions = torch.randint(500, 600, (m,), dtype=torch.int32, device=dev)
                slots = torch.randperm(64 * block_size, device=dev)[:m].to(torch.int32)
                k_pool = torch.zeros(64, nkv, block_size, d, dtype=torch.bfloat16, device=dev)
                v_pool = torch.zeros(64, nkv, d, block_size, dtype=torch.bfloat16, device=dev)
                rope = dict(n_heads=nh, n_kv_heads=nkv, head_dim=d, inv_freq=inv_freq, positions=positions, slots=slots,
                            k_pool=k_pool, v_pool=v_pool, block_size=block_size)
                q = torch.empty(m, nh * d, dtype=torch.bfloat16, device=dev)
                if decode:
                    rope["angles"] = ops.rotary_angles(positions, inv_freq)
                    run = lambda w: ops.gemm_decode(q, x, w, rope=rope, norm=norm)  # noqa: E731
                elif lin.few_rows(m, weights[0]):
                    run = lambda w: ops.gemm_stream(q, x, w, rope=rope)  # noqa: E731
                else:
                    wide = torch.empty(m, n, device=dev, dtype=torch.bfloat16)
                    run = lambda w: ops.rope_store(torch.mm(x, w.t(), out=wide), inv_freq, positions, slots, k_pool,  # noqa: E731
                                                   v_pool, nh, nkv, d, block_size)
                    how = "library + rope_store"
            elif name in ("o_proj", "down_proj"):
                residual = torch.zeros(m, n, device=dev, dtype=torch.bfloat16)
                if lin.adds_residual_in_epilogue(x, weights[0]):
                    run = lambda w: ops.gemm_decode(None, x, w, residual=residual)  # noqa: E731
                    how = "gemm_decode + residual"
                else:
                    run = lambda w: lin.linear_partial_sums(x, w) or lin.linear(x, w)  # noqa: E731
                    how = "partial sums" if lin.linear_partial_sums(x, weights[0]) is not None else how
            else:
                run = lambda w: lin.linear(x, w, out_dtype=torch.float32)  # noqa: E731
                if m <= lin.STREAM_LARGE_ROWS and n * k * 2 >= lin.STREAM_LARGE_BYTES:
                    how = "gemm_stream"
            if norm is not None and name in ("qkv", "gate_up"):
                how += " + norm"
            for w in weights[:2]:
                run(w)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for w in weights:
                    run(w)
            graph.replay()
            torch.cuda.synchronize()
            reps = max(1, 200 // copies)
            t0 = time.perf_counter()
            for _ in range(reps):
                graph.replay()
            torch.cuda.synchronize()
            us = (time.perf_counter() - t0) / (reps * copies) * 1e6
            results[f"{name}_m{m}"] = {"us": round(us, 2), "GBps": round(n * k * 2 / us / 1e3, 1), "kernel": how}
        del weights
    line = {"metric": "decode matrix products alone: microseconds per launch, weights streamed from HBM",
            "value": results["gate_up_m8"]["us"], "unit": "us", "n_gpus": 1, "steps": 0, "warmup": 0, "ms_per_step": 0.0,
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"model": args.model, "hidden": h, "intermediate": inter, "vocab": vocab, "heads": nh,
                       "kv_heads": nkv, "head_dim": d, "parallelism": "single-gpu"},
            "gemv": results}
    print(json.dumps(line))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=512)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--model", default="tinyllama-1.1b")
    ap.add_argument("--no-points", action="store_true", help="skip the further batch sizes")
    ap.add_argument("--points", default="1,16,24,32,64", help="further batch sizes to measure decoding at")
    ap.add_argument("--context-points", default="2048,4096", help="further context lengths to measure decoding at (default batch)")
    ap.add_argument("--no-serve", action="store_true", help="skip the short continuous-batching run")
    ap.add_argument("--phase", choices=["all", "decode", "prefill", "gemv"], default="all",
                    help="run one phase only (for profiles; the line then holds zeros for the other); gemv: the "
                         "decode products alone, each over copies of its weight that do not fit the caches")
    ap.add_argument("--workload", choices=["steps", "serve"], default="steps")
    ap.add_argument("--requests", type=int, default=64)
    ap.add_argument("--new-tokens", type=int, default=256)
    ap.add_argument("--prompt-min", type=int, default=128)
    ap.add_argument("--prompt-max", type=int, default=2048)
    ap.add_argument("--pages-fraction", type=float, default=1.0)
    ap.add_argument("--budget", type=int, default=2048, help="serve: tokens per step (max_num_batched_tokens)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU engine")
        return 2
    if args.workload == "serve":
        return serve(args)
    if args.phase == "gemv":
        return gemv(args)

    import torch

    from llmserve import EngineConfig, SamplingParams
    from llmserve.config import preset
    from llmserve.engine.runner import ModelRunner
    from llmserve.engine.scheduler import ContinuousBatchingEngine
    from llmserve.sampling import Sampler

    cfg = preset(args.model)
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    layers = cfg["num_hidden_layers"]
    h, inter, vocab = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = h // nh
    elem = 2 if args.dtype == "bfloat16" else 4
    block_size = 16
    extra = not args.no_points and args.phase in ("all", "decode")
    point_batches = [int(b) for b in args.points.split(",") if b] if extra else []
    point_contexts = [int(c) for c in args.context_points.split(",") if c] if extra else []
    max_batch = max([args.batch] + point_batches)
    budget = max(PREFILL_TOKENS, max_batch)

    def new_tokens_for(batch, context):
        # requests whose prompt went in first decode while the others' prompts still go in (and take a growing share
        # of every step's budget from them)
        return args.warmup + args.steps + 2 * -(-batch * context // budget) + 8

    runs = [(args.batch, args.context)] + [(b, args.context) for b in point_batches] + [(args.batch, c) for c in point_contexts]
    longest = max(c + new_tokens_for(b, c) + 1 for b, c in runs)
    cfg["max_position_embeddings"] = max(cfg["max_position_embeddings"], PREFILL_TOKENS + 8, longest)
    pages = max([b * -(-(c + new_tokens_for(b, c) + 1) // block_size) for b, c in runs]
                + [-(-(PREFILL_TOKENS + 8) // block_size)]) + 16
    engine_cfg = EngineConfig(dtype=args.dtype, block_size=block_size, num_blocks=pages, max_num_seqs=max_batch,
                              max_num_batched_tokens=budget, seed=0)
    runner = ModelRunner.from_random(cfg, seed=0, engine_config=engine_cfg)
    sampler = Sampler(runner.device)
    gen = torch.Generator().manual_seed(0)

    def prompts(n, length):
        lo = min(100, vocab // 4)
        return [torch.randint(lo, vocab, (length,), generator=gen).tolist() for _ in range(n)]

    def decode_rate(batch, context=args.context, **sampling):
        eng = ContinuousBatchingEngine(runner, sampler, max_num_seqs=batch,
                                       max_num_batched_tokens=engine_cfg.max_num_batched_tokens)
        for p in prompts(batch, context):
            eng.add_request(p, SamplingParams(max_new_tokens=new_tokens_for(batch, context), **sampling))
        while eng.waiting or any(r.num_tokens - r.num_computed_tokens > 1 for r in eng.running):
            eng.step()  # prompts in
        for _ in range(args.warmup):
            eng.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            eng.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert len(eng.running) == batch and eng.stats.preemptions == 0
        eng.run_until_complete()
        return batch * args.steps / dt, dt / args.steps

    def prefill_time(budget=PREFILL_TOKENS):
        eng = ContinuousBatchingEngine(runner, sampler, max_num_seqs=1, max_num_batched_tokens=budget)
        times = []
        for i in range(4):
            eng.add_request(prompts(1, PREFILL_TOKENS)[0], SamplingParams(max_new_tokens=1))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            while eng.has_unfinished():
                eng.step()  # the whole prompt in one step (or in portions of `budget`), first token sampled and read back
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        return sorted(times[1:])[len(times[1:]) // 2]

    value, step_s = decode_rate(args.batch) if args.phase != "prefill" else (0.0, float("inf"))
    points = {}
    for b in point_batches:
        points[f"decode_b{b}"] = round(decode_rate(b)[0], 1)
    for c in point_contexts:
        points[f"decode_b{args.batch}_ctx{c}"] = round(decode_rate(args.batch, c)[0], 1)
    if extra:  # every request with temperature, top-k and top-p (the device sampler's longest path) instead of greedy
        points[f"decode_b{args.batch}_sampled"] = round(decode_rate(args.batch, temperature=0.8, top_k=40, top_p=0.95)[0], 1)
    served = serve_summary(torch, runner, sampler, vocab, budget, max_batch) if extra and not args.no_serve else {}
    pre_s = prefill_time() if args.phase != "decode" else float("inf")
    chunked_s = prefill_time(PREFILL_CHUNK) if args.phase == "all" else float("inf")
    peaks = measured_peaks(torch) if args.phase == "all" else {}

    # bytes a decode step must read: every matrix and norm once, the rows of the embedding it
    # gathers, and the keys and values of the live requests at their mean length in the timed steps
    per_layer = ((nh + 2 * nkv) * d * h + h * nh * d + 3 * h * inter + 2 * h) * elem
    weight_bytes = layers * per_layer + (vocab * h + h) * elem + args.batch * h * elem
    mean_ctx = args.context + args.warmup + args.steps / 2
    kv_bytes = args.batch * mean_ctx * 2 * layers * nkv * d * elem
    achieved = (weight_bytes + kv_bytes) / step_s
    # flops of the prefill step: the linear layers on every token, causal attention, one row of logits
    t = PREFILL_TOKENS
    linear = 2 * t * layers * ((nh + 2 * nkv) * d * h + h * nh * d + 3 * h * inter)
    attention = layers * 4 * nh * d * t * (t + 1) / 2
    flops = linear + attention + 2 * vocab * h
    def ms(seconds):
        return round(seconds * 1e3, 4) if seconds != float("inf") else 0.0

    line = {
        "metric": f"decode tok/s at batch 1/8/64; prefill tok/s at 2,048 tokens ({MODEL_NAMES.get(args.model, args.model)})",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms(step_s), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": args.model, "global_batch": args.batch, "seq_len": args.context,
                   "parallelism": "single-gpu", "layers": layers, "layers_full": full_layers, "hidden": h,
                   "heads": nh, "kv_heads": nkv, "head_dim": d, "intermediate": inter, "vocab": vocab,
                   "block_size": block_size, "weights": "random", "prefill_tokens": PREFILL_TOKENS},
        "prefill": {"value": round(t / pre_s, 1), "tokens": t, "ms": ms(pre_s),
                    "frac": round(flops / pre_s / PEAK_FLOPS[args.dtype], 4),
                    "chunked": {"budget": PREFILL_CHUNK, "ms": ms(chunked_s)}},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4)},
        "points": points,
        "serve": served,
        "peak_mib": round(torch.cuda.max_memory_allocated() / 2 ** 20, 1),
        "measured_peaks": peaks,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
