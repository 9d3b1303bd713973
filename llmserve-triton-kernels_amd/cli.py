"""Command line in the manner of the reference's `python -m llmserve.cli`
(src/llmserve/cli.py:17-53): the same flags with the same meanings (--model, --prompt,
--max-new-tokens, --mode {naive,kv_cache}, --temperature, --device, --dtype) and the same
last line `[mode] ttft=... ms | decode=... tok/s | peak mem=... MiB`.

    python -m llmserve.cli --model tiny                      # random weights, token ids in and out
    python -m llmserve.cli --model DIR --prompt-ids 1,2,3 --max-new-tokens 32
    python -m llmserve.cli --model tinyllama-1.1b --random-weights --dtype bfloat16

`--model` is a local folder (config.json + safetensors; text prompts need its tokenizer
files), the literal `tiny` (the reference's offline mode: random weights, prompt ids
10..25), or, with --random-weights, the name of a size.
"""

from __future__ import annotations

import argparse
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="llmserve.cli", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="local folder, 'tiny', or a size name with --random-weights")
    ap.add_argument("--prompt", default="Explain KV caching in one paragraph.")
    ap.add_argument("--prompt-ids", default=None, help="comma-separated token ids instead of --prompt")
    ap.add_argument("--max-new-tokens", type=int, default=64)
    ap.add_argument("--mode", choices=["naive", "kv_cache"], default="kv_cache")
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--device", default="cuda", help="GPU to run on (there is no CPU path)")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--random-weights", action="store_true", help="--model names a size; fill it from --seed")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--num-blocks", type=int, default=None)
    ap.add_argument("--kv-mem-mib", type=float, default=None, help="cache budget instead of --num-blocks")
    ap.add_argument("--max-num-batched-tokens", type=int, default=2048)
    args = ap.parse_args(argv)

    if not args.device.startswith("cuda"):
        ap.error("this engine runs on the GPU only; --device must be cuda or cuda:N")

    from .config.engine_config import EngineConfig
    from .engine.llm import LLM
    from .sampling.params import SamplingParams

    engine = EngineConfig(dtype=args.dtype, block_size=args.block_size, num_blocks=args.num_blocks,
                          kv_bytes=int(args.kv_mem_mib * 2**20) if args.kv_mem_mib else None,
                          max_num_batched_tokens=args.max_num_batched_tokens, max_num_seqs=8, seed=args.seed)
    device = "cuda:0" if args.device == "cuda" else args.device
    tok = None
    eos = None
    if args.model == "tiny" or args.random_weights:
        if engine.num_blocks is None and engine.kv_bytes is None:
            engine.kv_bytes = 256 * 2**20
        llm = LLM(args.model, random_weights=True, seed=args.seed, engine=engine, device=device)
        prompt_ids = list(range(10, 26))  # src/llmserve/cli.py:33
    else:
        llm = LLM(args.model, engine=engine, device=device)
        prompt_ids = None
    if args.prompt_ids is not None:
        prompt_ids = [int(t) for t in args.prompt_ids.split(",") if t.strip()]
    if prompt_ids is None:
        tok = llm.tokenizer()
        prompt_ids, eos = tok(args.prompt).input_ids, tok.eos_token_id

    params = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                            max_new_tokens=args.max_new_tokens, eos_token_id=eos, seed=args.seed)
    if args.mode == "kv_cache":
        result = llm.generate([prompt_ids], params)[0]
    else:
        result = llm.generate_naive(prompt_ids, params)

    print(tok.decode(result.tokens, skip_special_tokens=True) if tok else result.tokens)
    print(f"\n[{args.mode}] ttft={result.ttft_s * 1e3:.1f} ms | "
          f"decode={result.decode_tokens_per_s:.1f} tok/s | "
          f"peak mem={result.peak_memory_bytes / 2**20:.0f} MiB")
    return 0


if __name__ == "__main__":
    sys.exit(main())
