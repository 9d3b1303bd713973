"""Python entry point.  The reference offers functions (`generate(model, prompt_ids, params)`
-> `GenerationResult`, src/llmserve/engine/generate.py:16-58, and the scheduler's
`add_request` / `run_until_complete`, src/llmserve/scheduler/engine.py:127-178); `LLM` puts the
same names behind one object: a model folder (or a named size with random weights) in,
`generate(prompts, params)` out, the scheduler reachable as `LLM.engine` for streaming."""

from __future__ import annotations

from pathlib import Path
from time import perf_counter

import torch

from ..config.engine_config import EngineConfig
from ..config.registry import is_preset, preset
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .request import GenerationResult
from .runner import ModelRunner, StepEntry
from .scheduler import ContinuousBatchingEngine


class LLM:
    def __init__(self, model: str | Path | dict, *, dtype: str | None = None, random_weights: bool = False,
                 seed: int = 0, engine: EngineConfig | None = None, device=None):
        """`model`: a folder with config.json and safetensors, or, with `random_weights`, the
        name of a size (`llmserve.config.preset_names()`: whatever the registered architectures offer) or a config.json dictionary."""
        engine = engine or EngineConfig()
        if dtype is not None:
            engine.dtype = dtype
        engine.seed = seed if engine.seed == 0 else engine.seed
        self.engine_config = engine
        if random_weights:
            config = model if isinstance(model, dict) else preset(str(model))
            self.runner = ModelRunner.from_random(config, seed, engine, device)
        else:
            if isinstance(model, str) and not Path(model).exists() and is_preset(model):
                raise FileNotFoundError(f"{model!r} is a size, not a folder; pass random_weights=True to run it "
                                        "with random weights")
            if not Path(model).is_dir():
                raise FileNotFoundError(f"model folder {model} does not exist")
            self.runner = ModelRunner.from_folder(model, engine, device)
        self.config = self.runner.config
        self.sampler = Sampler(self.runner.device)
        self.engine = ContinuousBatchingEngine(
            self.runner, self.sampler,
            max_num_seqs=min(engine.max_num_seqs, self.runner.manager.max_seqs),
            max_num_batched_tokens=max(engine.max_num_batched_tokens, engine.max_num_seqs),
            max_prefill_chunk=engine.max_prefill_chunk, seed=engine.seed)
        self._tokenizer = None
        self._model_dir = None if random_weights else Path(model)

    # ---- text, if the folder has a tokenizer ----------------------------------------------
    def tokenizer(self):
        if self._tokenizer is None:
            if self._model_dir is None:
                raise ValueError("a model with random weights has no tokenizer; pass token ids")
            from transformers import AutoTokenizer  # tokenizer only; used as a black box

            self._tokenizer = AutoTokenizer.from_pretrained(str(self._model_dir))
        return self._tokenizer

    def warm_up(self, max_requests: int | None = None, max_context: int | None = None) -> int:
        """Capture the decode graphs ahead of time (`ModelRunner.warm_up`): a server calls this once after loading,
        so that the first request of every batch size does not wait for a capture."""
        return self.runner.warm_up(max_requests or self.engine.max_num_seqs, max_context)

    # ---- generation ------------------------------------------------------------------------------
    def generate(self, prompts, params: SamplingParams | list[SamplingParams] | None = None) -> list[GenerationResult]:
        """Generate for every prompt (lists of token ids, or strings when the folder has a
        tokenizer) with continuous batching; results in the order of the prompts."""
        if prompts and isinstance(prompts[0], int):
            prompts = [prompts]
        ids_list = [self.tokenizer()(p).input_ids if isinstance(p, str) else list(p) for p in prompts]
        if params is None:
            params = SamplingParams()
        params_list = params if isinstance(params, list) else [params] * len(ids_list)
        if len(params_list) != len(ids_list):
            raise ValueError("one SamplingParams per prompt, or one for all")
        torch.cuda.reset_peak_memory_stats(self.runner.device)
        start = perf_counter()
        rids = [self.engine.add_request(ids, p, arrival_time=start) for ids, p in zip(ids_list, params_list)]
        done = self.engine.run_until_complete()
        total = perf_counter() - start
        peak = int(torch.cuda.max_memory_allocated(self.runner.device))
        results = []
        for rid in rids:
            req = done.pop(rid)
            times = req.token_times
            results.append(GenerationResult(
                tokens=list(req.generated), ttft_s=(times[0] - start) if times else 0.0,
                step_latencies_s=[b - a for a, b in zip(times, times[1:])], total_s=total,
                peak_memory_bytes=peak, finish_reason=req.finish_reason))
        return results

    def generate_naive(self, prompt_ids: list[int], params: SamplingParams) -> GenerationResult:
        """The reference's baseline (src/llmserve/baseline/naive.py:21-56): no cache is kept
        between tokens, every new token re-runs the whole sequence."""
        if len(prompt_ids) + params.max_new_tokens > self.runner.max_model_len:
            raise ValueError(f"prompt + max_new_tokens = {len(prompt_ids) + params.max_new_tokens} exceeds "
                             f"max_position_embeddings = {self.runner.max_model_len}")
        from ..sampling.sampler import request_seed

        seed = request_seed(params, self.engine_config.seed, 0)
        ids, out, times = list(prompt_ids), [], []
        torch.cuda.reset_peak_memory_stats(self.runner.device)
        start = perf_counter()
        while len(out) < params.max_new_tokens:
            self.runner.add_sequence("naive")
            try:
                logits = self.runner.step([StepEntry("naive", ids, [len(ids) - 1])])
            finally:
                self.runner.free_sequence("naive")
            tok = self.sampler.sample(logits, [(params, seed, len(out))])[0]
            times.append(perf_counter())
            out.append(tok)
            ids.append(tok)
            if params.eos_token_id is not None and tok == params.eos_token_id:
                break
        return GenerationResult(
            tokens=out, ttft_s=times[0] - start, step_latencies_s=[b - a for a, b in zip(times, times[1:])],
            total_s=perf_counter() - start, peak_memory_bytes=int(torch.cuda.max_memory_allocated(self.runner.device)),
            finish_reason="stop" if params.eos_token_id is not None and out[-1] == params.eos_token_id else "length")
