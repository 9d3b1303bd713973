"""The step function: runs a batch of (request, its next tokens) through the model, from
the cache that earlier steps left, and returns the logits at the wanted places.

The reference has no single step function: its scheduler runs one padded forward for new
prompts and one for decoding requests (src/llmserve/scheduler/engine.py:186-193,236-246).
Here one call runs everything a step holds as one flat batch: portions of prompts beside
single decoded tokens, cut anywhere.  Steps of single tokens are replayed from HIP graphs (one per
batch size and context range); other steps run at the sizes of a bucket and are replayed from a graph
from the bucket's second use on.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from pathlib import Path

import torch

from ..cache.manager import CacheManager, group_layers
from ..cache.storage import CacheStorage, pool_sizes_for_budget
from ..config.engine_config import EngineConfig
from ..config.registry import architecture_of, read_config
from ..ops import library as ops
from ..parts.model import Model
from ..parts.registry import BuildContext
from ..weights.loader import load_tensors
from ..weights.random import random_tensors
from .batch import BatchUploader, StaticDecodeBatch, StaticStepBatch, build_batch

_TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


@dataclass
class StepEntry:
    """One request's share of a step: its next tokens, and the places among them (0-based
    within `tokens`) whose logits are wanted."""

    seq_id: object
    tokens: list[int]
    want: list[int] = field(default_factory=list)


class ModelRunner:
    def __init__(self, model: Model, config, engine_config: EngineConfig, device: torch.device):
        self.model = model
        self.config = config
        self.engine_config = engine_config
        self.device = device
        self.dtype = model.ctx.dtype
        self.vocab_size = model.spec.vocab_size
        if engine_config.max_model_len is not None and engine_config.max_model_len > model.spec.max_positions:
            # (the reference refuses it too: src/llmserve/utils.py:8-13)
            raise ValueError(f"max_model_len={engine_config.max_model_len} is more than the model's "
                             f"{model.spec.max_positions} positions")
        self.max_model_len = engine_config.max_model_len or model.spec.max_positions
        self.block_size = engine_config.block_size
        groups = group_layers(model.cache_specs())
        elem = torch.empty(0, dtype=self.dtype).element_size()
        if engine_config.num_blocks is not None:
            num_blocks = engine_config.num_blocks
        else:
            budget = engine_config.kv_bytes
            if budget is None:
                free, _total = torch.cuda.mem_get_info(device)
                budget = int(free * engine_config.gpu_memory_fraction)
            # the state of all slots comes off the budget; every paged group gets pages for the same number of longest
            # requests, and no more than all slots could ever fill
            step_tokens = min(engine_config.max_num_batched_tokens, engine_config.max_prefill_chunk or self.max_model_len)
            num_blocks = pool_sizes_for_budget(groups, self.block_size, elem, budget, engine_config.max_num_seqs,
                                               self.max_model_len, step_tokens)
        self.manager = CacheManager(groups, num_blocks, self.block_size, engine_config.max_num_seqs)
        self.storage = CacheStorage(groups, num_blocks, self.block_size, engine_config.max_num_seqs,
                                    self.dtype, device, table_width=-(-self.max_model_len // self.block_size))
        ops.reset_arrival_counters(device)  # (whatever an earlier runner's failed step may have left)
        self._uploader = BatchUploader(device)
        self._graphs: dict[tuple[int, int], "_DecodeGraph"] = {}
        self._use_graphs = engine_config.use_graphs and model.graph_safe()
        # steps that bring portions of prompts run at the sizes of a bucket: fixed buffers per bucket (most
        # recently used last), and a graph from the bucket's second use on
        self._buckets: dict[tuple, "_StepBucket"] = {}
        self._step_graph_pool = None
        # rows the steps were asked to run, and rows they ran with the padding of buckets and graphs
        self.rows_asked = 0
        self.rows_run = 0
        # matrix elements a token meets on its way through the layers: what a step's device time goes by
        infos = model.param_infos()
        outer = tuple(model.spec.weights[role] for role in ("embedding", "head"))
        self._elements_per_token = sum(info.shape[0] * info.shape[1] for name, info in infos.items()
                                       if len(info.shape) == 2 and not name.startswith(outer))

    # ---- construction ---------------------------------------------------------------------
    @staticmethod
    def _device(device=None) -> torch.device:
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible; this engine runs on gfx950 only and has no CPU path")
        return torch.device(device or "cuda:0")

    @classmethod
    def from_folder(cls, model_dir: str | Path, engine_config: EngineConfig | None = None, device=None):
        """Model chosen by the folder's config.json, weights from its safetensors files."""
        engine_config = engine_config or EngineConfig()
        engine_config.validate()
        device = cls._device(device)
        ops.ensure_built(engine_config.dtype)
        arch, config, _raw = read_config(model_dir)
        dtype = _TORCH_DTYPES[engine_config.dtype]
        model = Model(arch.build_spec(config), BuildContext(dtype, device))
        infos = model.param_infos()
        ignore = {model.spec.weights["head"] + "weight"} if getattr(model.head, "tied", False) else set()
        model.load(load_tensors(model_dir, infos, dtype, device, ignore))
        return cls(model, config, engine_config, device)

    @classmethod
    def from_random(cls, config_dict: dict, seed: int = 0, engine_config: EngineConfig | None = None,
                    device=None, on_device: bool = True):
        """Seeded random weights made in memory (no folder).  `on_device` draws them on the GPU,
        which is fast for large models; a folder written by `write_random_model` uses the CPU
        streams instead, so the two do not hold the same numbers."""
        engine_config = engine_config or EngineConfig()
        engine_config.validate()
        device = cls._device(device)
        ops.ensure_built(engine_config.dtype)
        arch = architecture_of(config_dict)
        config = arch.config_class.from_dict(config_dict)
        dtype = _TORCH_DTYPES[engine_config.dtype]
        model = Model(arch.build_spec(config), BuildContext(dtype, device))
        tensors = random_tensors(model.param_infos(), seed, dtype, device if on_device else "cpu")
        model.load({k: v.to(device) for k, v in tensors.items()})
        return cls(model, config, engine_config, device)

    # ---- requests -------------------------------------------------------------------------
    def add_sequence(self, seq_id) -> None:
        self.manager.add_sequence(seq_id)

    def free_sequence(self, seq_id) -> None:
        self.manager.free_sequence(seq_id)

    # ---- the step ---------------------------------------------------------------------------
    lends_logits = True  # `step(..., borrow=True)` is understood

    @property
    def takes_device_tokens(self) -> bool:
        """Whether `step(..., device_tokens=...)` is available (decode-only steps are replayed graphs)."""
        return self._use_graphs

    @torch.inference_mode()
    def step(self, entries: list[StepEntry], device_tokens: torch.Tensor | None = None, *,
             borrow: bool = False) -> torch.Tensor:
        """Run the entries' tokens as one batch; float32 logits [sum(len(want)), vocab] in the
        order of the entries and of their `want`.  Raises `OutOfBlocks` (nothing changed) when
        the pages do not suffice.

        `device_tokens` (int32, one per entry, on the device): every entry brings one token, and
        its value is taken from this tensor instead of the entry (whose token is a placeholder):
        the ids the sampler chose for the previous step, which the host need not have seen yet.

        The logits belong to the caller.  With `borrow` they may instead be a view of memory that a
        replayed graph owns: valid until the next call of `step`, which may overwrite them (work
        queued on the same stream before that call still reads the right values)."""
        if not entries:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        if device_tokens is not None:
            if not self.takes_device_tokens:
                raise ValueError("this runner does not replay decode steps, so it takes tokens from the host only")
            if (device_tokens.dtype != torch.int32 or device_tokens.device != self.device or
                    tuple(device_tokens.shape) != (len(entries),) or any(len(e.tokens) != 1 for e in entries)):
                raise ValueError("device_tokens must be an int32 tensor on the runner's device, one id per entry, "
                                 "and every entry must bring exactly one token")
        for e in entries:
            if not e.tokens:
                raise ValueError(f"request {e.seq_id!r} brings no tokens")
            bad = [t for t in e.tokens if not 0 <= t < self.vocab_size]
            if bad:
                raise ValueError(f"request {e.seq_id!r}: token ids {bad[:5]} are outside the vocabulary "
                                 f"[0, {self.vocab_size})")
            if any(not 0 <= w < len(e.tokens) for w in e.want):
                raise ValueError(f"request {e.seq_id!r}: wanted places {e.want} are outside its {len(e.tokens)} tokens")
            length = self.manager.lengths.get(e.seq_id)
            if length is None:
                raise KeyError(f"unknown sequence {e.seq_id!r}")
            if length + len(e.tokens) > self.max_model_len:
                raise ValueError(f"request {e.seq_id!r} would reach {length + len(e.tokens)} tokens; "
                                 f"the limit is {self.max_model_len}")
        # requests that bring a single token go first (kernels for decoding take the leading rows)
        order = sorted(range(len(entries)), key=lambda i: len(entries[i].tokens) != 1)
        ordered = [entries[i] for i in order]
        layout = self.manager.append([e.seq_id for e in ordered], [len(e.tokens) for e in ordered])
        first_row = {}
        row = 0
        for e in ordered:
            first_row[id(e)] = row
            row += len(e.tokens)
        logit_rows = [first_row[id(e)] + w for e in entries for w in e.want]
        self.storage.clear_state(layout.fresh_slots)
        try:
            logits, owned = self._run(layout, ordered, logit_rows, device_tokens)
        except BaseException:
            # a launch that failed half-way may have left workgroups counted where the next step counts again
            ops.reset_arrival_counters(self.device)
            raise
        self.manager.release_passed(layout.seq_ids)
        return logits if owned or borrow else logits.clone()

    def _run(self, layout, ordered: list[StepEntry], logit_rows: list[int], device_tokens) -> tuple[torch.Tensor, bool]:
        """The step's logits and whether the caller owns them (not a view of a graph's memory)."""
        if not self._use_graphs:  # launched kernel by kernel, on exactly the step's tokens
            batch = build_batch(layout, [e.tokens for e in ordered], logit_rows, self._uploader, self.storage)
            return self.model.forward(batch, self.storage), True
        if all(len(e.tokens) == 1 for e in ordered):
            return self._replay_decode(layout, [e.tokens[0] for e in ordered], logit_rows, device_tokens), False
        if self._launch_bound(sum(layout.counts)):
            return self._run_bucketed_step(layout, [e.tokens for e in ordered], logit_rows)
        # the device is busy for longer than the host needs to launch the step: nothing to gain from a graph
        batch = build_batch(layout, [e.tokens for e in ordered], logit_rows, self._uploader, self.storage)
        logits = self.model.forward(batch, self.storage)
        self.rows_run += sum(layout.counts)
        self.rows_asked += sum(layout.counts)
        return logits, True

    # ---- decode-only steps as HIP graphs --------------------------------------------------------
    @staticmethod
    def _decode_bucket(n_requests: int, context: int) -> tuple[int, int]:
        """(capacity, reach) of the graph that a decode step of `n_requests` whose longest context is `context`
        replays: powers of two, the reach from 256."""
        capacity = 1
        while capacity < n_requests:
            capacity *= 2
        reach = 256
        while reach < context:
            reach *= 2
        return capacity, reach

    @torch.inference_mode()
    def warm_up(self, max_requests: int | None = None, max_context: int | None = None) -> int:
        """Capture, ahead of time, the graphs that decode steps of up to `max_requests` requests with contexts up
        to `max_context` replay (defaults: all the runner's slots, its longest request), so that no request waits
        for a capture in the middle of serving.  Returns the number of graphs captured now; 0 for a runner that
        launches its steps kernel by kernel."""
        if not self._use_graphs:
            return 0
        top_capacity, top_reach = self._decode_bucket(max_requests or self.manager.max_seqs,
                                                      max_context or self.max_model_len)
        made, capacity = 0, 1
        while capacity <= top_capacity:
            reach = 256
            while reach <= top_reach:
                if (capacity, reach) not in self._graphs:
                    self._graphs[(capacity, reach)] = _DecodeGraph(self, capacity, reach)
                    made += 1
                reach *= 2
            capacity *= 2
        return made

    def _replay_decode(self, layout, tokens: list[int], logit_rows: list[int],
                       device_tokens: torch.Tensor | None = None) -> torch.Tensor:
        """A step of single tokens: replay the graph captured for this batch size and context range
        (capture it at first use).  The logits it returns live in the graph's own memory and are
        overwritten by the next replay of the same graph."""
        n = len(tokens)
        capacity, reach = key = self._decode_bucket(n, max(layout.starts) + 1)
        graph = self._graphs.get(key)
        if graph is None:
            graph = _DecodeGraph(self, capacity, reach)
            self._graphs[key] = graph
        graph.static.fill(layout, tokens)
        if device_tokens is not None:  # (all entries bring one token, so their order is the caller's)
            graph.static.batch.token_ids[:n].copy_(device_tokens)
        graph.graph.replay()
        self.rows_run += capacity
        self.rows_asked += n
        if logit_rows == list(range(n)):
            return graph.logits[:n]
        return graph.logits[torch.tensor(logit_rows, dtype=torch.long, device=self.device)]

    # ---- steps with portions of prompts: padded to a bucket of sizes, replayed from the second time on ------
    MAX_STEP_GRAPHS = 32
    CAPTURE_AT_USE = 2  # a bucket is captured as a graph when it comes for this many-th time
    # A step is worth a graph while launching its kernels one by one (about 20 microseconds each, some two hundred
    # for a model of 22 layers) takes the host longer than the device needs to run them.  Per layer the host's time
    # is fixed and the device's goes by rows times matrix elements; up to this product (a step of 1,100 rows of the
    # 1.1B shape, of 250 rows of the 7B shape) the host is the limit.  A rule by sizes alone: the same step always
    # takes the same path.
    LAUNCH_BOUND_WORK_PER_LAYER = 5.0e10

    def _launch_bound(self, rows: int) -> bool:
        return rows * self._elements_per_token <= self.LAUNCH_BOUND_WORK_PER_LAYER * len(self.model.spec.schedule)

    @staticmethod
    def _row_bucket(n: int) -> int:
        """Rows of portions are padded to a multiple of 16, or of an eighth of the power of two below them if
        that is more: never more than 15 rows or 12.5 % beyond what was asked."""
        if n <= 0:
            return 0
        floor = 1 << (n.bit_length() - 1)
        unit = max(16, floor // 8)
        return -(-n // unit) * unit

    @classmethod
    def _step_shape(cls, n_decode: int, n_prefill: int, n_prefill_tokens: int, n_logits: int, context: int) -> tuple:
        """The sizes a step is padded to: powers of two for the requests, the wanted rows and the reach of
        the contexts (which only sets how attention spreads its work), `_row_bucket` for the rows of the portions."""
        def pow2(x, least=1):
            p = least
            while p < x:
                p *= 2
            return p
        return (pow2(n_decode) if n_decode else 0, pow2(n_prefill), cls._row_bucket(n_prefill_tokens),
                pow2(max(n_logits, 1)), pow2(context, 256))

    def _shape_of(self, layout, n_logits: int) -> tuple:
        n_dec = 0
        while n_dec < len(layout.counts) and layout.counts[n_dec] == 1:
            n_dec += 1
        context = max(s + c for s, c in zip(layout.starts, layout.counts))
        return self._step_shape(n_dec, len(layout.counts) - n_dec, sum(layout.counts[n_dec:]), n_logits, context)

    def _run_bucketed_step(self, layout, tokens: list[list[int]], logit_rows: list[int]) -> tuple[torch.Tensor, bool]:
        """A step with portions of prompts.  It always runs at the sizes of its bucket (`_step_shape`), from
        fixed buffers in which what the step does not use belongs to dummy requests without keys: launched
        kernel by kernel the first time the bucket comes, captured as a HIP graph the second time and replayed
        from then on.  Which kernels run, and in which arrangement, is therefore a function of the bucket
        alone: the first run and every replay give the same bits, and so do two runs of one trace.
        Returns (logits, whether the caller owns them)."""
        shape = self._shape_of(layout, len(logit_rows))
        bucket = self._buckets.pop(shape, None)
        if bucket is None:
            if len(self._buckets) >= self.MAX_STEP_GRAPHS:
                self._buckets.pop(next(iter(self._buckets)))  # the least recently used
            bucket = _StepBucket(self, shape)
        self._buckets[shape] = bucket  # (most recently used last)
        bucket.static.fill(layout, tokens, logit_rows)
        bucket.uses += 1
        self.rows_run += bucket.static.num_rows
        self.rows_asked += sum(layout.counts)
        n = len(logit_rows)
        if bucket.graph is None and bucket.uses >= self.CAPTURE_AT_USE:
            if self._step_graph_pool is None:
                self._step_graph_pool = torch.cuda.graph_pool_handle()
            bucket.capture(self, self._step_graph_pool)
        if bucket.graph is not None:
            bucket.graph.replay()
            return bucket.logits[:n], False
        return bucket.run(self)[:n], True

    @property
    def _step_graphs(self) -> dict:
        """The buckets that have been captured as graphs."""
        return {shape: b for shape, b in self._buckets.items() if b.graph is not None}


class _capturing:
    """`with _capturing(graph, pool):` records the launches inside it into `graph`.  Python's cycle collector
    stays off meanwhile, after one collection up front: an object it finds dead in the middle of a capture may
    own device memory or another graph, and giving those back is not allowed while a stream is capturing."""

    def __init__(self, graph: "torch.cuda.CUDAGraph", pool=None):
        self._context = torch.cuda.graph(graph, pool=pool) if pool is not None else torch.cuda.graph(graph)

    def __enter__(self):
        import gc

        gc.collect()
        self._gc_was_on = gc.isenabled()
        gc.disable()
        try:
            return self._context.__enter__()
        except BaseException:
            if self._gc_was_on:
                gc.enable()
            raise

    def __exit__(self, *exc):
        import gc

        try:
            return self._context.__exit__(*exc)
        finally:
            if self._gc_was_on:
                gc.enable()


class _StepBucket:
    """Fixed buffers, and from the second use on a captured graph, for steps of up to `decode` single tokens,
    `prefill` portions of `tokens` rows in all and `logits` wanted rows, contexts up to `reach`.  All such
    graphs share one memory pool: they never run at the same time, and a step's logits are consumed (or
    copied) before the next step is replayed."""

    def __init__(self, runner: "ModelRunner", shape: tuple):
        decode, prefill, tokens, logits, reach = shape
        group_ids = [g.group_id for g in runner.manager.paged_groups]
        self.static = StaticStepBatch(decode, prefill, tokens, logits, runner.storage, group_ids, runner.device)
        batch = self.static.batch
        batch.max_context = batch.max_decode_context = reach
        self.uses = 0
        self.graph = None
        self.logits = None

    def run(self, runner: "ModelRunner") -> torch.Tensor:
        """Launch the step that `static.fill` described, kernel by kernel.  (The runner is an argument, not a
        field: a bucket that pointed back at its runner would keep both alive until the cycle collector runs.)"""
        self.static.apply_table_updates()
        return runner.model.forward(self.static.batch, runner.storage)

    def capture(self, runner: "ModelRunner", pool) -> None:
        """Record the same launches as a graph (nothing runs; an earlier `run` of this bucket has loaded every
        library and warmed the memory pools)."""
        torch.cuda.synchronize(runner.device)
        self.graph = torch.cuda.CUDAGraph()
        with _capturing(self.graph, pool):
            self.logits = self.run(runner)


class _DecodeGraph:
    """One captured decode step for up to `capacity` requests whose contexts reach up to `reach` keys
    (the reach only sets how the attention kernel spreads its work; longer contexts stay correct)."""

    def __init__(self, runner: ModelRunner, capacity: int, reach: int):
        group_ids = [g.group_id for g in runner.manager.paged_groups]
        self.static = StaticDecodeBatch(capacity, runner.storage, group_ids, runner.device)
        batch = self.static.batch
        batch.max_context = batch.max_decode_context = reach
        # a first run outside the capture: libraries load, memory pools warm up
        self.static.apply_table_updates()
        runner.model.forward(batch, runner.storage)
        torch.cuda.synchronize(runner.device)
        self.graph = torch.cuda.CUDAGraph()
        with _capturing(self.graph):
            self.static.apply_table_updates()
            self.logits = runner.model.forward(batch, runner.storage)
