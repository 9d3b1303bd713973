"""A stand-in for the GPU step function, for scheduler tests without a GPU: the real
cache manager, and logits from the plain implementation run over each request's whole
history."""

import torch

import plain_llama
from llmserve.cache import CacheManager, group_layers
from llmserve.parts.spec import PagedCacheSpec
from llmserve.sampling import uniform


class PlainRunner:
    def __init__(self, cfg: dict, weights: dict, num_blocks: int, block_size: int, max_seqs: int = 8):
        self.cfg, self.weights = cfg, weights
        heads = cfg["num_attention_heads"]
        spec = PagedCacheSpec(cfg.get("num_key_value_heads", heads), cfg["hidden_size"] // heads)
        self.manager = CacheManager(group_layers([spec] * cfg["num_hidden_layers"]), num_blocks, block_size, max_seqs)
        self.vocab_size = cfg["vocab_size"]
        self.max_model_len = cfg.get("max_position_embeddings", 2048)
        self.history: dict = {}
        self.step_sizes: list[list[int]] = []

    def step(self, entries):
        self.manager.append([e.seq_id for e in entries], [len(e.tokens) for e in entries])  # may raise OutOfBlocks
        self.step_sizes.append([len(e.tokens) for e in entries])
        rows = []
        for e in entries:
            start = self.manager.lengths[e.seq_id] - len(e.tokens)
            hist = self.history.get(e.seq_id, [])[:start] + list(e.tokens)  # a re-admitted request starts over
            self.history[e.seq_id] = hist
            if e.want:
                logits = plain_llama.forward(self.cfg, self.weights, hist, torch.float32)
                rows += [logits[start + w] for w in e.want]
        return torch.stack(rows) if rows else torch.empty(0, self.vocab_size)


class PlainSampler:
    def sample(self, logits, items):
        return [plain_llama.sample(logits[i], p.temperature, p.top_k, p.top_p, uniform(seed, index))
                for i, (p, seed, index) in enumerate(items)]


class LaggedRunner(PlainRunner):
    """The same, taking a step's tokens from the sampler's pending ids (here a list stands in for
    the tensor on the device), as the GPU runner does when decode steps are replayed graphs."""

    takes_device_tokens = True

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.continuations = 0

    def step(self, entries, device_tokens=None):
        if device_tokens is not None:
            assert len(device_tokens) == len(entries) and all(e.tokens == [0] for e in entries)
            entries = [type(e)(e.seq_id, [int(t)], e.want) for e, t in zip(entries, device_tokens)]
            self.continuations += 1
        return super().step(entries)


class FakePending:
    def __init__(self, tokens):
        self.device = list(tokens)
        self.reads = 0

    def result(self):
        self.reads += 1
        assert self.reads == 1, "a step's tokens are read once"
        return list(self.device)


class LaggedSampler(PlainSampler):
    def sample_async(self, logits, items):
        return FakePending(self.sample(logits, items))
