"""Grouped-query causal attention over the paged cache
(src/llmserve/model/llama.py:57-109; mask and cache as src/llmserve/kvcache/paged.py:81-110).

Parameters: hidden, num_heads, num_kv_heads, head_dim, bias (q/k/v only; o_proj never has
one: src/llmserve/model/llama.py:67), window (None = all keys), position (a PartSpec).

q, k and v projections are stacked into one [(nh + 2 nkv) D, H] matrix at load.  One step:
project, rotate q and k and store k, v at the new tokens' cache slots, attend over the
request's pages (the new tokens included), project back.
"""

from __future__ import annotations

import math

import torch

from ..ops import library as ops
from .linear import adds_residual_in_epilogue, decode_product, few_rows, linear, linear_partial_sums
from .registry import ADDED_IN_PLACE, POSITION_ENCODINGS, DeferredNorm, Mixer, register_mixer
from .spec import PagedCacheSpec, ParamInfo


@register_mixer("attention")
class Attention(Mixer):
    graph_safe = True
    accepts_deferred_norm = True

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.hidden = int(spec["hidden"])
        self.num_heads = int(spec["num_heads"])
        self.num_kv_heads = int(spec["num_kv_heads"])
        self.head_dim = int(spec["head_dim"])
        self.bias = bool(spec.get("bias", False))
        self.window = spec.get("window")
        if self.num_heads % self.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if not 0 < self.head_dim <= 256:
            raise ValueError(f"head_dim={self.head_dim} is outside what the attention kernels take (1..256)")
        if self.window is not None and self.window < 1:
            raise ValueError("window must be >= 1")
        self.scale = 1.0 / math.sqrt(self.head_dim)  # SDPA's default scale
        self.position = POSITION_ENCODINGS.build(spec["position"], ctx)
        self.qkv_weight = self.qkv_bias = self.o_weight = None

    def cache_spec(self):
        return PagedCacheSpec(self.num_kv_heads, self.head_dim, self.window)

    def param_infos(self):
        h, d = self.hidden, self.head_dim
        infos = {"q_proj.weight": ParamInfo((self.num_heads * d, h)),
                 "k_proj.weight": ParamInfo((self.num_kv_heads * d, h)),
                 "v_proj.weight": ParamInfo((self.num_kv_heads * d, h)),
                 "o_proj.weight": ParamInfo((h, self.num_heads * d))}
        if self.bias:
            infos.update({"q_proj.bias": ParamInfo((self.num_heads * d,), "zeros"),
                          "k_proj.bias": ParamInfo((self.num_kv_heads * d,), "zeros"),
                          "v_proj.bias": ParamInfo((self.num_kv_heads * d,), "zeros")})
        return infos

    def load(self, tensors):
        self.qkv_weight = torch.cat([tensors[f"{n}_proj.weight"] for n in "qkv"], dim=0).contiguous()
        if self.bias:
            self.qkv_bias = torch.cat([tensors[f"{n}_proj.bias"] for n in "qkv"], dim=0).contiguous()
        self.o_weight = tensors["o_proj.weight"].contiguous()
        self.position.load({})

    def forward(self, x, batch, cache):
        nh, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
        view = batch.groups[cache.group_id]
        slots = view.slots if cache.store else None
        deferred = x if isinstance(x, DeferredNorm) else None  # (then the result goes to a norm, which takes partial sums)
        q = self.project_few_rows(x, batch, cache, slots)
        if q is None:
            if deferred is not None:
                x = deferred.materialize()
            q = linear(x, self.qkv_weight, self.qkv_bias)  # q, k and v side by side; q is read in place
            fused = getattr(self.position, "rotate_and_store", None)
            if fused is not None:
                fused(q, batch.positions, slots, cache.k_pool, cache.v_pool, nh, nkv, d, cache.block_size)
            else:
                self.position.rotate(q, batch.positions, nh, nkv, d)
                if slots is not None:
                    ops.rope_store(q, None, batch.positions, slots, cache.k_pool, cache.v_pool, nh, nkv, d,
                                   cache.block_size)
        out = torch.empty((q.shape[0], nh * d), dtype=q.dtype, device=q.device)
        self.attend(out, q, cache, view, batch)
        if deferred is not None and deferred.may_add_in_place and adds_residual_in_epilogue(out, self.o_weight):
            ops.gemm_decode(None, out, self.o_weight, residual=deferred.residual)  # the residual sum in the epilogue
            return ADDED_IN_PLACE
        return (linear_partial_sums(out, self.o_weight) if deferred is not None else None) or linear(out, self.o_weight)

    def _few_rows_unfit(self, rows) -> bool:
        if rows.dtype != torch.bfloat16 or self.head_dim % 16 != 0 or not ops.gemm_bf16_supported(rows, self.qkv_weight):
            return True
        return not (decode_product(rows, self.qkv_weight) or few_rows(rows.shape[0], self.qkv_weight))

    def project_few_rows(self, x, batch, cache, slots):
        """With few bfloat16 rows one kernel does the projection, the rotation and the cache store
        (ops.gemm_decode, which also norms its rows on the way in, or ops.gemm_stream).  Returns the rotated
        queries, or None when neither kernel applies."""
        deferred = isinstance(x, DeferredNorm)
        rows = x.residual if deferred else x
        m = rows.shape[0]
        if self._few_rows_unfit(rows):
            return None
        frequencies = getattr(self.position, "rotary_frequencies", None)
        if frequencies is None and not getattr(self.position, "identity", False):
            return None  # a position encoding this kernel does not know
        decode = decode_product(rows, self.qkv_weight)
        norm = x.fused() if deferred and decode and m <= ops.GEMM_DECODE_NORM_ROWS else None
        if norm is not None:
            x.resolve(None)  # nothing is left to add: the kernel norms the residual rows as they are
        elif deferred:
            rows = x.materialize()  # the residual sum and the norm by the norm's own kernel, the rest fused
        rope = dict(n_heads=self.num_heads, n_kv_heads=self.num_kv_heads, head_dim=self.head_dim,
                    inv_freq=frequencies() if frequencies is not None else None, positions=batch.positions,
                    slots=slots, k_pool=cache.k_pool, v_pool=cache.v_pool, block_size=cache.block_size)
        q = torch.empty((m, self.num_heads * self.head_dim), dtype=rows.dtype, device=rows.device)
        if decode:
            angles = getattr(self.position, "rotary_angles", None)
            if angles is not None and getattr(batch, "shared", None) is not None:
                rope["angles"] = angles(batch)  # worked out once per step, not once per layer and workgroup
            ops.gemm_decode(q, rows, self.qkv_weight, self.qkv_bias, rope=rope, norm=norm)
        else:
            ops.gemm_stream(q, rows, self.qkv_weight, self.qkv_bias, rope=rope)
        return q

    def attend(self, out, qkv, cache, view, batch):
        """out[n] = attention of token n's query heads (the first nh*D columns of qkv) over its
        request's pages.  Picks the kernel by dtype and by what the step holds."""
        nh, nkv, d, bs, window = self.num_heads, self.num_kv_heads, self.head_dim, cache.block_size, self.window or 0
        if not ops.attention_mfma_supported(qkv.dtype, d, bs):
            ops.attention_wave(out, qkv, cache.k_pool, cache.v_pool, view.block_tables, batch.token_seq,
                               batch.positions, nh, nkv, d, bs, window, self.scale, table_rows=batch.state_slots)
            return
        common = (out, qkv, cache.k_pool, cache.v_pool, view.block_tables, batch.cu_seqlens, batch.context_lens)
        n_dec = batch.num_decode
        if n_dec:  # requests that bring one token: their keys are spread over waves and workgroups
            splits, waves = self.decode_arrangement(n_dec, batch.max_decode_context, ops.compute_units(qkv.device))
            ops.attention_mfma(*common, 0, n_dec, 1, 0, n_dec, nh, nkv, d, bs, window, self.scale,
                               split_waves=True, num_splits=splits, waves=waves, table_rows=batch.state_slots)
        if n_dec < batch.num_seqs:  # portions of prompts: one wave per group of tokens and heads
            splits = self.prompt_splits(batch.num_seqs - n_dec, batch.max_count, batch.max_context, ops.compute_units(qkv.device))
            ops.attention_mfma(*common, n_dec, batch.num_seqs - n_dec, batch.max_count, n_dec,
                               batch.num_tokens - n_dec, nh, nkv, d, bs, window, self.scale, num_splits=splits,
                               table_rows=batch.state_slots)

    def prompt_splits(self, n_requests: int, max_new: int, max_context: int, cus: int = 256) -> int:
        """Workgroups that share the keys of one block of prompt tokens (a second kernel merges their shares).
        Blocks enough for a workgroup of 8 waves on every CU need no sharing: there each wave has a twin that
        takes every other tile of keys for the same tokens, and with two such workgroups per CU the long blocks
        and the short ones even out.  With exactly one per CU sharing pays only behind a long prefix (measured:
        from about 3,000 keys on).  A short portion behind a long prefix has few blocks and many keys: its keys
        are shared out, 8 tiles of keys a workgroup at least (16 where the blocks alone are half a chip), up to
        about two workgroups of 4 waves per CU, and not in more than 4 once the blocks alone are a quarter of a
        chip (measured on portions of 16 to 256 tokens behind 256 to 4,032 keys, at head sizes 64 and 128: the
        merge kernel's work grows with blocks times shares).  `cus`: the device's compute units."""
        if self.window:
            return 1
        g = self.num_heads // self.num_kv_heads
        hg = min(g, 16)
        blocks = -(-max_new // (4 * (16 // hg)))  # of 4 waves with one column group each
        workgroups = blocks * self.num_kv_heads * -(-g // hg) * n_requests
        tiles = -(-max_context // 32)
        if workgroups >= 2 * cus:
            return 1
        if workgroups >= cus:
            return 4 if tiles >= 96 else 1
        per_share = 16 if workgroups >= cus // 2 else 8
        most = 4 if workgroups >= cus // 4 else 8
        return max(1, min(2 * cus // max(workgroups, 1), tiles // per_share, most))

    def decode_arrangement(self, n_requests: int, max_context: int, cus: int = 256) -> tuple[int, int]:
        """(workgroups per request and KV head, waves per workgroup) for decoding.  The waves of a
        workgroup take 32 keys at a time each and merge in LDS; workgroups that share a request hand
        their shares to the one that finishes last, through memory, which costs more (2 to 3
        microseconds) than a few extra tiles per wave.  So a small batch first gets 8 waves, and is
        split over workgroups only when a wave would still walk more than 4 tiles (measured: at a
        context of 512 no split pays at any batch size, at 4,096 four to eight do up to batch 8); once
        the batch alone fills the chip (a workgroup for each of its `cus` compute units) nothing is split."""
        g = self.num_heads // self.num_kv_heads
        groups = n_requests * self.num_kv_heads * -(-g // 16)
        reach = min(max_context, self.window) if self.window else max_context
        waves = 8 if self.head_dim <= 160 else 4  # (8 waves of wider heads would not fit the registers)
        if groups >= cus:
            return 1, waves
        tiles = -(-reach // 32)
        splits = max(1, min(cus // groups, -(-tiles // (4 * waves))))
        return splits, waves
