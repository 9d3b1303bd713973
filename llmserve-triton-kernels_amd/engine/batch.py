"""One step's batch as the kernels see it: a flat run of new tokens, no padding.

The reference describes a step by `PagedBatch` (src/llmserve/kvcache/paged.py:65-79):
positions and a validity mask over a right-padded [B, T] grid, write blocks and offsets,
block tables, context lengths, last indices.  Here the new tokens of all requests lie end
to end (request b owns rows cu_seqlens[b] .. cu_seqlens[b+1]), any mixture of portions of
prompts and single decoded tokens; requests that bring one token come first.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ..cache.manager import StepLayout


@dataclass
class GroupView:
    """One cache group's part of a step."""

    block_tables: torch.Tensor  # int32 [state slots, M], resident on the device; request b owns row state_slots[b]
    slots: torch.Tensor  # int32 [N]: page * block_size + offset of every new token


@dataclass
class StepBatch:
    num_tokens: int
    num_seqs: int
    token_ids: torch.Tensor  # int32 [N]
    positions: torch.Tensor  # int32 [N] absolute position of each new token
    token_seq: torch.Tensor  # int32 [N] index (0..B-1) of the request a token belongs to
    cu_seqlens: torch.Tensor  # int32 [B+1]
    context_lens: torch.Tensor  # int32 [B] keys present after this step's store
    state_slots: torch.Tensor  # int32 [B] state slot of each request
    logit_rows: torch.Tensor  # int32 [R] rows whose logits are wanted
    groups: dict[int, GroupView]
    # host copies, for choosing kernels without a read-back
    counts: list[int] = field(default_factory=list)
    starts: list[int] = field(default_factory=list)
    state_slot_list: list[int] = field(default_factory=list)  # host copy of state_slots
    num_decode: int = 0  # leading requests that bring exactly one token
    max_count: int = 0
    max_context: int = 0
    max_decode_context: int = 0  # longest context among the leading single-token requests
    # what a part has worked out for this step and the same kind of part in later layers can use again (the sines
    # and cosines of the tokens' angles); emptied by the model when a step starts
    shared: dict = field(default_factory=dict)
    all_rows_wanted: bool = False  # logit_rows is 0, 1, ..., num_tokens - 1 (known on the host: nothing to pick)


class BatchUploader:
    """Packs a step's integer arrays into one pinned buffer and sends them with one copy.

    A small ring of pinned buffers, each guarded by an event, lets a caller issue steps
    back to back without waiting for the device."""

    def __init__(self, device: torch.device, ring: int = 4):
        self.device = device
        self._ring = [None] * ring
        self._events = [None] * ring
        self._next = 0

    def upload(self, flat: list[int]) -> torch.Tensor:
        n = len(flat)
        i = self._next
        self._next = (i + 1) % len(self._ring)
        if self._events[i] is not None:
            self._events[i].synchronize()
        buf = self._ring[i]
        if buf is None or buf.numel() < n:
            buf = torch.empty(max(n, 4096), dtype=torch.int32, pin_memory=True)
            self._ring[i] = buf
        buf[:n] = torch.tensor(flat, dtype=torch.int32)
        dev = torch.empty(n, dtype=torch.int32, device=self.device)
        dev.copy_(buf[:n], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record(torch.cuda.current_stream(self.device))
        self._events[i] = ev
        return dev


def _update_arrays(updates: list[tuple[int, int, int]], width: int, rows: int) -> tuple[list[int], list[int]]:
    index, value = [], []
    for row, i, page in updates:
        if not (0 <= row < rows and 0 <= i < width):
            raise ValueError(f"block table entry ({row}, {i}) is outside the device table [{rows}, {width}]")
        index.append(row * width + i)
        value.append(page)
    return index, value


def build_batch(layout: StepLayout, tokens: list[list[int]], logit_rows: list[int], uploader: BatchUploader,
                storage) -> StepBatch:
    """Device tensors for a step whose pages `layout` has already fixed; the pages it took are written
    into the device-resident block tables of `storage`."""
    from ..ops import library as ops

    counts, starts = layout.counts, layout.starts
    n_seqs = len(counts)
    flat_tokens = [t for row in tokens for t in row]
    n_tokens = len(flat_tokens)
    positions, token_seq, cu = [], [], [0]
    for b, (start, n) in enumerate(zip(starts, counts)):
        positions.extend(range(start, start + n))
        token_seq.extend([b] * n)
        cu.append(cu[-1] + n)
    context = [s + n for s, n in zip(starts, counts)]

    sections: list[list[int]] = [flat_tokens, positions, token_seq, cu, context, layout.state_slots,
                                 list(logit_rows)]
    group_ids = sorted(layout.slots)
    n_updates = {}
    for g in group_ids:
        index, value = _update_arrays(layout.table_updates[g], storage.table_width, storage.max_seqs)
        n_updates[g] = len(index)
        sections += [layout.slots[g], index, value]
    flat: list[int] = []
    offsets = []
    for sec in sections:
        offsets.append(len(flat))
        flat.extend(sec)
        flat.extend([0] * (-len(flat) % 4))  # keep every section 16-byte aligned
    dev = uploader.upload(flat)

    def view(i: int, n: int) -> torch.Tensor:
        return dev[offsets[i]: offsets[i] + n]

    groups = {}
    for j, g in enumerate(group_ids):
        if n_updates[g]:
            ops.scatter_i32(storage.tables[g], view(8 + 3 * j, n_updates[g]), view(9 + 3 * j, n_updates[g]))
        groups[g] = GroupView(storage.tables[g], view(7 + 3 * j, n_tokens))
    num_decode = 0
    while num_decode < n_seqs and counts[num_decode] == 1:
        num_decode += 1
    return StepBatch(
        num_tokens=n_tokens, num_seqs=n_seqs, token_ids=view(0, n_tokens), positions=view(1, n_tokens),
        token_seq=view(2, n_tokens), cu_seqlens=view(3, n_seqs + 1), context_lens=view(4, n_seqs),
        state_slots=view(5, n_seqs), logit_rows=view(6, len(logit_rows)), groups=groups,
        all_rows_wanted=list(logit_rows) == list(range(n_tokens)),
        counts=list(counts), starts=list(starts), state_slot_list=list(layout.state_slots),
        num_decode=num_decode, max_count=max(counts), max_context=max(context),
        max_decode_context=max(context[:num_decode], default=0))


class StaticDecodeBatch:
    """Fixed device buffers for decode-only steps of up to `capacity` requests, so that such a step
    can be captured once as a HIP graph and replayed: every step writes its tokens, positions, slots,
    context lengths and newly taken pages into the same memory with one copy.  Unused rows belong to
    dummy requests of context length 0, which every kernel leaves alone or computes harmlessly
    (rows never mix)."""

    def __init__(self, capacity: int, storage, group_ids: list[int], device: torch.device):
        self.capacity = capacity
        self.storage = storage
        self.group_ids = list(group_ids)
        c = capacity
        sizes = [c, c, c, c + 1, c, c, c] + [c] * (3 * len(group_ids))
        self._offsets, total = [], 0
        for n in sizes:
            self._offsets.append(total)
            total += n + (-n % 4)
        self._sizes = sizes
        self.host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(total, dtype=torch.int32, device=device)
        self._event = None
        v = self._view
        groups = {g: GroupView(storage.tables[g], v(7 + 3 * j)) for j, g in enumerate(group_ids)}
        self.batch = StepBatch(
            num_tokens=c, num_seqs=c, token_ids=v(0), positions=v(1), token_seq=v(2), cu_seqlens=v(3),
            context_lens=v(4), state_slots=v(5), logit_rows=v(6), groups=groups, counts=[1] * c, starts=[0] * c,
            state_slot_list=[0] * c, num_decode=c, max_count=1, max_context=1, max_decode_context=1,
            all_rows_wanted=True)
        # what never changes: one token per request, every row's logits wanted
        h = self._host_view
        h(2)[:] = range(c)
        h(3)[:] = range(c + 1)
        h(6)[:] = range(c)
        for j in range(len(group_ids)):
            h(7 + 3 * j)[:] = -1  # until a step is filled in, no row stores anything
            h(8 + 3 * j)[:] = -1  # and no block table entry is written
        self.dev.copy_(self.host)

    def _view(self, i: int) -> torch.Tensor:
        return self.dev[self._offsets[i]: self._offsets[i] + self._sizes[i]]

    def _host_view(self, i: int):
        return self.host_np[self._offsets[i]: self._offsets[i] + self._sizes[i]]

    def apply_table_updates(self) -> None:
        """Write the step's new pages into the device block tables (part of the captured graph)."""
        from ..ops import library as ops

        for j, g in enumerate(self.group_ids):
            ops.scatter_i32(self.storage.tables[g], self._view(8 + 3 * j), self._view(9 + 3 * j))

    def fill(self, layout: StepLayout, tokens: list[int]) -> None:
        """Write a decode-only step (one token per request) into the buffers."""
        n = len(tokens)
        if self._event is not None:
            self._event.synchronize()  # the previous copy out of the pinned buffer has finished
        h = self._host_view
        h(0)[:n] = tokens
        h(0)[n:] = 0
        h(1)[:n] = layout.starts
        h(1)[n:] = 0
        ctx = h(4)
        ctx[:n] = layout.starts
        ctx[:n] += 1
        ctx[n:] = 0  # dummy requests: no keys, nothing to attend to
        h(5)[:n] = layout.state_slots
        h(5)[n:] = 0
        for j, g in enumerate(self.group_ids):
            slots = h(7 + 3 * j)
            slots[:n] = layout.slots[g]
            slots[n:] = -1  # dummy tokens store nothing
            index, value = _update_arrays(layout.table_updates[g], self.storage.table_width, self.storage.max_seqs)
            k = len(index)
            if k > self.capacity:
                raise ValueError("more new pages than requests in a decode step")
            ui, uv = h(8 + 3 * j), h(9 + 3 * j)
            ui[:k] = index
            ui[k:] = -1
            uv[:k] = value
        self.dev.copy_(self.host, non_blocking=True)
        self._event = torch.cuda.Event()
        self._event.record(torch.cuda.current_stream(self.dev.device))


class StaticStepBatch:
    """Fixed device buffers for steps of any mixture, so that such steps can be captured as HIP graphs and
    replayed: up to `decode` requests that bring one token (rows 0 .. decode-1), then up to `prefill`
    requests that bring portions, `tokens` rows in all, and `logits` wanted rows.  What a step does not
    use belongs to dummy requests without keys (context length 0, no cache slot), which every kernel
    leaves alone or computes harmlessly, rows never mixing: the unused decode rows are requests of one
    token each, the unused prefill requests bring no token, and one last dummy request owns the rows
    after the last real token."""

    def __init__(self, decode: int, prefill: int, tokens: int, logits: int, storage, group_ids: list[int],
                 device: torch.device):
        self.decode, self.prefill, self.tokens, self.logits = decode, prefill, tokens, logits
        self.storage = storage
        self.group_ids = list(group_ids)
        n, b = decode + tokens, decode + prefill + 1
        self.num_rows, self.num_seqs = n, b
        self.updates = decode + prefill + -(-tokens // storage.block_size) + 1  # new pages a step can take
        sizes = [n, n, n, b + 1, b, b, logits]
        for _ in group_ids:
            sizes += [n, self.updates, self.updates]
        self._offsets, total = [], 0
        for size in sizes:
            self._offsets.append(total)
            total += size + (-size % 4)
        self._sizes = sizes
        self.host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(total, dtype=torch.int32, device=device)
        self._event = None
        v = self._view
        groups = {g: GroupView(storage.tables[g], v(7 + 3 * j)) for j, g in enumerate(group_ids)}
        self.batch = StepBatch(
            num_tokens=n, num_seqs=b, token_ids=v(0), positions=v(1), token_seq=v(2), cu_seqlens=v(3),
            context_lens=v(4), state_slots=v(5), logit_rows=v(6), groups=groups,
            counts=[1] * decode + [0] * prefill + [tokens], starts=[0] * b, state_slot_list=[0] * b,
            num_decode=decode, max_count=max(tokens, 1), max_context=1, max_decode_context=1)
        h = self._host_view
        for j in range(len(group_ids)):
            h(7 + 3 * j)[:] = -1  # until a step is filled in, no row stores anything
            h(8 + 3 * j)[:] = -1  # and no block table entry is written
        h(2)[:decode] = range(decode)
        h(2)[decode:] = b - 1
        h(3)[: decode + 1] = range(decode + 1)
        h(3)[decode + 1: b] = decode
        h(3)[b] = n
        self.dev.copy_(self.host)

    def _view(self, i: int) -> torch.Tensor:
        return self.dev[self._offsets[i]: self._offsets[i] + self._sizes[i]]

    def _host_view(self, i: int):
        return self.host_np[self._offsets[i]: self._offsets[i] + self._sizes[i]]

    def apply_table_updates(self) -> None:
        """Write the step's new pages into the device block tables (part of the captured graph)."""
        from ..ops import library as ops

        for j, g in enumerate(self.group_ids):
            ops.scatter_i32(self.storage.tables[g], self._view(8 + 3 * j), self._view(9 + 3 * j))

    def fill(self, layout: StepLayout, tokens: list[list[int]], logit_rows: list[int]) -> None:
        """Write a step into the buffers: `layout` lists the requests that bring one token first."""
        import numpy as np

        counts, starts = layout.counts, layout.starts
        n_dec = 0
        while n_dec < len(counts) and counts[n_dec] == 1:
            n_dec += 1
        n_pre = len(counts) - n_dec
        d, b, n = self.decode, self.num_seqs, self.num_rows
        if self._event is not None:
            self._event.synchronize()  # the previous copy out of the pinned buffer has finished
        h = self._host_view
        tok, pos, seq, cu, ctx, state, rows = (h(i) for i in range(7))
        tok[:] = 0
        pos[:] = 0
        ctx[:] = 0  # dummy requests: no keys, nothing to attend to
        state[:] = 0
        # requests of one token
        tok[:n_dec] = [t[0] for t in tokens[:n_dec]]
        pos[:n_dec] = starts[:n_dec]
        ctx[:n_dec] = starts[:n_dec]
        ctx[:n_dec] += 1
        state[:n_dec] = layout.state_slots[:n_dec]
        # portions, end to end from row d; the rows behind them go to the last dummy request
        row = d
        for j in range(n_pre):
            i = n_dec + j
            c = counts[i]
            tok[row: row + c] = tokens[i]
            pos[row: row + c] = np.arange(starts[i], starts[i] + c)
            seq[row: row + c] = d + j
            ctx[d + j] = starts[i] + c
            state[d + j] = layout.state_slots[i]
            row += c
            cu[d + j + 1] = row
        seq[row:] = b - 1
        cu[d + n_pre + 1: b] = row
        used = row - d
        rows[:] = 0
        shift = d - n_dec  # a row of the step's own numbering that lies behind the decode rows moves by this
        rows[: len(logit_rows)] = [r if r < n_dec else r + shift for r in logit_rows]
        for j, g in enumerate(self.group_ids):
            slots = h(7 + 3 * j)
            slots[:] = -1  # dummy tokens store nothing
            own = layout.slots[g]
            slots[:n_dec] = own[:n_dec]
            slots[d: d + used] = own[n_dec:]
            index, value = _update_arrays(layout.table_updates[g], self.storage.table_width, self.storage.max_seqs)
            k = len(index)
            if k > self.updates:
                raise ValueError("more new pages than this batch has room for")
            ui, uv = h(8 + 3 * j), h(9 + 3 * j)
            ui[:k] = index
            ui[k:] = -1
            uv[:k] = value
        self.dev.copy_(self.host, non_blocking=True)
        self._event = torch.cuda.Event()
        self._event.record(torch.cuda.current_stream(self.dev.device))
