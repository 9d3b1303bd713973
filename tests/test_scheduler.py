"""The scheduler's decisions, on the CPU: the real cache manager and scheduler, with the plain
implementation standing in for the GPU step function.  Workloads are the reference's own
(tests/test_scheduler.py there), plus portions under a token budget."""

import pytest
import torch

import plain_llama
from conftest import TINY_A
from fakes import LaggedRunner, LaggedSampler, PlainRunner, PlainSampler
from llmserve.engine.scheduler import ContinuousBatchingEngine
from llmserve.sampling import SamplingParams
from llmserve.weights import random_tensors


@pytest.fixture(scope="module")
def weights():
    from llmserve.config import architecture_of
    from llmserve.parts.model import Model
    from llmserve.parts.registry import BuildContext

    arch = architecture_of(TINY_A)
    model = Model(arch.build_spec(arch.config_class.from_dict(TINY_A)), BuildContext(torch.float32, torch.device("cpu")))
    return random_tensors(model.param_infos(), 21, torch.float32)


def prompt(n, seed):
    return torch.randint(0, TINY_A["vocab_size"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def engine(weights, *, num_blocks=64, block_size=4, max_batch=4, budget=2048, chunk=None, lagged=False):
    """`lagged`: runner and sampler that let the scheduler read a step's tokens one step late and start
    the next step on the ids the sampler left behind, as on the GPU."""
    runner = (LaggedRunner if lagged else PlainRunner)(TINY_A, weights, num_blocks, block_size)
    return ContinuousBatchingEngine(runner, LaggedSampler() if lagged else PlainSampler(), max_num_seqs=max_batch,
                                    max_num_batched_tokens=budget, max_prefill_chunk=chunk)


LAGGED = pytest.mark.parametrize("lagged", [False, True], ids=["immediate", "lagged"])


_REFERENCE = {}


def reference(weights, p, max_new):
    key = (tuple(p), max_new)
    if key not in _REFERENCE:
        _REFERENCE[key] = plain_llama.generate(TINY_A, weights, p, max_new, torch.float32)
    return _REFERENCE[key]


WORKLOAD = [(5, 9), (13, 4), (8, 12), (3, 7), (17, 5), (6, 10)]  # (prompt_len, max_new)


@LAGGED
@pytest.mark.parametrize("budget,chunk", [(2048, None), (16, None), (8, 5), (4, 2)])
def test_batched_outputs_equal_independent_generation(weights, budget, chunk, lagged):
    eng = engine(weights, max_batch=3, budget=budget, chunk=chunk, lagged=lagged)
    prompts = [prompt(n, 100 + i) for i, (n, _) in enumerate(WORKLOAD)]
    ids = [eng.add_request(p, SamplingParams(max_new_tokens=m)) for p, (_, m) in zip(prompts, WORKLOAD)]
    done = eng.run_until_complete()
    for rid, p, (_, m) in zip(ids, prompts, WORKLOAD):
        assert done[rid].generated == reference(weights, p, m), f"request {rid}"
        assert done[rid].finish_reason == "length"
    assert eng.manager.num_free_blocks == eng.manager.num_blocks and eng.manager.num_free_slots == eng.manager.max_seqs
    assert all(sum(sizes) <= budget for sizes in eng.runner.step_sizes)
    if chunk:
        assert all(n <= chunk for sizes in eng.runner.step_sizes for n in sizes)
    assert eng.stats.tokens_generated == sum(m for _, m in WORKLOAD)
    if lagged:
        assert eng.runner.continuations > 0, "some steps must have started on tokens not yet read"


def test_portions_run_beside_decoding(weights):
    eng = engine(weights, max_batch=2, budget=6)
    a = eng.add_request(prompt(4, 1), SamplingParams(max_new_tokens=8))
    eng.step()
    b = eng.add_request(prompt(14, 2), SamplingParams(max_new_tokens=3))
    eng.step()
    assert eng.runner.step_sizes[-1] == [1, 5]  # one decoded token of a, a portion of b's prompt
    eng.step()
    assert eng.runner.step_sizes[-1] == [1, 5]
    done = eng.run_until_complete()
    assert done[a].generated == reference(weights, prompt(4, 1), 8)
    assert done[b].generated == reference(weights, prompt(14, 2), 3)


def test_requests_arriving_mid_flight_join_the_running_batch(weights):
    eng = engine(weights, max_batch=4)
    p0, p1 = prompt(6, 1), prompt(9, 2)
    r0 = eng.add_request(p0, SamplingParams(max_new_tokens=10))
    for _ in range(4):
        eng.step()
    assert len(eng.running) == 1
    r1 = eng.add_request(p1, SamplingParams(max_new_tokens=6))
    eng.step()
    assert len(eng.running) == 2
    done = eng.run_until_complete()
    assert done[r0].generated == reference(weights, p0, 10) and done[r1].generated == reference(weights, p1, 6)


def test_admission_is_in_order_and_keeps_headroom(weights):
    eng = engine(weights, num_blocks=8, block_size=4, max_batch=4)
    big = eng.add_request(prompt(20, 1), SamplingParams(max_new_tokens=4))  # 5 pages now, 6 at the end
    eng.step()
    assert [r.req_id for r in eng.running] == [big]
    eng.add_request(prompt(12, 2), SamplingParams(max_new_tokens=2))  # 3 pages + 1 spare page per live request > 3 free
    small = eng.add_request(prompt(2, 3), SamplingParams(max_new_tokens=2))  # would fit, but may not overtake
    eng.step()
    assert [r.req_id for r in eng.running] == [big] and len(eng.waiting) == 2
    done = eng.run_until_complete()
    assert done[small].generated == reference(weights, prompt(2, 3), 2)


@LAGGED
def test_preemption_recompute_preserves_greedy_outputs(weights, lagged):
    # 14 pages of 4 and four (6, 14) requests cannot all grow (tests/test_scheduler.py:69-82 there)
    eng = engine(weights, num_blocks=14, block_size=4, max_batch=4, lagged=lagged)
    work = [(6, 14)] * 4
    prompts = [prompt(n, 50 + i) for i, (n, _) in enumerate(work)]
    ids = [eng.add_request(p, SamplingParams(max_new_tokens=m)) for p, (_, m) in zip(prompts, work)]
    done = eng.run_until_complete()
    assert eng.stats.preemptions > 0, "the test must exercise preemption"
    assert sum(r.num_preemptions for r in done.values()) == eng.stats.preemptions
    for rid, p, (_, m) in zip(ids, prompts, work):
        assert done[rid].generated == reference(weights, p, m)
    assert eng.manager.num_free_blocks == eng.manager.num_blocks
    eng.manager.check_invariants()


def test_preemption_takes_the_newest_and_requeues_it_first(weights):
    eng = engine(weights, num_blocks=6, block_size=4, max_batch=3)
    ids = [eng.add_request(prompt(4, 70 + i), SamplingParams(max_new_tokens=12)) for i in range(3)]
    while eng.stats.preemptions == 0:
        eng.step()
    # all three were admitted in the first step (3 pages + 2 spare <= 6), so the newest is the last one
    assert eng.waiting[0].req_id == ids[-1]
    assert eng.waiting[0].num_computed_tokens == 0 and eng.waiting[0].num_preemptions == 1
    assert [r.req_id for r in eng.running] == ids[:2]  # the older ones keep running, in admission order
    eng.run_until_complete()
    assert eng.manager.num_free_blocks == 6


@LAGGED
def test_eos_finishes_early_and_frees_blocks(weights, lagged):
    p = prompt(7, 9)
    first = reference(weights, p, 1)[0]
    eng = engine(weights, lagged=lagged)
    rid = eng.add_request(p, SamplingParams(max_new_tokens=20, eos_token_id=first))
    done = eng.run_until_complete()
    assert done[rid].generated == [first] and done[rid].finish_reason == "stop"
    assert eng.manager.num_free_blocks == eng.manager.num_blocks


def test_abort_waiting_and_running(weights):
    eng = engine(weights, max_batch=1)
    a = eng.add_request(prompt(5, 1), SamplingParams(max_new_tokens=30))
    b = eng.add_request(prompt(5, 2), SamplingParams(max_new_tokens=30))
    eng.step()
    eng.step()
    eng.abort(b)
    eng.abort(a)
    events = eng.step()
    assert {e.req_id for e in events if e.finished} == {a, b}
    assert all(e.token is None and e.finish_reason == "abort" for e in events)
    assert not eng.has_unfinished() and eng.manager.num_free_blocks == eng.manager.num_blocks
    assert eng.finished[a].finish_reason == "abort"


def test_validate_rejects_impossible_requests(weights):
    eng = engine(weights, num_blocks=4, block_size=4)  # 16 slots in all
    with pytest.raises(ValueError, match="cache pages"):
        eng.add_request([1] * 10, SamplingParams(max_new_tokens=10))
    with pytest.raises(ValueError, match="the model stops at 128"):
        eng.add_request([1] * 200, SamplingParams(max_new_tokens=5))
    with pytest.raises(ValueError, match="empty prompt"):
        eng.add_request([], SamplingParams(max_new_tokens=5))
    with pytest.raises(ValueError, match="max_new_tokens"):
        eng.add_request([1], SamplingParams(max_new_tokens=0))
    with pytest.raises(ValueError, match="vocabulary"):
        eng.add_request([999], SamplingParams(max_new_tokens=1))
    assert not eng.has_unfinished()  # a refused request leaves nothing behind


def test_seeded_sampling_is_reproducible_and_survives_batching(weights):
    params = SamplingParams(temperature=0.9, top_k=20, seed=1234, max_new_tokens=12)
    p = prompt(6, 3)
    alone = []
    for _ in range(2):
        eng = engine(weights)
        rid = eng.add_request(p, params)
        alone.append(eng.run_until_complete()[rid].generated)
    assert alone[0] == alone[1]
    # the same request in a crowd, cut into portions, with a pool that forces preemption
    eng = engine(weights, num_blocks=12, block_size=4, max_batch=3, budget=5)
    others = [eng.add_request(prompt(5, 80 + i), SamplingParams(temperature=0.7, seed=i, max_new_tokens=14)) for i in range(2)]
    rid = eng.add_request(p, params)
    done = eng.run_until_complete()
    assert done[rid].generated == alone[0] and len(done[others[0]].generated) == 14
    assert len(set(alone[0])) > 1


def test_snapshot_and_events(weights):
    eng = engine(weights)
    rid = eng.add_request(prompt(5, 4), SamplingParams(max_new_tokens=3))
    events = eng.step()
    assert [(e.req_id, e.finished) for e in events] == [(rid, False)]
    snap = eng.snapshot()
    assert snap["running"] == 1 and snap["waiting"] == 0 and snap["free_blocks"] < snap["total_blocks"]
    assert 0 < snap["kv_utilization"] <= 1 and snap["prefill_tokens"] == 5
    events = eng.step() + eng.step()
    assert events[-1].finished and events[-1].finish_reason == "length"
    assert eng.snapshot()["decode_tokens"] == 2
    eng.add_request(prompt(5, 5), SamplingParams(max_new_tokens=3))
    eng.step()
    eng.reset()
    assert not eng.has_unfinished() and eng.manager.num_free_blocks == eng.manager.num_blocks


# ------------------------------------------------------- tokens read one step late (as on the GPU)
def test_late_reading_without_device_tokens_feeds_the_real_ids(weights):
    """A runner that cannot take tokens from the device (decode steps launched kernel by kernel) beside a
    sampler that reads late: no step may start on placeholder ids; every step's tokens come from the host."""
    from fakes import PlainRunner as Base

    class HostTokensOnly(Base):
        takes_device_tokens = False

        def step(self, entries, device_tokens=None):
            assert device_tokens is None, "this runner never said it takes tokens from the device"
            return super().step(entries)

    runner = HostTokensOnly(TINY_A, weights, 64, 4)
    eng = ContinuousBatchingEngine(runner, LaggedSampler(), max_num_seqs=3, max_num_batched_tokens=2048)
    work = [(5, 9), (13, 4), (8, 12)]
    prompts = [prompt(n, 100 + i) for i, (n, _) in enumerate(work)]
    ids = [eng.add_request(p, SamplingParams(max_new_tokens=m)) for p, (_, m) in zip(prompts, work)]
    done = eng.run_until_complete()
    for rid, p, (_, m) in zip(ids, prompts, work):
        assert done[rid].generated == reference(weights, p, m)


def test_lagged_sampling_draws_the_same_tokens(weights):
    """Reading tokens a step late must not shift which uniform number a token is drawn with."""
    work = [(6, 12, 0.9, 11), (9, 10, 0.6, 12), (4, 14, 1.2, 13)]
    outs = []
    for lagged in (False, True):
        eng = engine(weights, max_batch=3, lagged=lagged)
        ids = [eng.add_request(prompt(n, 30 + i), SamplingParams(temperature=t, top_k=20, seed=sd, max_new_tokens=m))
               for i, (n, m, t, sd) in enumerate(work)]
        done = eng.run_until_complete()
        outs.append([done[r].generated for r in ids])
        if lagged:
            assert eng.runner.continuations > 0
    assert outs[0] == outs[1]


def test_lagged_late_stop_drops_the_row_computed_for_nothing(weights):
    """A request whose end-of-sequence token is seen a step late has a row in the step already started:
    its token is dropped, its pages are freed, and the other request goes on as if alone."""
    a, b = prompt(7, 9), prompt(5, 12)
    ref_a, ref_b = reference(weights, a, 12), reference(weights, b, 12)
    stop_at = 4
    eos = ref_a[stop_at]
    assert eos not in ref_a[:stop_at] and eos not in ref_b
    eng = engine(weights, lagged=True)
    ra = eng.add_request(a, SamplingParams(max_new_tokens=12, eos_token_id=eos))
    rb = eng.add_request(b, SamplingParams(max_new_tokens=12, eos_token_id=eos))
    done = eng.run_until_complete()
    assert done[ra].generated == ref_a[: stop_at + 1] and done[ra].finish_reason == "stop"
    assert done[rb].generated == ref_b and done[rb].finish_reason == "length"
    assert eng.runner.continuations > 0
    assert eng.stats.tokens_generated == stop_at + 1 + 12
    assert eng.manager.num_free_blocks == eng.manager.num_blocks and eng.manager.num_free_slots == eng.manager.max_seqs
    eng.manager.check_invariants()


def test_lagged_abort_and_late_arrival(weights):
    eng = engine(weights, max_batch=3, lagged=True)
    r0 = eng.add_request(prompt(5, 40), SamplingParams(max_new_tokens=16))
    r1 = eng.add_request(prompt(6, 41), SamplingParams(max_new_tokens=16))
    for _ in range(5):
        eng.step()
    assert eng.runner.continuations > 0
    eng.abort(r1)
    late = eng.add_request(prompt(4, 42), SamplingParams(max_new_tokens=6))  # ends the run of continuations
    done = eng.run_until_complete()
    assert done[r1].finish_reason == "abort" and len(done[r1].generated) < 16
    assert done[r1].generated == reference(weights, prompt(6, 41), 16)[: len(done[r1].generated)]
    assert done[r0].generated == reference(weights, prompt(5, 40), 16)
    assert done[late].generated == reference(weights, prompt(4, 42), 6)
    assert eng.manager.num_free_blocks == eng.manager.num_blocks


def test_lagged_events_arrive_one_step_later_and_reset_forgets_them(weights):
    eng = engine(weights, lagged=True)
    rid = eng.add_request(prompt(5, 4), SamplingParams(max_new_tokens=3))
    assert eng.step() == []  # the prompt went in; its token has not been read
    assert eng.has_unfinished()
    events = eng.step()
    assert [(e.req_id, e.finished) for e in events] == [(rid, False)]
    events = eng.step() + eng.step() + eng.step()
    assert [e.finished for e in events] == [False, True] and not eng.has_unfinished()
    eng.add_request(prompt(5, 5), SamplingParams(max_new_tokens=3))
    eng.step()
    eng.reset()
    assert not eng.has_unfinished() and eng.manager.num_free_blocks == eng.manager.num_blocks
    assert eng.step() == []


# ------------------------------------------------------------------ what a request costs is the cache manager's answer
class CountingRunner:
    """A step function for models that are not the reference's: the real cache manager over the given groups, and
    logits that name (sum of the request's tokens so far) % vocab, kept per state slot as a model with fixed-size
    state would keep it."""

    def __init__(self, groups, num_blocks, block_size, max_seqs, vocab=50, max_model_len=4096):
        from llmserve.cache import CacheManager

        self.manager = CacheManager(groups, num_blocks, block_size, max_seqs)
        self.vocab_size, self.max_model_len = vocab, max_model_len
        self.sums = [0] * max_seqs
        self.peak_used: dict[int, int] = {}

    def step(self, entries):
        layout = self.manager.append([e.seq_id for e in entries], [len(e.tokens) for e in entries])
        for gid, a in self.manager.allocators.items():
            self.peak_used[gid] = max(self.peak_used.get(gid, 0), a.num_used)
        for slot in layout.fresh_slots:
            self.sums[slot] = 0
        rows = []
        for e, slot in zip(entries, layout.state_slots):
            for i, t in enumerate(e.tokens):
                self.sums[slot] += t
                if i in e.want:
                    rows.append(torch.nn.functional.one_hot(torch.tensor(self.sums[slot] % self.vocab_size), self.vocab_size).float())
        self.manager.release_passed(layout.seq_ids)
        return torch.stack(rows) if rows else torch.empty(0, self.vocab_size)


def counted(p, max_new, vocab=50):
    ids = list(p)
    for _ in range(max_new):
        ids.append(sum(ids) % vocab)
    return ids[len(p):]


def test_a_model_that_keeps_only_fixed_size_state_is_served_with_default_sizing():
    """No layer has pages: the pools are sized as the runner sizes them from a byte budget (none at all), and the
    scheduler admits by slots alone; requests far longer than any page count would allow go through."""
    from llmserve.cache import group_layers
    from llmserve.cache.storage import pool_sizes_for_budget
    from llmserve.parts.spec import StateCacheSpec

    groups = group_layers([StateCacheSpec((6,), "float32")] * 2)
    sizes = pool_sizes_for_budget(groups, 16, 2, 1 << 20, max_seqs=2, longest=4096, step_tokens=64)
    assert sizes == {}
    eng = ContinuousBatchingEngine(CountingRunner(groups, sizes, 16, 2), PlainSampler(), max_num_seqs=2,
                                   max_num_batched_tokens=64)
    prompts = [[(7 * i + j) % 50 for j in range(n)] for i, n in enumerate([48, 300, 5, 1000])]
    ids = [eng.add_request(p, SamplingParams(max_new_tokens=6)) for p in prompts]
    done = eng.run_until_complete()
    for rid, p in zip(ids, prompts):
        assert done[rid].generated == counted(p, 6)
    assert eng.stats.preemptions == 0 and eng.manager.num_free_slots == 2
    with pytest.raises(ValueError, match="positions"):
        eng.add_request([1] * 4096, SamplingParams(max_new_tokens=1))


def test_admission_charges_every_cache_group_what_it_costs_there():
    """Two groups: one keeps every key (a large pool), one keeps a window of 8 keys (a small pool).  A prompt of 90
    tokens costs 23 pages in the first and, in portions of up to 8 tokens, never more than 5 in the second, which
    has 12: two such requests run side by side, where charging ceil(tokens / block_size) against the smaller
    pool would refuse every one of them."""
    from llmserve.cache import group_layers
    from llmserve.parts.spec import PagedCacheSpec

    full, windowed = PagedCacheSpec(1, 16), PagedCacheSpec(1, 16, window=8)
    groups = group_layers([full, windowed])
    gid = {g.spec: g.group_id for g in groups}
    runner = CountingRunner(groups, {gid[full]: 60, gid[windowed]: 12}, 4, 3)
    eng = ContinuousBatchingEngine(runner, PlainSampler(), max_num_seqs=3, max_num_batched_tokens=16, max_prefill_chunk=8)
    prompts = [[(3 * i + j) % 50 for j in range(90)] for i in range(3)]
    ids = [eng.add_request(p, SamplingParams(max_new_tokens=4)) for p in prompts]
    eng.step()
    assert len(eng.running) == 2 and len(eng.waiting) == 1  # the full group has room for two (2 x 24 + spare), not three
    done = eng.run_until_complete()
    for rid, p in zip(ids, prompts):
        assert done[rid].generated == counted(p, 4)
    assert runner.peak_used[gid[windowed]] <= 2 * 5 and runner.peak_used[gid[full]] >= 46
    assert eng.manager.free_pages() == eng.manager.capacity() and eng.stats.preemptions == 0
    with pytest.raises(ValueError, match="whole pool is 60"):  # the group that keeps every key is the one that refuses
        eng.add_request([1] * 300, SamplingParams(max_new_tokens=4))


def test_an_id_that_is_live_is_refused_and_reset_forgets_cancellations(weights):
    eng = engine(weights, max_batch=2)
    eng.add_request(prompt(5, 1), SamplingParams(max_new_tokens=3), req_id=7)
    with pytest.raises(ValueError, match="already queued or running"):
        eng.add_request(prompt(4, 2), SamplingParams(max_new_tokens=3), req_id=7)
    eng.step()
    with pytest.raises(ValueError, match="already queued or running"):
        eng.add_request(prompt(4, 2), SamplingParams(max_new_tokens=3), req_id=7)
    eng.abort(7)
    eng.reset()  # the cancellation of the old request 7 must not hit a new one
    eng.add_request(prompt(4, 2), SamplingParams(max_new_tokens=3), req_id=7)
    done = eng.run_until_complete()
    assert done[7].finish_reason == "length" and done[7].generated == reference(weights, prompt(4, 2), 3)
