"""The scheduler's decisions against a stub model, on the CPU.

As in the reference's tests (tests/test_sched.py:62-126) the cache accounting is
real and the "model" is a function of a sequence's own last token and position,
next = (last * 7 + position * 13 + 1) % 64, so any difference between schedules
is a scheduling fault.  The fixtures are the reference's, as behaviours.
"""

import pytest

from paged_attention_engine_amd import CacheManager, EventKind, Request, Scheduler
from paged_attention_engine_amd.cache import PagedSpec, attention_pages, StateSpec

VOCAB = 64


class StubExecutor:
    def __init__(self, cache):
        self.cache = cache
        self.calls = 0
        self.batches = []

    def execute(self, work, record_logits=False):
        self.calls += 1
        self.batches.append([(w.seq.request_id, len(w.token_ids), w.positions[0]) for w in work])
        out = []
        for w in work:
            # positions are the run the cache implies
            held = self.cache.num_tokens(w.seq.seq_id)
            assert w.positions == tuple(range(held - len(w.token_ids), held))
            token = (w.token_ids[-1] * 7 + w.positions[-1] * 13 + 1) % VOCAB
            out.append(((token, None) if record_logits else token) if w.samples else None)
        return out


def make(num_blocks, block_size=4, window=None, slots=64, **kw):
    cache = CacheManager([attention_pages(1, 1, window)], [None], block_size, num_blocks, slots, device=None)
    executor = StubExecutor(cache)
    return Scheduler(executor, cache, **kw), cache, executor


def request(rid, prompt_len, max_new, **kw):
    return Request(rid, tuple((i * 5 + len(rid)) % VOCAB for i in range(prompt_len)), max_new, **kw)


def expected_tokens(req):
    history = list(req.prompt_token_ids)
    out = []
    for _ in range(req.max_new_tokens):
        token = (history[-1] * 7 + (len(history) - 1) * 13 + 1) % VOCAB
        out.append(token)
        history.append(token)
    return tuple(out)


def run_all(requests, **kw):
    sched, cache, executor = make(**kw)
    for r in requests:
        assert sched.add_request(r)
    out = sched.run_to_completion()
    assert all(f == g.allocator.num_blocks for f, g in zip(cache.free_blocks(), cache.groups))
    assert cache.slots.num_free == cache.slots.num_slots and not cache.sequence_ids()
    return out, sched, executor


MIXED = [request("r0", 5, 8), request("r1", 17, 8), request("r2", 33, 8), request("r3", 1, 8),
         request("r4", 9, 3), request("r5", 48, 4)]


def test_concurrent_equals_each_request_alone():
    out, sched, _ = run_all(MIXED, num_blocks=64)
    assert out == {r.request_id: expected_tokens(r) for r in MIXED}
    assert not sched.events_of(EventKind.PREEMPT)


@pytest.mark.parametrize("budget", [None, 7, 16, 2])
def test_portions_do_not_change_the_tokens(budget):
    out, sched, executor = run_all(MIXED, num_blocks=64, max_num_batched_tokens=budget)
    assert out == {r.request_id: expected_tokens(r) for r in MIXED}
    if budget is not None:
        assert all(sum(n for _, n, _ in batch) <= budget for batch in executor.batches)
        assert any(n > 1 and start > 0 for batch in executor.batches for _, n, start in batch)  # a later portion


def test_forced_preemption_is_transparent():
    growth = [request(f"g{i}", 4, 60) for i in range(4)]  # tests/test_sched.py:193-195
    out, sched, _ = run_all(growth, num_blocks=6, block_size=16)
    assert sched.events_of(EventKind.PREEMPT) and sched.events_of(EventKind.RECOMPUTE)
    assert out == {r.request_id: expected_tokens(r) for r in growth}
    for seq in sched.finished.values():
        assert seq.preemption_count == len([e for e in sched.events_of(EventKind.PREEMPT)
                                            if e.request_id == seq.request_id])


def test_admission_guard_boundary():
    sched, cache, _ = make(num_blocks=8, block_size=4, admission_margin_blocks=1)
    limit = (8 - 1) * 4  # tests/test_sched.py:298-308
    assert sched.add_request(request("fits", limit - 3, 3))
    assert not sched.add_request(request("over", limit - 3, 4))
    assert "over" in sched.rejected and sched.events_of(EventKind.REJECT)[0].request_id == "over"
    assert [s.request_id for s in sched.waiting] == ["fits"]
    out = sched.run_to_completion()
    assert set(out) == {"fits"}


def test_requests_longer_than_the_models_positions_are_rejected():
    sched, _, _ = make(num_blocks=64, max_positions=20)
    assert sched.add_request(request("ok", 10, 10))
    assert not sched.add_request(request("long", 10, 11))
    assert "positions" in sched.events_of(EventKind.REJECT)[0].detail


def test_first_come_first_served_without_backfilling():
    # tests/test_sched.py:314-337: a big request holds most of an 8-page pool; the next does not
    # fit, and the small one behind it must not jump the queue
    sched, cache, _ = make(num_blocks=8, block_size=16, admission_margin_blocks=1)
    big, head, tail = request("big", 96, 4), request("head", 32, 4), request("tail", 8, 4)
    for r in (big, head, tail):
        assert sched.add_request(r)
    result = sched.step()
    assert result.admitted == ("big",) and [s.request_id for s in sched.waiting] == ["head", "tail"]
    order = []
    while sched.waiting or sched.running:
        order += list(sched.step().admitted)
    assert order == ["head", "tail"]


def test_required_preemption_fixture():
    """tests/test_sched.py:628-733: three pages of four, A older, B newer, both on a page's edge.
    B is squeezed out exactly once, waits while A runs to its end, and is readmitted as a replay."""
    sched, cache, _ = make(num_blocks=3, block_size=4)
    a, b = request("A", 4, 4), request("B", 4, 4)
    assert sched.add_request(a) and sched.add_request(b)
    turns = 0
    while sched.waiting or sched.running:
        sched.step()
        turns += 1
        assert turns <= 8
    ev = sched.events

    def index(kind, rid):
        return [i for i, e in enumerate(ev) if e.kind is kind and e.request_id == rid]

    assert len(index(EventKind.PREEMPT, "B")) == 1 and not index(EventKind.PREEMPT, "A")
    assert len(index(EventKind.ADMIT, "B")) == 2
    preempt_b, finish_a, readmit_b = index(EventKind.PREEMPT, "B")[0], index(EventKind.FINISH, "A")[0], index(EventKind.ADMIT, "B")[1]
    assert preempt_b < finish_a < readmit_b
    assert len(index(EventKind.RECOMPUTE, "B")) == 1 and index(EventKind.RECOMPUTE, "B")[0] > preempt_b
    assert cache.free_blocks() == (3,)
    assert sched.finished["A"].preemption_count == 0 and sched.finished["B"].preemption_count == 1
    assert tuple(sched.finished["A"].generated) == expected_tokens(a)
    assert tuple(sched.finished["B"].generated) == expected_tokens(b)


def test_thrash_fixture_one_pass_per_step_and_exact_tokens():
    # tests/test_sched.py:1034-1120: 12 pages of 4, no margin, five requests of 5 + 24
    reqs = [request(f"t{i}", 5, 24) for i in range(5)]
    sched, cache, executor = make(num_blocks=12, block_size=4, admission_margin_blocks=0)
    for r in reqs:
        sched.add_request(r)
    steps, both = 0, 0
    while sched.waiting or sched.running:
        before = len(sched.events)
        calls = executor.calls
        result = sched.step()
        steps += 1
        assert executor.calls - calls == (1 if result.batch_size else 0)  # one pass per step
        kinds = {e.kind for e in sched.events[before:]}
        both += EventKind.PREEMPT in kinds and EventKind.RECOMPUTE in kinds
    assert sched.events_of(EventKind.PREEMPT) and both == 0  # a step that evicts admits nobody
    assert {rid: tuple(s.generated) for rid, s in sched.finished.items()} == {r.request_id: expected_tokens(r) for r in reqs}
    assert cache.free_blocks() == (12,)


def test_victims_are_newest_first_and_never_everyone():
    sched, cache, _ = make(num_blocks=6, block_size=16)
    for i in range(4):
        sched.add_request(request(f"g{i}", 4, 60))
    while sched.waiting or sched.running:
        running_before = [s.request_id for s in sched.running]
        result = sched.step()
        if result.preempted:
            stayed = [r for r in running_before if r not in result.preempted]
            assert stayed, "the whole running set was evicted"
            # every victim arrived after every survivor
            assert max(int(r[1:]) for r in stayed) < min(int(r[1:]) for r in result.preempted)


def test_max_num_seqs_caps_the_running_set():
    reqs = [request(f"c{i}", 8, 12) for i in range(12)]  # tests/test_sched.py:1203-1225
    for cap in (1, 2, 4, 8):
        sched, cache, _ = make(num_blocks=256, max_num_seqs=cap)
        for r in reqs:
            sched.add_request(r)
        peak = 0
        while sched.waiting or sched.running:
            result = sched.step()
            peak = max(peak, result.batch_size)
            assert result.batch_size <= cap
        assert peak == cap
        assert {k: tuple(v.generated) for k, v in sched.finished.items()} == {r.request_id: expected_tokens(r) for r in reqs}


def test_token_budget_counts_real_tokens_and_defers_decodes():
    # tests/test_sched.py:1257-1279: budget 64, one long prompt of 48 beside eight short ones
    sched, cache, executor = make(num_blocks=256, max_num_batched_tokens=64)
    reqs = [request("long", 48, 6)] + [request(f"s{i}", 4, 6) for i in range(8)]
    for r in reqs:
        sched.add_request(r)
    first = sched.step()
    assert first.batched_token_cost <= 64 and first.admitted[0] == "long"
    sched.run_to_completion()
    assert all(sum(n for _, n, _ in b) <= 64 for b in executor.batches)
    # a budget lowered below the number of running sequences defers decodes without evicting them
    sched, cache, executor = make(num_blocks=256, max_num_batched_tokens=8)
    reqs = [request(f"d{i}", 2, 5) for i in range(4)]
    for r in reqs:
        sched.add_request(r)
    assert sched.step().batch_size == 4
    sched.max_num_batched_tokens = 3
    deferred = 0
    while sched.waiting or sched.running:
        result = sched.step()
        deferred += len(result.deferred)
        assert result.batched_token_cost <= 3 and not result.preempted
    assert deferred > 0
    assert {k: tuple(v.generated) for k, v in sched.finished.items()} == {r.request_id: expected_tokens(r) for r in reqs}


def test_a_prompt_longer_than_the_budget_still_finishes():
    # tests/test_sched.py:1282-1295: 100 tokens under a budget of 16
    out, sched, executor = run_all([request("big", 100, 5)], num_blocks=64, max_num_batched_tokens=16)
    assert out["big"] == expected_tokens(request("big", 100, 5))
    assert [n for b in executor.batches[:7] for _, n, _ in b] == [16] * 6 + [4]


def test_replay_is_cut_into_portions_too():
    growth = [request(f"g{i}", 4, 40) for i in range(4)]
    out, sched, executor = run_all(growth, num_blocks=6, block_size=16, max_num_batched_tokens=5)
    assert sched.events_of(EventKind.RECOMPUTE)
    assert out == {r.request_id: expected_tokens(r) for r in growth}


def test_stop_tokens_end_a_request_early():
    r = request("s", 6, 30)
    full = expected_tokens(r)
    stop = full[4]
    cut = full[: full.index(stop) + 1]
    out, _, _ = run_all([Request("s", r.prompt_token_ids, 30, stop_token_ids=(stop,))], num_blocks=32)
    assert out["s"] == cut


def test_windowed_cache_returns_pages_while_running():
    sched, cache, _ = make(num_blocks=6, block_size=4, window=6, admission_margin_blocks=0,
                           max_num_batched_tokens=4)
    r = request("w", 30, 30)  # 60 tokens would need 15 pages without the window
    assert sched.add_request(r)
    out = sched.run_to_completion()
    assert out["w"] == expected_tokens(r) and not sched.events_of(EventKind.PREEMPT)
    assert cache.free_blocks() == (6,)


def test_step_results_and_events_carry_pool_state():
    clock = iter(range(1000))
    sched, cache, _ = make(num_blocks=16, clock=lambda: float(next(clock)))
    sched.add_request(request("a", 6, 3))
    r1 = sched.step()
    assert r1.admitted == ("a",) and r1.prefilled == ("a",) and r1.decoded == () and r1.running == 1
    r2 = sched.step()
    assert r2.decoded == ("a",) and r2.batch_size == 1 and r2.batched_token_cost == 1
    r3 = sched.step()
    assert r3.finished == ("a",) and r3.free_blocks == 16
    admit = sched.events_of(EventKind.ADMIT)[0]
    assert admit.step == 1 and admit.running == 1 and admit.timestamp == 0.0
    finish = sched.events_of(EventKind.FINISH)[0]
    assert finish.free_blocks == 16 and finish.tokens_held == 0


def test_livelock_backstop_and_argument_checks():
    sched, _, _ = make(num_blocks=16)
    sched.add_request(request("a", 4, 50))
    with pytest.raises(RuntimeError):
        sched.run_to_completion(max_steps=3)
    with pytest.raises(ValueError):
        Request("x", (), 3)
    with pytest.raises(ValueError):
        Request("x", (1,), 0)
    with pytest.raises(ValueError):
        make(num_blocks=4, max_num_seqs=0)
    with pytest.raises(ValueError):
        make(num_blocks=4, admission_margin_blocks=-1)


def test_temperature_draws_depend_on_seed_request_and_index_only():
    from paged_attention_engine_amd.sampling import uniform_for

    a = [uniform_for(5, "r1", i) for i in range(200)]
    assert a == [uniform_for(5, "r1", i) for i in range(200)]
    assert all(0.0 <= u < 1.0 for u in a) and 0.35 < sum(a) / len(a) < 0.65
    assert a != [uniform_for(6, "r1", i) for i in range(200)]
    assert a != [uniform_for(5, "r2", i) for i in range(200)]


# ------------------------------------------------------------------ steps that overlap
class LaunchingExecutor(StubExecutor):
    """The stub with the asynchronous half of the executor's surface: `launch` returns at once,
    a token id that reads PENDING is resolved from the step before (as the device does it), and
    the tokens are only handed out by `wait`."""

    class Launched:
        def __init__(self, tokens, sampling):
            self._tokens, self.sampling = tokens, sampling
            self.row_of = {id(w.seq): k for k, w in enumerate(sampling)}
            self.waited = False

        def wait(self):
            self.waited = True
            return list(self._tokens)

    def launch(self, work, previous=None):
        from paged_attention_engine_amd.engine.scheduler import PENDING
        self.calls += 1
        self.batches.append([(w.seq.request_id, len(w.token_ids), w.positions[0]) for w in work])
        assert previous is None or not previous.waited, "the step before must still be in flight when the next is launched"
        tokens, sampling = [], []
        for w in work:
            held = self.cache.num_tokens(w.seq.seq_id)
            assert w.positions == tuple(range(held - len(w.token_ids), held))
            ids = list(w.token_ids)
            for i, t in enumerate(ids):
                if t == PENDING:
                    ids[i] = previous._tokens[previous.row_of[id(w.seq)]]
            assert all(0 <= t < VOCAB for t in ids)
            if w.samples:
                tokens.append((ids[-1] * 7 + w.positions[-1] * 13 + 1) % VOCAB)
                sampling.append(w)
        return self.Launched(tokens, sampling)


@pytest.mark.parametrize("seed", range(12))
def test_overlapped_steps_decide_and_generate_what_single_steps_do(seed):
    """Random streams in pools from ample to tight (preemption, replay in portions, deferral):
    the loop that launches the next step before it has seen the current one's tokens makes the
    same batches, logs the same events and ends with the same tokens as `step()` in a loop."""
    import random
    rng = random.Random(seed)
    reqs = [request(f"r{i}", rng.randint(1, 30), rng.randint(1, 25)) for i in range(rng.randint(3, 9))]
    num_blocks = rng.choice([16, 24, 40, 200])
    kw = dict(max_num_seqs=rng.choice([None, 2, 4]), max_num_batched_tokens=rng.choice([None, 7, 16]))

    def run(overlapped):
        cache = CacheManager([attention_pages(1, 1, None)], [None], 4, num_blocks, 64, device=None)
        executor = LaunchingExecutor(cache)
        sched = Scheduler(executor, cache, **kw)
        for r in reqs:
            sched.add_request(r)
        if overlapped:
            assert sched.can_overlap()
            steps = sched.run_overlapped()
        else:
            steps = 0
            while sched.waiting or sched.running:
                sched.step()
                steps += 1
        tokens = {rid: tuple(s.generated) for rid, s in sched.finished.items()}
        events = [(e.step, e.kind, e.request_id, e.detail, e.free_blocks, e.running, e.waiting) for e in sched.events]
        assert tuple(cache.free_blocks()) == (num_blocks,)
        return steps, tokens, events, executor.batches

    one, two = run(False), run(True)
    assert one[0] == two[0] and one[1] == two[1] and one[3] == two[3]
    assert one[2] == two[2]
    for r in reqs:
        if r.request_id in one[1]:
            assert one[1][r.request_id] == expected_tokens(r)


def test_overlapped_steps_need_requests_without_stop_tokens():
    sched, _, _ = make(40)
    sched.executor = LaunchingExecutor(sched.cache)
    sched.add_request(request("a", 3, 4, stop_token_ids=(5,)))
    assert not sched.can_overlap()
    with pytest.raises(RuntimeError):
        sched.run_overlapped()
    plain, _, _ = make(40)  # the stub without launch()
    plain.add_request(request("a", 3, 4))
    assert not plain.can_overlap()


def test_overlapped_steps_stop_after_a_given_number():
    sched, _, _ = make(40)
    sched.executor = LaunchingExecutor(sched.cache)
    sched.add_request(request("a", 3, 10))
    assert sched.run_overlapped(4, until_idle=False) == 4
    seq = sched.running[0]
    assert len(seq.generated) == 4 and all(t >= 0 for t in seq.generated)  # every token has been settled
    assert sched.run_overlapped(100, until_idle=False) == 6 and "a" in sched.finished
    assert tuple(sched.finished["a"].generated) == expected_tokens(request("a", 3, 10))
