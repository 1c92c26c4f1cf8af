"""The scheduler's decisions with a fake model. The first part restates the vectors of the
reference's ``tests/test_scheduler.py`` (cited per test); the second covers what happens when pages
run out in further shapes, and random workloads that must all finish with nothing held."""

from __future__ import annotations

import random

import pytest

from mini_engine_amd.cache import BlockManager, GroupSpec
from mini_engine_amd.engine.scheduler import ScheduledSeq, Scheduler, SchedulerConfig
from mini_engine_amd.engine.sequence import SamplingParams, Sequence, SequenceStatus
from test_block_manager import check_invariants

BS = 4
EOS = 2


def make(num_blocks: int = 64, groups=(GroupSpec(),), slots: int = 0, **cfg: int) -> Scheduler:
    return Scheduler(SchedulerConfig(**cfg), BlockManager(num_blocks, BS, groups=groups, num_state_slots=slots), {EOS})


def step(s: Scheduler, token: int = 0) -> tuple[list[ScheduledSeq], list[Sequence]]:
    batch = s.schedule()
    tokens: list[int | None] = [token if item.samples else None for item in batch]
    return batch, s.postprocess(batch, tokens)


def add(s: Scheduler, n_prompt: int, max_tokens: int = 4, first: int = 10) -> Sequence:
    seq = Sequence(list(range(first, first + n_prompt)), SamplingParams(max_tokens=max_tokens))
    s.add(seq)
    return seq


# ------------------------------------------------------------------ the reference's own vectors
def test_prefill_then_decode_in_one_mixed_batch():  # :31-38
    s = make()
    a = add(s, 6)
    batch, _ = step(s)
    assert [(i.seq, i.num_tokens) for i in batch] == [(a, 6)]
    b = add(s, 5, first=100)
    batch, _ = step(s)
    assert [(i.seq, i.num_tokens) for i in batch] == [(a, 1), (b, 5)]


def test_runs_to_completion_and_frees_blocks():  # :41-49
    s = make()
    seqs = [add(s, 5, max_tokens=3, first=10 * k) for k in range(1, 4)]
    finished: list[Sequence] = []
    while s.has_unfinished():
        finished += step(s)[1]
    assert set(finished) == set(seqs)
    assert all(q.is_finished and q.num_output_tokens == 3 for q in seqs)
    assert all(rc == 0 for rc in s.bm.ref_counts)


def test_eos_stops_unless_ignored():  # :52-61
    s = make()
    a = add(s, 3, max_tokens=10)
    b = Sequence([50, 51], SamplingParams(max_tokens=3, ignore_eos=True))
    s.add(b)
    _, done = step(s, token=EOS)
    assert done == [a] and a.output_token_ids == [EOS]
    while s.has_unfinished():
        step(s, token=EOS)
    assert b.output_token_ids == [EOS] * 3


def test_max_num_seqs_caps_admission():  # :64-69
    s = make(max_num_seqs=2)
    for k in range(3):
        add(s, 3, first=10 * k + 10)
    batch, _ = step(s)
    assert len(batch) == 2 and len(s.waiting) == 1


def test_token_budget_chunks_long_prefill():  # :72-83
    s = make(max_num_batched_tokens=8)
    a = add(s, 20)
    b = add(s, 3, first=100)
    sizes = []
    while a.num_output_tokens == 0:
        batch, _ = step(s)
        sizes.append([(i.seq is a, i.num_tokens) for i in batch])
    assert sizes == [[(True, 8)], [(True, 8)], [(True, 4), (False, 3)]]
    assert b.status is SequenceStatus.RUNNING


def test_preempts_newest_and_readmits_first():  # :86-101
    s = make(num_blocks=4)
    a = add(s, 7, max_tokens=6)
    b = add(s, 7, max_tokens=6, first=100)
    step(s)
    step(s)
    batch, _ = step(s)
    assert [i.seq for i in batch] == [a]
    assert b.status is SequenceStatus.WAITING and b.num_computed_tokens == 0
    assert s.waiting[0] is b and s.num_preemptions == 1
    while s.has_unfinished():
        step(s)
    assert a.num_output_tokens == b.num_output_tokens == 6
    assert all(rc == 0 for rc in s.bm.ref_counts)


def test_preemption_keeps_generated_tokens_and_hits_prefix_cache():  # :104-118
    s = make(num_blocks=4)
    add(s, 7, max_tokens=6)
    b = add(s, 7, max_tokens=6, first=100)
    for _ in range(3):
        step(s)
    assert b.output_token_ids == [0, 0]
    while b.status is SequenceStatus.WAITING:
        step(s)
    assert b.num_cached_tokens == BS
    while s.has_unfinished():
        step(s)
    assert b.num_output_tokens == 6


def test_prefix_hit_skips_cached_tokens():  # :121-129
    s = make()
    a = add(s, 9)
    step(s)
    b = add(s, 11)
    batch, _ = step(s)
    entry = next(i for i in batch if i.seq is b)
    assert b.num_cached_tokens == 8 and entry.num_tokens == 3
    assert b.block_table[:2] == a.block_table[:2]


def test_a_step_says_when_its_items_read_pages_out_of_the_prefix_cache():
    """The second word of the packed ``live_items`` section: bit 0 is set when a quarter or more of the keys that the
    step's items read came out of the prefix cache (decode attention then keeps to loads that stay in the caches)."""
    import numpy as np

    def flags(s: Scheduler) -> int:
        lay = s.core.step_layout()
        arr = np.zeros(lay["total"], dtype=np.int32)
        s.core.step_pack(arr)
        assert arr[lay["live_items"]] == lay["items"]
        return int(arr[lay["live_items"] + 1])

    s = make()
    a = add(s, 9, max_tokens=8)
    batch = s.schedule()
    assert flags(s) == 0  # nothing cached yet
    s.postprocess(batch, [0])
    b = add(s, 11, max_tokens=8)
    batch = s.schedule()  # a decodes, b brings the 3 tokens behind its 8 cached ones: 8 of 10 + 11 keys
    assert b.num_cached_tokens == 8 and flags(s) == 1
    s.postprocess(batch, [0, 0])
    for _ in range(3):  # both decode: 8 cached of 11 + 12 keys and more
        batch = s.schedule()
        assert flags(s) == 1
        s.postprocess(batch, [0, 0])
    c = add(s, 30, max_tokens=2, first=500)  # a long request of its own: 8 of (15 + 15 + 30) keys are no quarter
    batch = s.schedule()
    assert c.num_cached_tokens == 0 and flags(s) == 0


def test_rejects_requests_that_can_never_fit():  # :132-137
    s = make(num_blocks=2, max_model_len=64)
    with pytest.raises(ValueError, match="KV blocks"):
        add(s, 8, max_tokens=4)
    with pytest.raises(ValueError, match="max_model_len"):
        make(max_model_len=10).add(Sequence([1] * 8, SamplingParams(max_tokens=4)))


# ------------------------------------------------------------------------- when pages run out
def test_no_admission_in_a_step_that_preempted_and_no_queue_jumping():
    s = make(num_blocks=4)
    a = add(s, 7, max_tokens=6)
    b = add(s, 7, max_tokens=6, first=100)
    step(s)
    step(s)
    c = add(s, 1, max_tokens=1, first=200)  # would fit, but waits behind the preempted b
    batch, _ = step(s)
    assert [i.seq for i in batch] == [a] and list(s.waiting) == [b, c]


def test_a_sequence_that_is_its_own_victim_waits_for_the_next_step():
    s = make(num_blocks=2, max_model_len=16)
    a = add(s, 7, max_tokens=1)
    hog = Sequence([1])
    assert s.bm.try_allocate(hog, 4)  # someone else holds a page
    batch, _ = step(s)
    assert batch == [] and a.status is SequenceStatus.WAITING  # cannot be admitted yet
    s.bm.free(hog)
    batch, _ = step(s)
    assert [(i.seq, i.num_tokens) for i in batch] == [(a, 7)]


def test_state_slots_limit_admission():
    s = make(slots=1)
    a, b = add(s, 3, max_tokens=2), add(s, 3, max_tokens=2, first=50)
    batch, _ = step(s)
    assert [i.seq for i in batch] == [a] and a.state_slot == 0 and b.state_slot == -1
    while not a.is_finished:
        step(s)
    batch, _ = step(s)
    assert [i.seq for i in batch] == [b] and b.state_slot == 0 and a.state_slot == -1


def test_window_group_lets_a_long_request_run_in_few_pages():
    s = make(num_blocks=4, groups=(GroupSpec(window=6),), max_num_batched_tokens=4, max_model_len=128)
    a = add(s, 30, max_tokens=20)
    while s.has_unfinished():
        step(s)
    assert a.num_output_tokens == 20 and s.num_preemptions == 0
    check_invariants(s.bm, [])


@pytest.mark.parametrize("seed", range(5))
def test_random_workloads_finish_with_nothing_held(seed):
    rng = random.Random(seed)
    s = make(num_blocks=rng.randint(12, 20), slots=4, max_num_seqs=4, max_num_batched_tokens=rng.randint(5, 16), max_model_len=48)
    seqs = []
    steps = 0
    while steps < 2000 and (s.has_unfinished() or len(seqs) < 12):
        if len(seqs) < 12 and rng.random() < 0.4:
            seqs.append(add(s, rng.randint(1, 20), max_tokens=rng.randint(1, 10), first=rng.choice([10, 10, 30])))
        if s.has_unfinished():
            batch, _ = step(s, token=rng.randrange(5))
            assert sum(i.num_tokens for i in batch) <= s.config.max_num_batched_tokens
            assert len(s.running) <= 4
            live = [q for q in seqs if q.status is SequenceStatus.RUNNING]
            check_invariants(s.bm, live)
        steps += 1
    assert all(q.is_finished for q in seqs)
    assert all(1 <= q.num_output_tokens <= q.params.max_tokens for q in seqs)
    check_invariants(s.bm, [])


# ------------------------------------------------------------------------------- one step ahead
def decode_rows(s: Scheduler) -> list[tuple[int, int, int]]:
    """(handle, first position, tokens) of the planned step's items."""
    handles, starts, counts, _, _ = s.core.step_items()
    return list(zip(handles, starts, counts))


def test_a_step_is_planned_ahead_and_settled_one_step_late():
    """Three requests decode. The step after the launched one is planned before its draws are known: every
    request advances by a stand-in token that the device feeds; the draws arrive a step late and replace
    the stand-ins. A request that reaches its count of tokens is not planned ahead, one that draws an end
    token has run one token for nothing, which the next settling passes over."""
    import numpy as np

    s = make()
    a, b, c = add(s, 5, max_tokens=8), add(s, 3, max_tokens=2, first=50), add(s, 6, max_tokens=8, first=80)
    step(s, token=7)  # the prompts; every request has one output now
    assert s.core.plan() == 3 and decode_rows(s) == [(a._handle, 5, 1), (b._handle, 3, 1), (c._handle, 6, 1)]
    # launched; b ends with this step by its count, so only a and c go on
    assert s.core.plan_ahead() == 2
    assert decode_rows(s) == [(a._handle, 6, 1), (c._handle, 7, 1)]
    assert len(a) == 7 and a.token_ids[-1] == 0 and len(b) == 4  # a stand-in at a's end, none at b's
    arr = np.zeros(64, dtype=np.int32)
    lay = s.core.step_layout()
    s.core.step_pack(arr, None, 0, 0, 0)
    source = arr[lay["token_source"]:lay["token_source"] + 2].tolist()
    assert source == [0, 2]  # a's id is row 0 of the draws in flight, c's is row 2
    with pytest.raises(RuntimeError, match="in flight"):
        s.core.plan()
    done = s.settle_in_flight(np.array([11, 12, EOS], dtype=np.int32))
    assert set(done) == {b, c} and b.output_token_ids == [7, 12] and c.output_token_ids == [7, EOS]
    assert a.token_ids[-1] == 11 and a.num_computed_tokens == 6
    # the step planned ahead is settled like any other; c's item in it counts for nothing
    assert s.core.plan_ahead() == 0  # c's item is dead: the engine settles and plans from the queues
    assert s.settle_rows(np.array([13, 99], dtype=np.int32)) == []
    assert a.output_token_ids == [7, 11, 13] and c.output_token_ids == [7, EOS] and c.is_finished
    while s.has_unfinished():
        step(s, token=5)
    assert a.num_output_tokens == 8 and all(rc == 0 for rc in s.bm.ref_counts)


def test_nothing_is_planned_ahead_when_a_request_waits_or_pages_run_out():
    s = make(max_num_seqs=4)
    a = add(s, 5, max_tokens=8)
    step(s, token=7)
    add(s, 4, max_tokens=8, first=60)  # waits and could be admitted: the next step is planned from the queues
    assert s.core.plan() == 2 and s.core.plan_ahead() == 0
    s.settle_rows(__import__("numpy").array([7, 7], dtype="int32"))
    # a full house is no reason to wait for admissions
    s2 = make(max_num_seqs=1)
    x = add(s2, 5, max_tokens=8)
    add(s2, 4, max_tokens=8, first=60)
    step(s2, token=7)
    assert s2.core.plan() == 1 and s2.core.plan_ahead() == 1
    # no page for the token after next: nothing changes, and the engine settles and plans as usual
    s3 = make(num_blocks=3)
    y = add(s3, 7, max_tokens=3)
    step(s3, token=7)  # 8 tokens: two pages, both full
    z = add(s3, 1, max_tokens=3, first=90)
    assert s3.core.plan() == 2  # y decodes, z is admitted to the third page
    assert s3.core.plan_ahead() == 0 and len(y) == 8 and len(z) == 1
    assert a is not None and x is not None


def test_random_workloads_finish_the_same_with_steps_planned_ahead():
    """The same requests and the same 'model' (the token is a function of the request and its length) with
    and without steps planned ahead, under end tokens and a small pool: equal outputs, nothing held."""
    import numpy as np

    def token_for(handle: int, length: int) -> int:
        v = (handle * 7919 + length * 104729) % 23
        return EOS if v == 0 else 3 + v

    def run(ahead: bool, seed: int) -> list[list[int]]:
        rng = random.Random(seed)
        s = make(num_blocks=24, max_num_seqs=6, max_num_batched_tokens=32)
        seqs = [add(s, rng.randint(1, 20), max_tokens=rng.randint(1, 12), first=100 * k) for k in range(14)]
        launched = None  # (handles, lengths at draw time) of a step whose draws are not settled
        steps = 0
        while s.has_unfinished() or launched is not None:
            steps += 1
            assert steps < 2000
            if launched is None:
                assert s.core.plan() > 0
                handles, starts, counts, wants, _ = s.core.step_items()
                launched = [(h, st + n + 1) if w else None for h, st, n, w in zip(handles, starts, counts, wants)]
            nxt = None
            if ahead and all(x is not None for x in launched) and s.core.plan_ahead() > 0:
                handles, starts, counts, wants, _ = s.core.step_items()
                nxt = [(h, st + n + 1) for h, st, n in zip(handles, starts, counts)]
            drawn = np.array([token_for(*x) for x in launched if x is not None], dtype=np.int32)
            if nxt is not None:
                s.settle_in_flight(drawn)
            else:
                s.settle_rows(drawn)
            launched = nxt
        assert all(rc == 0 for rc in s.bm.ref_counts)
        return [q.output_token_ids for q in seqs]

    for seed in range(6):
        assert run(True, seed) == run(False, seed)
