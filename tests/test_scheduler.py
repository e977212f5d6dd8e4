"""The scheduler's decisions on the CPU, with a stand-in for the step function.

Vectors of the reference's scheduler tests (tests/test_scheduler.py) run with chunked prefill
off, where our scheduler must decide exactly as the reference does; the rest covers what is
new: portions under the token budget, and what happens when pages run out."""

import pytest

from clockwork_amd.cache import CacheManager, PrefixCache, plan_groups
from clockwork_amd.config.engine import SchedulerConfig
from clockwork_amd.config.spec import KVPagesSpec
from clockwork_amd.engine.scheduler import Scheduler
from clockwork_amd.engine.sequence import SamplingParams, Sequence, SequenceStatus

BS = 4


def make_env(num_blocks=64, max_num_seqs=8, budget=64, watermark=0.0, prefix=False, chunked=False, chunk=0):
    manager = CacheManager(plan_groups([KVPagesSpec(1, 16)]), BS, num_blocks, max_num_seqs, watermark)
    cache = PrefixCache(BS, manager.share_handle, manager.drop_handle) if prefix else None
    cfg = SchedulerConfig(max_num_seqs=max_num_seqs, max_num_batched_tokens=budget,
                          enable_chunked_prefill=chunked, max_prefill_chunk=chunk)
    return Scheduler(cfg, manager, cache), manager, cache


def make_seq(seq_id, prompt, arrival, max_tokens=64):
    return Sequence(seq_id, list(prompt), SamplingParams(max_tokens=max_tokens), arrival_time=arrival)


def apply(sched, out):
    """What the engine does after a step: mark the portion computed, append a token where one
    was sampled, finish at max_tokens, give back what finished requests held."""
    for p in out.portions:
        p.seq.num_computed_tokens = p.start + p.num_tokens
        if p.samples:
            p.seq.append_token(7)
            if len(p.seq.output_token_ids) >= p.seq.sampling_params.max_tokens:
                p.seq.status = SequenceStatus.FINISHED_LENGTH
    sched.free_finished()


def engine_step(sched):
    out = sched.schedule()
    apply(sched, out)
    return out


def ids(seqs):
    return [s.seq_id for s in seqs]


# ------------------------------------------------------------------ the reference's vectors
def test_token_budget_splits_a_batch():
    # tests/test_scheduler.py:49-67
    sched, _, _ = make_env(budget=10)
    a, b = make_seq("a", range(6), 0.0), make_seq("b", range(6), 1.0)
    sched.add_seq(a)
    sched.add_seq(b)
    out1 = sched.schedule()
    assert ids(out1.prefill_seqs) == ["a"] and out1.decode_seqs == [] and out1.num_batched_tokens == 6
    assert b.status is SequenceStatus.WAITING
    apply(sched, out1)
    out2 = sched.schedule()
    assert ids(out2.decode_seqs) == ["a"] and ids(out2.prefill_seqs) == ["b"] and out2.num_batched_tokens == 7


def test_max_num_seqs_cap():
    sched, _, _ = make_env(max_num_seqs=2)
    a, b, c = make_seq("a", range(4), 0.0, 1), make_seq("b", range(4), 1.0, 8), make_seq("c", range(4), 2.0, 8)
    for s in (a, b, c):
        sched.add_seq(s)
    out1 = engine_step(sched)
    assert ids(out1.prefill_seqs) == ["a", "b"] and c.status is SequenceStatus.WAITING and a.is_finished()
    out2 = engine_step(sched)
    assert ids(out2.decode_seqs) == ["b"] and ids(out2.prefill_seqs) == ["c"]


def pressure_env(max_num_seqs=2):
    # tests/test_scheduler.py:88-96: 6 pages; two 2-page prompts fit, decode growth runs the pool dry
    sched, manager, _ = make_env(num_blocks=6, max_num_seqs=max_num_seqs)
    a, b = make_seq("a", range(8), 0.0, 6), make_seq("b", range(100, 108), 1.0, 6)
    sched.add_seq(a)
    sched.add_seq(b)
    return sched, manager, a, b


def run_until_preemption(sched, limit=20):
    for _ in range(limit):
        out = engine_step(sched)
        if out.preempted:
            return out
    raise AssertionError("no preemption occurred")


def test_preemption_recompute_and_readmission():
    sched, manager, a, b = pressure_env()
    out = run_until_preemption(sched)
    assert ids(out.preempted) == ["b"]  # the latest arrival is the victim
    assert b.status is SequenceStatus.PREEMPTED and b.num_computed_tokens == 0 and not manager.has("b")
    assert sched.waiting[0] is b and a in out.decode_seqs and sched.stats.num_preempted_total == 1
    for _ in range(20):
        if b.is_finished():
            break
        engine_step(sched)
    assert b.status is SequenceStatus.FINISHED_LENGTH and len(b.output_token_ids) == 6
    assert a.status is SequenceStatus.FINISHED_LENGTH and not sched.has_unfinished()
    assert manager.num_free_blocks() == 6


def test_preempted_requests_are_readmitted_before_newcomers():
    sched, _, a, b = pressure_env()
    c = make_seq("c", range(200, 204), 2.0, 2)
    sched.add_seq(c)
    run_until_preemption(sched)
    assert ids(sched.waiting) == ["b", "c"]
    for _ in range(20):
        out = sched.schedule()
        if out.prefill_seqs:
            break
        apply(sched, out)
    assert out.prefill_seqs[0] is b and b.status is SequenceStatus.RUNNING


def cached_env(budget):
    sched, manager, cache = make_env(num_blocks=16, budget=budget, prefix=True)
    tokens = list(range(100, 112))
    handles = [(p,) for p in manager.pools[0].take_many(2)]
    cache.insert(tokens[:8], handles)
    for h in handles:
        manager.drop_handle(h)
    return sched, manager, cache, tokens, handles


def test_prefix_hit_lowers_the_admission_cost():
    # tests/test_scheduler.py:173-194
    sched, manager, _, tokens, handles = cached_env(budget=6)
    seq = make_seq("s", tokens, 0.0)
    sched.add_seq(seq)
    out = sched.schedule()
    assert ids(out.prefill_seqs) == ["s"] and out.num_batched_tokens == 4
    assert seq.num_cached_tokens == 8 and seq.num_computed_tokens == 8
    assert manager.block_table("s")[:2] == [h[0] for h in handles] and len(manager.block_table("s")) == 3
    assert sched.stats.total_cached_tokens == 8 and sched.stats.total_prompt_tokens == 12
    cold_sched, _, _, _, _ = cached_env(budget=6)
    cold = make_seq("cold", range(200, 212), 0.0)
    cold_sched.add_seq(cold)
    assert cold_sched.schedule().is_empty() and cold.status is SequenceStatus.WAITING


def test_failed_admission_undoes_the_prefix_match():
    # tests/test_scheduler.py:197-209
    sched, manager, cache, tokens, handles = cached_env(budget=3)
    seq = make_seq("s", tokens, 0.0)
    sched.add_seq(seq)
    assert sched.schedule().is_empty()
    assert not manager.has("s") and seq.num_cached_tokens == 0 and seq.num_computed_tokens == 0
    assert cache.evictable_blocks() == 2
    assert all(manager.pools[0].refcount(h[0]) == 1 for h in handles)


def test_abort_in_every_state():
    sched, manager, _ = make_env()
    a = make_seq("a", range(4), 0.0)
    sched.add_seq(a)
    sched.abort("a")
    assert a.status is SequenceStatus.FINISHED_ABORTED and not sched.has_unfinished()
    b = make_seq("b", range(6), 1.0)
    sched.add_seq(b)
    sched.schedule()
    assert b.status is SequenceStatus.RUNNING
    sched.abort("b")
    assert b.status is SequenceStatus.FINISHED_ABORTED and sched.running == [] and manager.num_free_blocks() == 64
    sched.abort("missing")  # a no-op
    sched2, manager2, a2, b2 = pressure_env()
    run_until_preemption(sched2)
    sched2.abort("b")
    assert b2.status is SequenceStatus.FINISHED_ABORTED and b2 not in sched2.waiting
    for _ in range(20):
        if not sched2.has_unfinished():
            break
        engine_step(sched2)
    assert a2.is_finished() and manager2.num_free_blocks() == 6


def test_abort_running_releases_prefix_locks():
    sched, manager, cache, tokens, handles = cached_env(budget=64)
    seq = make_seq("s", tokens, 0.0)
    sched.add_seq(seq)
    sched.schedule()
    assert seq.num_cached_tokens == 8 and cache.evictable_blocks() == 0
    sched.abort("s")
    assert manager.num_free_blocks() == 14 and cache.evictable_blocks() == 2
    assert all(manager.pools[0].refcount(h[0]) == 1 for h in handles)


def scripted_session(chunked):
    # tests/test_scheduler.py:270-301: 7 pages, budget 16; admission splits, preemptions, drain
    sched, manager, _ = make_env(num_blocks=7, max_num_seqs=3, budget=16, chunked=chunked)
    seqs = [make_seq("a", range(8), 0.0, 6), make_seq("b", range(100, 108), 1.0, 6),
            make_seq("c", range(200, 204), 2.0, 4), make_seq("d", range(300, 312), 3.0, 3)]
    for s in seqs:
        sched.add_seq(s)
    history = []
    for _ in range(60):
        out = engine_step(sched)
        history.append((tuple((p.seq.seq_id, p.start, p.num_tokens) for p in out.portions),
                        tuple(ids(out.preempted)), out.num_batched_tokens))
        # pages are held only by running requests
        assert set(manager.live_requests()) == {s.seq_id for s in sched.running}
        if not sched.has_unfinished():
            break
    assert not sched.has_unfinished() and manager.num_free_blocks() == 7
    assert [len(s.output_token_ids) for s in seqs] == [6, 6, 4, 3]
    return history


@pytest.mark.parametrize("chunked", [False, True])
def test_a_scripted_session_is_deterministic_and_drains(chunked):
    h = scripted_session(chunked)
    assert h == scripted_session(chunked)
    assert any(step[1] for step in h), "the session was meant to force a preemption"


# ------------------------------------------------------------------ chunked prefill
def test_a_prompt_longer_than_the_budget_runs_in_portions():
    sched, manager, _ = make_env(budget=10, chunked=True)
    a = make_seq("a", range(25), 0.0, 2)
    sched.add_seq(a)
    seen = []
    for _ in range(6):
        out = engine_step(sched)
        seen.append([(p.start, p.num_tokens, p.samples) for p in out.portions])
        if a.is_finished():
            break
    assert seen == [[(0, 10, False)], [(10, 10, False)], [(20, 5, True)], [(25, 1, True)]]
    assert manager.num_free_blocks() == 64


def test_decoding_requests_go_first_and_prefill_takes_the_rest_of_the_budget():
    sched, _, _ = make_env(budget=8, chunked=True)
    a, b = make_seq("a", range(3), 0.0, 10), make_seq("b", range(30), 1.0, 2)
    sched.add_seq(a)
    out = engine_step(sched)
    assert [(p.seq.seq_id, p.num_tokens) for p in out.portions] == [("a", 3)]
    sched.add_seq(b)
    out = engine_step(sched)
    assert [(p.seq.seq_id, p.start, p.num_tokens, p.samples) for p in out.portions] == [("a", 3, 1, True), ("b", 0, 7, False)]
    assert ids(out.decode_seqs) == ["a"] and ids(out.prefill_seqs) == ["b"] and out.num_batched_tokens == 8
    out = engine_step(sched)
    assert [(p.seq.seq_id, p.start, p.num_tokens) for p in out.portions] == [("a", 4, 1), ("b", 7, 7)]


def test_max_prefill_chunk_caps_a_portion_and_two_prompts_share_a_step():
    sched, _, _ = make_env(budget=64, chunked=True, chunk=5)
    a, b = make_seq("a", range(12), 0.0, 1), make_seq("b", range(7), 1.0, 1)
    sched.add_seq(a)
    sched.add_seq(b)
    out = engine_step(sched)
    assert [(p.seq.seq_id, p.start, p.num_tokens) for p in out.portions] == [("a", 0, 5), ("b", 0, 5)]
    out = engine_step(sched)
    assert [(p.seq.seq_id, p.start, p.num_tokens, p.samples) for p in out.portions] == [("a", 5, 5, False), ("b", 5, 2, True)]


def test_admission_sets_pages_aside_for_the_whole_request():
    """A half-prefilled request never has to fight for pages to finish its prompt: the second
    request waits although its first portion alone would fit."""
    sched, manager, _ = make_env(num_blocks=8, budget=8, chunked=True)
    a, b = make_seq("a", range(20), 0.0, 1), make_seq("b", range(16), 1.0, 1)
    sched.add_seq(a)
    sched.add_seq(b)
    out = sched.schedule()
    assert [(p.seq.seq_id, p.num_tokens) for p in out.portions] == [("a", 8)]
    assert len(manager.block_table("a")) == 5 and b.status is SequenceStatus.WAITING


def test_a_half_prefilled_request_can_be_the_victim_and_starts_over():
    # a (8-token prompt) decodes and grows; b's 16-token prompt is set aside whole (4 pages) and
    # runs in portions of 2; a's next page edge comes while b is still in its prompt
    sched, manager, _ = make_env(num_blocks=7, budget=3, chunked=True)
    a = make_seq("a", range(8), 0.0, 12)
    sched.add_seq(a)
    for _ in range(3):
        engine_step(sched)  # 3 + 3 + 2 tokens of the prompt, first token sampled
    assert len(a) == 9 and a.num_uncomputed_tokens() == 1
    b = make_seq("b", range(100, 116), 1.0, 2)
    sched.add_seq(b)
    before = None
    for _ in range(10):
        before = b.num_computed_tokens
        out = engine_step(sched)
        if out.preempted:
            break
    assert ids(out.preempted) == ["b"] and 0 < before < 16, "b was meant to be caught in its prompt"
    assert b.num_computed_tokens == 0 and b.status is SequenceStatus.PREEMPTED and not manager.has("b")
    assert ids(out.decode_seqs) == ["a"]
    for _ in range(40):
        if not sched.has_unfinished():
            break
        engine_step(sched)
    assert a.is_finished() and b.is_finished() and len(b.output_token_ids) == 2
    assert manager.num_free_blocks() == 7


def test_idle_prefix_blocks_are_evicted_before_a_request_is_refused_or_preempted():
    sched, manager, cache = make_env(num_blocks=6, budget=64, prefix=True, chunked=True)
    first = make_seq("first", range(16), 0.0, 1)
    sched.add_seq(first)
    engine_step(sched)
    # the engine inserts finished prompts; stand in for it here
    handles = [(p,) for p in manager.pools[0].take_many(4)]
    cache.insert(list(range(500, 516)), handles)
    for h in handles:
        manager.drop_handle(h)
    assert manager.num_free_blocks() == 2 and cache.evictable_blocks() == 4
    big = make_seq("big", range(300, 320), 1.0, 3)  # 5 pages, then a sixth while decoding
    sched.add_seq(big)
    out = engine_step(sched)
    assert ids(out.prefill_seqs) == ["big"] and cache.num_blocks() <= 1
    for _ in range(4):
        out = engine_step(sched)
        assert not out.preempted
    assert big.is_finished()
    cache.reset()
    assert manager.num_free_blocks() == 6


def test_pages_run_out_for_the_only_request():
    """Nothing else to preempt: the request itself is preempted and waits; with a pool that can
    never hold it the scheduler keeps returning an empty schedule (the engine raises)."""
    sched, manager, _ = make_env(num_blocks=2, budget=64, chunked=True)
    a = make_seq("a", range(8), 0.0, 4)
    sched.add_seq(a)
    engine_step(sched)
    out = engine_step(sched)  # position 8 needs a third page
    assert ids(out.preempted) == ["a"] and not out.portions
    out = sched.schedule()  # 9 tokens now need 3 pages: never admissible
    assert out.is_empty() and a.status is SequenceStatus.PREEMPTED and manager.num_free_blocks() == 2


def test_stats_count_admissions_and_batches():
    sched, _, _ = make_env()
    a = make_seq("a", range(5), 0.0, 2)
    sched.add_seq(a)
    assert (sched.stats.num_waiting, sched.stats.num_running) == (1, 0)
    engine_step(sched)
    assert (sched.stats.num_waiting, sched.stats.num_running, sched.stats.total_prompt_tokens) == (0, 1, 5)
    engine_step(sched)
    assert sched.stats.num_scheduled_batches == 2 and sched.stats.num_running == 0


# ------------------------------------------------------------------ one step ahead
def portions_of(out):
    return [(p.seq.seq_id, p.start, p.num_tokens, p.samples) for p in out.portions]


def run_session(use_ahead: bool):
    """Three requests of different lengths, one arriving late; returns each step's portions."""
    sched, manager, _ = make_env(num_blocks=64, budget=16, chunked=True)
    sched.add_seq(make_seq("a", range(5), 0.0, max_tokens=9))
    sched.add_seq(make_seq("b", range(11), 1.0, max_tokens=4))
    late = make_seq("c", range(3), 2.0, max_tokens=6)
    history, ahead, used = [], None, 0
    for step in range(40):
        if step == 7:
            sched.add_seq(late)
        if ahead is not None and ahead.version == sched.version:
            out = ahead
            sched.commit_ahead(out)
            used += 1
        else:
            out = sched.schedule()
        if not out.portions:
            break
        history.append(portions_of(out))
        # the engine looks ahead while the step runs, before its tokens are known
        ahead = sched.schedule_ahead(out) if use_ahead else None
        apply(sched, out)
    assert not sched.has_unfinished()
    assert manager.min_free_blocks() == manager.num_blocks
    return history, used, sched.stats.num_scheduled_batches


def test_schedule_ahead_decides_what_schedule_would():
    plain_history, _, plain_batches = run_session(False)
    ahead_history, used, ahead_batches = run_session(True)
    assert ahead_history == plain_history
    assert ahead_batches == plain_batches
    assert used >= 5  # the plain decode stretches ran from schedules made ahead


def test_schedule_ahead_leaves_the_hard_cases_to_schedule():
    sched, manager, _ = make_env(num_blocks=8, budget=16, chunked=True)
    a = make_seq("a", range(6), 0.0, max_tokens=3)
    sched.add_seq(a)
    out = sched.schedule()                      # the prompt: a portion, not a decode step
    assert sched.schedule_ahead(out) is None
    apply(sched, out)
    out = sched.schedule()                      # first decode step; the token after it is the last (3 of 3)
    assert portions_of(out) == [("a", 6, 1, True)]
    ahead = sched.schedule_ahead(out)
    assert ahead is not None and portions_of(ahead) == [("a", 7, 1, True)]
    apply(sched, out)
    sched.commit_ahead(ahead)
    assert sched.schedule_ahead(ahead) is None  # max_tokens: this token ends the request
    # somebody waits: the ordinary schedule has to look at admission
    sched2, _, _ = make_env(num_blocks=8, budget=16, chunked=True)
    sched2.add_seq(make_seq("x", range(4), 0.0))
    apply(sched2, sched2.schedule())
    out = sched2.schedule()
    sched2.add_seq(make_seq("y", range(4), 1.0))
    assert sched2.schedule_ahead(out) is None
    # a schedule made ahead goes stale when a request is aborted
    sched3, _, _ = make_env(num_blocks=8, budget=16, chunked=True)
    sched3.add_seq(make_seq("p", range(4), 0.0))
    sched3.add_seq(make_seq("q", range(4), 1.0))
    apply(sched3, sched3.schedule())
    out = sched3.schedule()
    ahead = sched3.schedule_ahead(out)
    assert ahead is not None
    apply(sched3, out)
    sched3.abort("q")
    assert ahead.version != sched3.version
    with pytest.raises(RuntimeError):
        sched3.commit_ahead(ahead)


def test_schedule_ahead_never_preempts_or_evicts():
    # 3 pages of 4: two requests of 5 tokens hold 2 pages each? no: one page is free for one of them only
    sched, manager, _ = make_env(num_blocks=4, budget=16, chunked=True)
    a, b = make_seq("a", range(4), 0.0), make_seq("b", range(4), 1.0)
    sched.add_seq(a)
    sched.add_seq(b)
    apply(sched, sched.schedule())              # both prompts; each holds one full page
    out = sched.schedule()                      # decode at position 4: a second page each
    assert len(out.portions) == 2 and manager.min_free_blocks() == 0
    ahead = sched.schedule_ahead(out)           # position 5 lies in the pages they hold
    assert ahead is not None
    apply(sched, out)
    sched.commit_ahead(ahead)
    apply(sched, ahead)
    for _ in range(2):                          # positions 6 and 7
        out = sched.schedule()
        apply(sched, out)
    before = sched.stats.num_preempted_total
    assert sched.schedule_ahead(out) is None    # position 8 needs a page that is not there
    assert sched.stats.num_preempted_total == before and len(sched.running) == 2
    out = sched.schedule()                      # the ordinary schedule preempts the later request
    assert ids(out.preempted) == ["b"]


def test_schedule_ahead_counts_the_pages_of_all_requests_together():
    # 7 pages of 4: three requests of 4 tokens hold a page each and decode their fifth token into a
    # second one (6 held); at position 8 each needs a third page and one is free: each alone could
    # go on, all three cannot, and looking ahead must leave that to the ordinary schedule
    # untouched (it once took pages for the first requests and then failed on the last)
    sched, manager, _ = make_env(num_blocks=7, budget=16, chunked=True)
    seqs = [make_seq(name, range(4), float(i)) for i, name in enumerate("abc")]
    for seq in seqs:
        sched.add_seq(seq)
    apply(sched, sched.schedule())              # the prompts
    for _ in range(4):                          # positions 4 to 7
        out = sched.schedule()
        assert len(out.portions) == 3
        apply(sched, out)
    assert manager.min_free_blocks() == 1
    assert all(manager.can_extend(s.seq_id, 8, 9) for s in seqs)
    assert not manager.can_extend_all([(s.seq_id, 8, 9) for s in seqs])
    held = {s.seq_id: list(manager.block_table(s.seq_id, 0)) for s in seqs}
    assert sched.schedule_ahead(out) is None
    assert manager.min_free_blocks() == 1 and held == {s.seq_id: list(manager.block_table(s.seq_id, 0)) for s in seqs}
    out = sched.schedule()                      # the ordinary schedule makes room by preempting
    assert ids(out.preempted) and len(out.portions) + len(out.preempted) >= 2


def test_a_preempted_request_that_outgrew_the_budget_runs_again_in_portions():
    # chunked prefill off, a budget of 8 tokens, 5 pages of 4. Two prompts of 7 tokens run whole,
    # one after the other. Both generate; at position 8 each needs a third page and there is one:
    # b, the later arrival, is preempted with 7 + 2 = 9 tokens, more than a step may hold. Once a
    # is finished b must come back, in a portion of 8 tokens and then the rest, not wait forever.
    sched, manager, _ = make_env(num_blocks=5, budget=8, chunked=False)
    a, b = make_seq("a", range(7), 0.0, max_tokens=6), make_seq("b", range(7), 1.0, max_tokens=6)
    sched.add_seq(a)
    sched.add_seq(b)
    preempted = False
    for _ in range(12):
        out = engine_step(sched)
        preempted = preempted or ids(out.preempted) == ["b"]
        if a.is_finished():
            break
    assert preempted and a.is_finished() and b.status is SequenceStatus.PREEMPTED and len(b) == 9
    out = engine_step(sched)
    assert [(p.seq.seq_id, p.start, p.num_tokens, p.samples) for p in out.portions] == [("b", 0, 8, False)]
    out = engine_step(sched)
    assert [(p.seq.seq_id, p.start, p.num_tokens, p.samples) for p in out.portions] == [("b", 8, 1, True)]
    while not b.is_finished():
        engine_step(sched)
    assert len(b.output_token_ids) == 6 and manager.min_free_blocks() == 5
    # a prompt that is longer than the budget still never runs without chunked prefill
    sched2, _, _ = make_env(num_blocks=16, budget=8, chunked=False)
    sched2.add_seq(make_seq("long", range(9), 0.0))
    assert not sched2.schedule().portions


# 1424 and 1950: a step decided ahead for requests that each alone, but not all together, find a page
@pytest.mark.parametrize("seed", [*range(300), 1424, 1950])
def test_random_sessions_end_with_every_page_back(seed):
    """Scheduler options and sessions drawn at random, run as the engine runs them (a step decided
    ahead is used when nothing changed meanwhile; when nothing can run, the idle prefix blocks are
    evicted once): requests arrive over time, stop at random tokens or at their length, are aborted
    now and then. No step raises, every request ends, the page pools pass their audit after every
    step and are whole at the end, and a request never holds fewer pages than its cached tokens need."""
    import random

    rng = random.Random(seed)
    chunked = rng.random() < 0.7
    budget = rng.choice([8, 16, 48, 96])
    max_prompt = 60
    if not chunked:
        budget = max(budget, max_prompt)
    num_blocks = rng.choice([24, 32, 64, 200])  # pages of 4: the longest request (60 + 40 tokens) fits alone
    sched, manager, cache = make_env(num_blocks=max(num_blocks, (max_prompt + 40) // BS + 2), max_num_seqs=rng.choice([2, 4, 12]),
                                     budget=budget, watermark=rng.choice([0.0, 0.05]), prefix=rng.random() < 0.6,
                                     chunked=chunked, chunk=rng.choice([0, 0, 7]))
    opening = [rng.randrange(50) for _ in range(32)]
    pending = []
    for i in range(rng.randint(3, 40)):
        prompt = (opening[: rng.choice([0, 0, 4, 17, 32])] + [rng.randrange(50) for _ in range(rng.choice([1, 2, 9, 30]))])[:max_prompt]
        pending.append(make_seq(f"q{i}", prompt, float(i), max_tokens=rng.choice([1, 2, 10, 40])))
    seqs = list(pending)

    def run(out):
        """The stand-in for the step: tokens drawn at random, one in ten of them a stop token."""
        for p in out.portions:
            p.seq.num_computed_tokens = p.start + p.num_tokens
            if p.samples:
                p.seq.append_token(rng.randrange(50))
                if rng.random() < 0.1:
                    p.seq.status = SequenceStatus.FINISHED_STOPPED
                elif len(p.seq.output_token_ids) >= p.seq.sampling_params.max_tokens:
                    p.seq.status = SequenceStatus.FINISHED_LENGTH
        sched.free_finished()

    ahead = None
    for _ in range(5000):
        if not pending and not sched.has_unfinished():
            break
        for _ in range(rng.choice([0, 0, 1, 2])):
            if pending:
                sched.add_seq(pending.pop(0))
        live = sched.running + sched.waiting
        if live and rng.random() < 0.04:
            sched.abort(rng.choice(live).seq_id)
        if not sched.has_unfinished():
            continue
        if ahead is not None and ahead.version == sched.version:
            out = ahead
            sched.commit_ahead(out)
        else:
            out = sched.schedule()
            if not out.portions and not out.preempted and cache is not None and cache.evict(manager.num_blocks) > 0:
                out = sched.schedule()
            assert out.portions or out.preempted, "nothing runs although requests wait and the prefix cache is empty"
        for p in out.portions:
            held = len(manager.block_table(p.seq.seq_id, 0)) * BS
            assert held >= p.start + p.num_tokens, f"{p.seq.seq_id} runs tokens that no page backs"
        ahead = sched.schedule_ahead(out) if out.portions and rng.random() < 0.8 else None
        run(out)
        manager.audit()
    assert not pending and not sched.has_unfinished(), "the session does not end"
    assert all(s.is_finished() for s in seqs)
    if cache is not None:
        cache.reset()
    manager.audit()
    assert manager.min_free_blocks() == manager.num_blocks
