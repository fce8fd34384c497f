"""The scheduler's decisions, driven by a stand-in runtime that feeds back a constant token
(the reference's tests/unit/test_scheduler.py:37-58 pattern), invariants checked every step."""

from __future__ import annotations

import random

import pytest

from turboserve_amd.cache.manager import CacheManager
from turboserve_amd.config.engine_config import SchedulerConfig
from turboserve_amd.engine.scheduler import Scheduler
from turboserve_amd.engine.sequence import SeqStatus
from turboserve_amd.sampling.params import FinishReason, SamplingParams

NEXT_TOKEN = 7


def make(num_blocks=64, block_size=4, budget=16, seqs=4, chunked=True, windows=(None,)):
    config = SchedulerConfig(max_num_seqs=seqs, max_num_batched_tokens=budget, block_size=block_size,
                             num_blocks=num_blocks, enable_chunked_prefill=chunked)
    return Scheduler(config, CacheManager(list(windows), num_blocks, block_size, seqs))


def run_step(scheduler, out, eos=frozenset()):
    for item in out.sampled():
        scheduler.append_token(item.seq, NEXT_TOKEN, eos_token_ids=eos)


def drive(scheduler, max_steps=2000):
    steps = []
    for _ in range(max_steps):
        if not scheduler.has_unfinished():
            return steps
        out = scheduler.schedule()
        scheduler.check_invariants()
        steps.append(out)
        run_step(scheduler, out)
    raise AssertionError("the workload did not finish")


def test_budgets_hold_over_a_random_workload():
    """tests/unit/test_scheduler.py:64-77."""
    rng = random.Random(20260916)
    scheduler = make(num_blocks=40, budget=16, seqs=4)
    for i in range(30):
        scheduler.add_request(f"r{i}", [rng.randrange(100) for _ in range(rng.randrange(1, 40))],
                              SamplingParams(max_tokens=rng.randrange(1, 12)))
    for out in drive(scheduler):
        assert out.num_tokens <= 16 and len(out.scheduled) <= 4
        assert len({item.seq.seq_id for item in out.scheduled}) == len(out.scheduled)  # one entry per request
        kinds = [item.is_prefill for item in out.scheduled]
        assert kinds == sorted(kinds, reverse=True)  # portions of prompts first, then decodes
    assert scheduler.stats()["num_finished"] == 30
    assert all(pool.num_in_use == 0 for pool in scheduler.cache.pools)


def test_a_prompt_is_cut_under_the_token_budget():
    """tests/unit/test_scheduler.py:80-102: 20 tokens at a budget of 8 -> 8, 8, 4."""
    scheduler = make(budget=8)
    seq = scheduler.add_request("a", list(range(20)), SamplingParams(max_tokens=2))
    sizes, chunk_flags = [], []
    for _ in range(3):
        out = scheduler.schedule()
        sizes.append(out.scheduled[0].num_new_tokens)
        chunk_flags.append(out.scheduled[0].is_chunk)
        assert out.scheduled[0].start == sum(sizes[:-1])
        run_step(scheduler, out)
    assert sizes == [8, 8, 4] and chunk_flags == [True, True, False]
    assert seq.num_output_tokens == 1 and seq.num_computed_tokens == 20
    out = scheduler.schedule()
    assert [(i.num_new_tokens, i.is_prefill, i.start) for i in out.scheduled] == [(1, False, 20)]


def test_chunking_off_and_rejections():
    """tests/unit/test_scheduler.py:105-128."""
    scheduler = make(budget=8, chunked=False)
    with pytest.raises(ValueError, match="chunked prefill is off"):
        scheduler.add_request("long", list(range(9)))
    scheduler.add_request("a", list(range(6)), SamplingParams(max_tokens=1))
    scheduler.add_request("b", list(range(6)), SamplingParams(max_tokens=1))
    out = scheduler.schedule()
    assert [i.seq.request_id for i in out.scheduled] == ["a"]  # b does not fit whole and may not be cut
    with pytest.raises(ValueError, match="already in flight"):
        scheduler.add_request("a", [1])
    with pytest.raises(ValueError, match="empty prompt"):
        scheduler.add_request("e", [])
    small = make(num_blocks=2, block_size=4)
    with pytest.raises(ValueError, match="cache pages"):
        small.add_request("big", list(range(9)))


def test_prefills_come_before_decodes_and_rows_match():
    """tests/unit/test_scheduler.py:134-159."""
    scheduler = make(budget=32, seqs=8)
    first = scheduler.add_request("a", list(range(6)), SamplingParams(max_tokens=4))
    run_step(scheduler, scheduler.schedule())
    scheduler.add_request("b", list(range(100, 109)), SamplingParams(max_tokens=4))
    out = scheduler.schedule()
    assert [i.seq.request_id for i in out.scheduled] == ["b", "a"]
    assert (out.num_prefill_seqs, out.num_decode_seqs, out.num_prefill_tokens, out.num_decode_tokens) == (1, 1, 9, 1)
    assert [i.context_len for i in out.scheduled] == [9, 7]
    entries = out.entries()
    assert [list(e.tokens) for e in entries] == [list(range(100, 109)), [NEXT_TOKEN]]
    assert [e.start for e in entries] == [0, 6] and [list(e.want) for e in entries] == [[8], [0]]
    assert out.sample_indices() == [8, 9]
    assert [i.seq for i in out.sampled()] == [out.scheduled[0].seq, first]
    assert entries[1].slots == [[first_slot] for first_slot in [scheduler.cache.get(first.seq_id).tables[0][1] * 4 + 2]]


def test_scheduling_is_deterministic():
    """tests/unit/test_scheduler.py:193-208."""
    def trace():
        rng = random.Random(5)
        scheduler = make(num_blocks=12, budget=12, seqs=3)
        for i in range(10):
            scheduler.add_request(f"r{i}", [rng.randrange(50) for _ in range(rng.randrange(1, 20))], SamplingParams(max_tokens=6))
        return [[(i.seq.request_id, i.start, i.num_new_tokens, tuple(i.slots[0])) for i in out.scheduled] for out in drive(scheduler)]

    assert trace() == trace()


def test_running_out_of_pages_preempts_and_everybody_still_finishes():
    """tests/unit/test_scheduler.py:214-248: 3 requests of 8 + 10 tokens on 6 pages of 4."""
    scheduler = make(num_blocks=6, block_size=4, budget=64, seqs=8)
    seqs = [scheduler.add_request(f"r{i}", list(range(i * 50, i * 50 + 8)), SamplingParams(max_tokens=10)) for i in range(3)]
    preempted_any = False
    for _ in range(500):
        if not scheduler.has_unfinished():
            break
        out = scheduler.schedule()
        scheduler.check_invariants()
        for seq in out.preempted:
            preempted_any = True
            assert seq.status is SeqStatus.PREEMPTED and seq.num_computed_tokens == 0
            assert not scheduler.cache.has(seq.seq_id)
        for item in out.scheduled:
            if item.start == 0 and item.seq.num_preemptions:
                # re-run as one long prompt: what it had produced is kept and recomputed
                assert item.num_new_tokens == item.seq.num_tokens and item.samples
                assert item.token_ids[8:] == [NEXT_TOKEN] * item.seq.num_output_tokens
        run_step(scheduler, out)
    assert preempted_any and all(s.is_finished and s.num_output_tokens == 10 for s in seqs)
    assert all(s.finish_reason is FinishReason.LENGTH for s in seqs)
    assert scheduler.stats()["num_preemptions"] >= 1 and scheduler.cache.pools[0].num_in_use == 0


def test_the_victim_is_the_lowest_priority_most_recent_request():
    """tests/unit/test_scheduler.py:251-270."""
    scheduler = make(num_blocks=4, block_size=4, budget=64, seqs=8)
    high = scheduler.add_request("high", list(range(4)), SamplingParams(max_tokens=8), priority=5)
    low = scheduler.add_request("low", list(range(100, 104)), SamplingParams(max_tokens=8))
    scheduler.add_request("late", list(range(200, 204)), SamplingParams(max_tokens=8))
    run_step(scheduler, scheduler.schedule())
    victims = []
    for _ in range(6):
        out = scheduler.schedule()
        victims.extend(seq.request_id for seq in out.preempted)
        run_step(scheduler, out)
        if victims:
            break
    assert victims and victims[0] == "late"
    assert high.status is not SeqStatus.PREEMPTED and low.num_preemptions == 0


def test_a_request_that_outgrows_the_pool_is_ended_not_starved():
    """Decided here (the reference would wait forever): alone and still too large -> ``length``."""
    scheduler = make(num_blocks=3, block_size=4, budget=64, seqs=2)
    seq = scheduler.add_request("grows", list(range(8)), SamplingParams(max_tokens=100))
    dropped = []
    for out in drive(scheduler, max_steps=200):
        dropped.extend(out.dropped)
    assert dropped == [seq] and seq.finish_reason is FinishReason.LENGTH
    assert seq.num_output_tokens == 5  # 12 tokens fit three pages; the 13th has no page
    assert scheduler.cache.pools[0].num_in_use == 0


def test_stops_abort_and_head_of_line():
    """tests/unit/test_scheduler.py:322-348."""
    scheduler = make()
    a = scheduler.add_request("a", [1, 2, 3], SamplingParams(max_tokens=10, stop_token_ids=[NEXT_TOKEN]))
    b = scheduler.add_request("b", [1, 2, 3], SamplingParams(max_tokens=10))
    c = scheduler.add_request("c", [1, 2, 3], SamplingParams(max_tokens=10, ignore_eos=True))
    run_step(scheduler, scheduler.schedule(), eos=frozenset({NEXT_TOKEN}))
    assert a.finish_reason is FinishReason.STOP and a.output_token_ids == [NEXT_TOKEN] and a.stop_token_id == NEXT_TOKEN
    assert b.finish_reason is FinishReason.STOP and not c.is_finished  # end of sequence, unless ignored
    assert scheduler.cache.pools[0].num_in_use == 1
    assert scheduler.abort("c") and c.finish_reason is FinishReason.ABORT and not scheduler.abort("c")
    assert scheduler.cache.pools[0].num_in_use == 0 and not scheduler.has_unfinished()
    waiting = scheduler.add_request("w", [1])
    assert scheduler.abort("w") and waiting.status is SeqStatus.FINISHED
    # Head of line: a request that cannot be funded blocks the ones behind it.
    tight = make(num_blocks=4, block_size=4, budget=64, seqs=8)
    tight.add_request("x", list(range(12)), SamplingParams(max_tokens=1))
    tight.add_request("big", list(range(8)), SamplingParams(max_tokens=1))
    tight.add_request("small", [1], SamplingParams(max_tokens=1))
    out = tight.schedule()
    assert [i.seq.request_id for i in out.scheduled] == ["x"]


def test_window_groups_let_long_requests_run_on_few_pages():
    scheduler = make(num_blocks=8, block_size=4, budget=8, seqs=2, windows=(8,))
    seq = scheduler.add_request("long", list(range(50)), SamplingParams(max_tokens=30))
    drive(scheduler)
    assert seq.is_finished and seq.num_output_tokens == 30 and scheduler.stats()["num_preemptions"] == 0
