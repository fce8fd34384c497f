"""The engine's loop on the host, with a stand-in model whose next token is a known function of
the last token and its position: the tokens every request gets must be the same with and
without ``run_ahead`` (a decode step launched before the step before it has been read), through
stop tokens, ``max_tokens``, arrivals in the middle, preemption and aborts."""

from __future__ import annotations

import random

import pytest
import torch

from turboserve_amd.cache.manager import CacheManager
from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
from turboserve_amd.engine.llm_engine import LLMEngine
from turboserve_amd.engine.scheduler import Scheduler
from turboserve_amd.sampling.params import SamplingParams
from turboserve_amd.sampling.sampler import PendingSample

VOCAB = 97


def next_token(last: int, position: int) -> int:
    """The stand-in model: the token that follows ``last`` at ``position``."""
    return (last * 7 + position * 3 + 1) % VOCAB


def continuation(prompt: list[int], params: SamplingParams) -> list[int]:
    tokens, out = list(prompt), []
    while len(out) < params.max_tokens:
        token = next_token(tokens[-1], len(tokens) - 1)
        tokens.append(token)
        out.append(token)
        if token in params.stop_token_ids:
            break
    return out


class ToyRunner:
    """Logits that put all weight on ``next_token`` of each wanted place; a single token may
    come from a tensor the step before left (``tokens_from``), as on the device."""

    vocab_size = VOCAB

    def __init__(self, max_ahead_batch: int = 64) -> None:
        self.steps = 0
        self.steps_ahead = 0
        self.max_ahead_batch = max_ahead_batch

    def takes_tokens_from(self, num_entries: int) -> bool:
        return 0 < num_entries <= self.max_ahead_batch

    def step(self, entries, *, fresh_state_slots=(), tokens_from=None):
        self.steps += 1
        self.steps_ahead += tokens_from is not None
        rows = []
        for index, entry in enumerate(entries):
            tokens = list(entry.tokens)
            if tokens_from is not None and index in tokens_from[1]:
                assert tokens == [-1], "a token that is still on the device stands as -1 in the entry"
                tokens = [int(tokens_from[0][tokens_from[1][index]])]
            assert all(0 <= t < VOCAB for t in tokens), tokens
            for place in entry.want:
                row = torch.zeros(VOCAB)
                row[next_token(tokens[place], entry.start + place)] = 1.0
                rows.append(row)
        return torch.stack(rows) if rows else torch.zeros((0, VOCAB))

    def release(self) -> None:
        pass


class ToySampler:
    def launch_sequences(self, logits, sequences):
        return PendingSample(logits.argmax(dim=1).to(torch.int32), None, [seq.sampling for seq in sequences])


def make_engine(run_ahead: bool, *, num_blocks: int = 64, max_num_seqs: int = 8, budget: int = 32, page: int = 4,
                sampler=None):
    cfg = SchedulerConfig(max_num_seqs=max_num_seqs, max_num_batched_tokens=budget, block_size=page, num_blocks=num_blocks)
    scheduler = Scheduler(cfg, CacheManager([None], num_blocks, page, max_num_seqs))
    runner = ToyRunner()
    engine = LLMEngine(EngineConfig(model="/nonexistent", scheduler=cfg, run_ahead=run_ahead), model=object(),
                       scheduler=scheduler, runner=runner, sampler=sampler or ToySampler())
    return engine, runner


def drive(engine, arrivals, *, abort_at=None):
    """``arrivals``: step number -> list of (request id, prompt, params).  Returns the tokens and
    finish reason of every request."""
    got: dict[str, list[int]] = {}
    reasons: dict[str, str] = {}
    step = 0
    while arrivals or engine.has_unfinished():
        for request_id, prompt, params in arrivals.pop(step, []):
            engine.add_request(request_id, prompt, params)
            got[request_id] = []
        if abort_at is not None and step == abort_at[0]:
            engine.abort(abort_at[1])
        for output in engine.step():
            got.setdefault(output.request_id, []).extend(output.new_token_ids)
            if output.finished:
                reasons[output.request_id] = output.finish_reason.value
        step += 1
        assert step < 2000, "no progress"
    engine.scheduler.check_invariants()
    assert all(pool.num_in_use == 0 for pool in engine.scheduler.cache.pools)
    return got, reasons


def workload(seed: int, count: int, *, stops: bool = True):
    rng = random.Random(seed)
    arrivals: dict[int, list] = {}
    expected = {}
    for index in range(count):
        prompt = [rng.randrange(VOCAB) for _ in range(rng.randint(1, 20))]
        params = SamplingParams(max_tokens=rng.randint(1, 30), temperature=0.0, ignore_eos=True)
        plain = continuation(prompt, params)
        if stops and len(plain) > 4 and rng.random() < 0.5:
            params = SamplingParams(max_tokens=params.max_tokens, temperature=0.0, ignore_eos=True,
                                    stop_token_ids=(plain[rng.randint(2, len(plain) - 1)],))
        expected[f"r{index}"] = continuation(prompt, params)
        arrivals.setdefault(rng.choice([0, 0, 0, 3, 9, 17]), []).append((f"r{index}", prompt, params))
    return arrivals, expected


@pytest.mark.parametrize("seed", range(6))
def test_run_ahead_gives_the_same_tokens(seed):
    arrivals, expected = workload(seed, 7)
    plain_got, plain_reasons = drive(make_engine(False)[0], {k: list(v) for k, v in arrivals.items()})
    engine, runner = make_engine(True)
    got, reasons = drive(engine, arrivals)
    assert plain_got == expected
    assert got == expected and reasons == plain_reasons
    assert runner.steps_ahead > 0  # it did run ahead


def test_run_ahead_with_preemption_and_an_abort():
    """Short prompts that grow past the pool, so that running requests are preempted and
    recomputed while steps are launched ahead; one request is aborted while a step that holds
    it is in flight."""
    preemptions = 0
    for seed in range(4):
        rng = random.Random(200 + seed)
        arrivals, expected = {0: []}, {}
        for index in range(5):
            prompt = [rng.randrange(VOCAB) for _ in range(rng.randint(1, 3))]
            params = SamplingParams(max_tokens=rng.randint(20, 30), temperature=0.0, ignore_eos=True)
            if seed % 2 == 0:
                params = SamplingParams(max_tokens=params.max_tokens, temperature=0.0, ignore_eos=True,
                                        stop_token_ids=(continuation(prompt, params)[rng.randint(10, 19)],))
            expected[f"r{index}"] = continuation(prompt, params)
            arrivals[0].append((f"r{index}", prompt, params))
        engine, runner = make_engine(True, num_blocks=14, max_num_seqs=6)
        for request_id, prompt, params in arrivals.pop(0):
            sequence = engine.add_request(request_id, prompt, params)
            if request_id == "r2":
                aborted = sequence
        got, reasons = drive(engine, arrivals, abort_at=(6, "r2"))
        preemptions += engine.scheduler.stats()["num_preemptions"]
        assert runner.steps_ahead > 0
        for request_id, tokens in expected.items():
            if request_id == "r2":
                assert "r2" not in reasons and got[request_id] == tokens[: len(got[request_id])]  # aborted on the way
                assert aborted.output_token_ids == got[request_id]  # no place of an unread token is left behind
            else:
                assert got[request_id] == tokens, (seed, request_id)
    assert preemptions > 0


def test_a_step_is_not_launched_ahead_of_a_request_that_ends_by_length_or_has_a_penalty():
    engine, runner = make_engine(True)
    engine.add_request("a", [5, 6, 7], SamplingParams(max_tokens=2, temperature=0.0, ignore_eos=True))
    outputs = []
    while engine.has_unfinished():
        outputs.extend(engine.step())
    assert [t for o in outputs for t in o.new_token_ids] == continuation([5, 6, 7], SamplingParams(max_tokens=2))
    # the second step is launched ahead of the first's token; nothing is launched ahead of the
    # second's, which is the request's last
    assert runner.steps == 2 and runner.steps_ahead == 1
    engine, runner = make_engine(True)
    engine.add_request("b", [5, 6, 7], SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True, repetition_penalty=1.2))
    while engine.has_unfinished():
        engine.step()
    assert runner.steps == 6 and runner.steps_ahead == 0  # the penalty needs the tokens on the host

    class UnreadSampler(ToySampler):
        """A sampler that can be given the token the host has not read (as the real one can)."""

        takes_unread = True

        def __init__(self):
            self.seen = []

        def launch_sequences(self, logits, sequences, unread=None):
            if unread is not None:
                tokens, places = unread
                assert len(places) == len(sequences)
                assert all(seq.output_token_ids[-1] == seq.UNREAD_TOKEN for seq in sequences)
                self.seen.append([int(tokens[place]) for place in places])
            return super().launch_sequences(logits, sequences)

    sampler = UnreadSampler()
    engine, runner = make_engine(True, sampler=sampler)
    params = SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True, repetition_penalty=1.2)
    engine.add_request("b", [5, 6, 7], params)
    engine.add_request("d", [9, 3], params)
    outputs = []
    while engine.has_unfinished():
        outputs.extend(engine.step())
    assert runner.steps_ahead == 5  # with such a sampler a penalty does not keep a step from being launched ahead
    tokens = {rid: [t for o in outputs if o.request_id == rid for t in o.new_token_ids] for rid in ("b", "d")}
    assert tokens["b"] == continuation([5, 6, 7], params) and tokens["d"] == continuation([9, 3], params)
    # every launch ahead named, for each request, that request's own token of the launch before
    assert sampler.seen == [[tokens["b"][i], tokens["d"][i]] for i in range(5)]
    engine, runner = make_engine(True)
    engine.add_request("c", [5, 6, 7], SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))
    while engine.has_unfinished():
        engine.step()
    assert runner.steps == 6 and runner.steps_ahead == 5  # no step is wasted when requests end by length
    # a stop token costs one step whose result is dropped
    stop = continuation([5, 6, 7], SamplingParams(max_tokens=6))[2]
    engine, runner = make_engine(True)
    engine.add_request("d", [5, 6, 7], SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True, stop_token_ids=(stop,)))
    tokens = []
    while engine.has_unfinished():
        tokens.extend(t for o in engine.step() for t in o.new_token_ids)
    expected = continuation([5, 6, 7], SamplingParams(max_tokens=6, stop_token_ids=(stop,)))
    assert tokens == expected and tokens[-1] == stop and len(tokens) < 6 and runner.steps == len(tokens) + 1
    assert engine.step() == [] and engine.step() == []  # the dropped step is read and forgotten


def test_requests_that_end_at_different_lengths_do_not_stop_the_running_ahead():
    """A request whose token in flight is its last takes no part in the step launched ahead;
    the others go on.  A request that ended on a stop token leaves a dropped row and the others
    go on all the same."""
    engine, runner = make_engine(True)
    lengths = {"a": 3, "b": 9, "c": 6}
    for name, length in lengths.items():
        engine.add_request(name, [1, 2, ord(name) % VOCAB], SamplingParams(max_tokens=length, temperature=0.0, ignore_eos=True))
    got = {name: [] for name in lengths}
    while engine.has_unfinished():
        for output in engine.step():
            got[output.request_id].extend(output.new_token_ids)
    for name, length in lengths.items():
        assert got[name] == continuation([1, 2, ord(name) % VOCAB], SamplingParams(max_tokens=length))
    assert runner.steps == 9 and runner.steps_ahead == 8  # every step but the first
    stop = continuation([1, 2, 3], SamplingParams(max_tokens=9))[3]
    engine, runner = make_engine(True)
    engine.add_request("s", [1, 2, 3], SamplingParams(max_tokens=9, temperature=0.0, ignore_eos=True, stop_token_ids=(stop,)))
    engine.add_request("t", [4, 5, 6], SamplingParams(max_tokens=9, temperature=0.0, ignore_eos=True))
    got = {"s": [], "t": []}
    while engine.has_unfinished():
        for output in engine.step():
            got[output.request_id].extend(output.new_token_ids)
    assert got["s"] == continuation([1, 2, 3], SamplingParams(max_tokens=9, stop_token_ids=(stop,))) and len(got["s"]) < 9
    assert got["t"] == continuation([4, 5, 6], SamplingParams(max_tokens=9))
    assert runner.steps == 9 and runner.steps_ahead == 8


class LetterTokenizer:
    """Token i decodes to the letter chr(ord('a') + i % 26)."""

    def decode(self, ids, skip_special_tokens=True):
        return "".join(chr(ord("a") + i % 26) for i in ids)

    def encode(self, text, add_special_tokens=False):
        return [ord(c) - ord("a") for c in text]


def test_a_stop_string_ends_a_request_at_the_same_place_when_steps_run_ahead():
    prompt = [3, 1, 4]
    plain = continuation(prompt, SamplingParams(max_tokens=12))
    text = LetterTokenizer().decode(plain)
    stop = text[4:6]  # the request must end before these two letters
    results = []
    for ahead in (False, True):
        cfg = SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=32, block_size=4, num_blocks=32)
        runner = ToyRunner()
        engine = LLMEngine(EngineConfig(model="/nonexistent", scheduler=cfg, run_ahead=ahead), model=object(),
                           tokenizer=LetterTokenizer(), scheduler=Scheduler(cfg, CacheManager([None], 32, 4, 4)),
                           runner=runner, sampler=ToySampler())
        outputs = engine.generate([prompt, [2, 7, 1]], [SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True, stop=[stop]),
                                                        SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True)])
        results.append([(o.new_token_ids, o.text_delta, o.finish_reason) for o in outputs])
        assert outputs[0].finish_reason == "stop" and outputs[0].text_delta == text[: text.index(stop)]
        assert outputs[1].new_token_ids == continuation([2, 7, 1], SamplingParams(max_tokens=12))
        assert (runner.steps_ahead > 0) == ahead
    assert results[0] == results[1]
