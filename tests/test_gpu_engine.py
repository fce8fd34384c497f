"""The engine's entry point on the GPU: greedy generation equals the plain implementation,
whatever the token budget and however few pages there are; sampling follows the stated rule."""

from __future__ import annotations

import itertools

import pytest
import torch

import tiny
from plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu


def make_engine(folder, dtype, page, *, num_blocks, budget=2048, max_num_seqs=8, seed=None, run_ahead=False):
    from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
    from turboserve_amd.engine.llm_engine import LLMEngine

    return LLMEngine(EngineConfig(
        model=str(folder), dtype=dtype, seed=seed, run_ahead=run_ahead,
        scheduler=SchedulerConfig(max_num_seqs=max_num_seqs, max_num_batched_tokens=budget, block_size=page,
                                  num_blocks=num_blocks),
    ))


@pytest.fixture(scope="module", params=["A", "B", "C", "D"])
def model(request, tmp_path_factory):
    config, seed, page = tiny.TINY[request.param]
    folder = tiny.make_model_dir(tmp_path_factory.mktemp(f"engine{request.param}"), config, seed, torch.float32)
    raw, tensors = tiny.read_model_dir(folder)
    lengths = {"A": [5, 17, 33], "B": [1, 9, 24, 40], "C": [20, 50, 97], "D": [2, 31, 52, 20]}[request.param]
    prompts = [tiny.random_tokens(config["vocab_size"], n, 50 + n) for n in lengths]
    # The same architecture with a wider spread of weights, for the 32-bit token-for-token tests:
    # its greedy continuations do not settle on one token, so every step's logits matter.
    wide = tiny.make_model_dir(tmp_path_factory.mktemp(f"engine{request.param}_wide"), config, seed + 1, torch.float32,
                               std=tiny.WIDE_STD)
    wide_raw, wide_tensors = tiny.read_model_dir(wide)
    # And one stored in bfloat16 (a spread that keeps the rounding error inside the bounds), so
    # that the plain implementation computes with the very numbers the bfloat16 engine holds.
    half = tiny.make_model_dir(tmp_path_factory.mktemp(f"engine{request.param}_bf16"), config, seed + 2, torch.bfloat16,
                               std=tiny.std_for(torch.bfloat16, config["hidden_size"]))
    half_raw, half_tensors = tiny.read_model_dir(half)
    return {"name": request.param, "folder": folder, "page": page, "raw": raw, "tensors": tensors, "prompts": prompts,
            "vocab": config["vocab_size"], "wide_folder": wide, "wide_raw": wide_raw, "wide_tensors": wide_tensors,
            "bf16_folder": half, "bf16_raw": half_raw, "bf16_tensors": half_tensors}


def check_logprobs(logits: torch.Tensor, output) -> None:
    """A bfloat16 engine's greedy tokens and their log-probabilities against the plain
    implementation's 32-bit logits for the same sequence (``logits[i]``: the row that chose token
    ``i``): each token is the argmax up to the rounding bound of the logits (2% of the row's
    largest, see ``test_gpu_replay``), and its log-probability, a difference of two such
    numbers, is off by at most twice that."""
    assert len(output.new_token_ids) == len(output.logprobs) > 0
    for row, token, got in zip(logits, output.new_token_ids, output.logprobs):
        bound = 2e-2 * float(row.abs().max())
        assert float(row.max() - row[token]) <= bound, f"token {token} is not a near-argmax"
        assert abs(got - plain.log_softmax_at(row, token)) <= 2 * bound, (token, got, plain.log_softmax_at(row, token))


def test_greedy_generation_equals_plain(model):
    """Mixed-length prompts in one continuous batch, token for token
    (tests/unit/test_engine_e2e.py:103-116 in the reference)."""
    from turboserve_amd.sampling.params import SamplingParams

    new = 8 if model["name"] == "A" else 12
    want = [plain.greedy_generate(model["wide_raw"], model["wide_tensors"], p, new) for p in model["prompts"]]
    assert all(len(set(tokens)) > 2 for tokens in want), "the continuations should not repeat one token"
    for budget, blocks in ((2048, 64), (max(16, model["page"]), 64), (7 if model["page"] <= 7 else model["page"], 64)):
        with make_engine(model["wide_folder"], "float32", model["page"], num_blocks=blocks, budget=budget) as engine:
            outputs = engine.generate(model["prompts"], SamplingParams(max_tokens=new, temperature=0.0, ignore_eos=True))
            assert [o.new_token_ids for o in outputs] == want, f"budget {budget}"
            assert all(o.finish_reason == "length" and o.output_tokens == new for o in outputs)
            engine.scheduler.check_invariants()
            assert all(pool.num_in_use == 0 for pool in engine.scheduler.cache.pools)


def test_preemption_keeps_the_tokens(model):
    """So few pages that running requests are preempted and recomputed: same tokens
    (tests/unit/test_engine_e2e.py:149-165)."""
    from turboserve_amd.sampling.params import SamplingParams

    new = 20
    want = [plain.greedy_generate(model["wide_raw"], model["wide_tensors"], p, new) for p in model["prompts"]]
    longest = max(len(p) for p in model["prompts"]) + new
    blocks = -(-longest // model["page"])  # the longest request just fits alone; together they do not
    with make_engine(model["wide_folder"], "float32", model["page"], num_blocks=blocks, budget=64) as engine:
        outputs = engine.generate(model["prompts"], SamplingParams(max_tokens=new, temperature=0.0, ignore_eos=True))
        assert [o.new_token_ids for o in outputs] == want
        assert engine.stats()["num_preemptions"] > 0
        engine.scheduler.check_invariants()
        # the structured snapshot of the reference (engine.py:80-115), merged into the flat one
        snapshot = engine.engine_stats()
        assert snapshot.num_finished == len(model["prompts"]) and snapshot.num_unfinished == 0
        assert snapshot.num_generated_tokens == new * len(model["prompts"])
        assert snapshot.kv_utilization == 0.0 and snapshot.prefix_hit_rate == 0.0
        assert engine.stats()["num_generated_tokens"] == snapshot.num_generated_tokens
        assert str(engine.device) == "cuda:0" and engine.dtype == torch.float32


def test_temperature_sampling_follows_the_rule(model):
    """Seeded temperature sampling: each token is the first whose cumulative probability
    (plain implementation, 64-bit) exceeds the request's Philox uniform for that draw."""
    from turboserve_amd.sampling.params import SamplingParams

    new = 12
    params = [SamplingParams(max_tokens=new, temperature=0.8, seed=1000 + i, ignore_eos=True, logprobs=True)
              for i in range(len(model["prompts"]))]
    with make_engine(model["folder"], "float32", model["page"], num_blocks=64, budget=7 if model["page"] <= 7 else max(16, model["page"])) as engine:
        outputs = engine.generate(model["prompts"], params)
    for i, (prompt, output) in enumerate(zip(model["prompts"], outputs)):
        tokens = list(prompt)
        assert len(output.new_token_ids) == new
        for draw, token in enumerate(output.new_token_ids):
            logits = plain.forward_logits(model["raw"], model["tensors"], tokens)[-1]
            _, cdf = plain.sample_token(logits, temperature=0.8, seed=1000 + i, draw_index=draw)
            u = plain.philox_uniform(1000 + i, draw)
            low = float(cdf[token - 1]) if token > 0 else 0.0
            assert low - 1e-5 <= u <= float(cdf[token]) + 1e-5, f"request {i} draw {draw}: token {token}"
            assert abs(output.logprobs[draw] - plain.log_softmax_at(logits, token)) < 1e-4
            tokens.append(token)


def test_seeded_request_does_not_depend_on_its_neighbours(model):
    """A seeded request alone and in a batch draws the same tokens (tests/unit/test_sampler.py:131-149)."""
    from turboserve_amd.sampling.params import SamplingParams

    params = SamplingParams(max_tokens=6, temperature=1.0, seed=77, ignore_eos=True)
    with make_engine(model["folder"], "float32", model["page"], num_blocks=64) as engine:
        alone = engine.generate([model["prompts"][-1]], params)[0].new_token_ids
    with make_engine(model["folder"], "float32", model["page"], num_blocks=64, seed=5) as engine:
        others = SamplingParams(max_tokens=6, temperature=1.0, ignore_eos=True)
        batch = engine.generate([*model["prompts"][:-1], model["prompts"][-1]],
                                [*[others] * (len(model["prompts"]) - 1), params])
    assert batch[-1].new_token_ids == alone


def test_stop_ids_and_length(model):
    """A stop id ends the request and stays in the output (tests/unit/test_engine_e2e.py:296-313)."""
    from turboserve_amd.sampling.params import SamplingParams

    prompt = model["prompts"][1]
    free = plain.greedy_generate(model["raw"], model["tensors"], prompt, 6)
    with make_engine(model["folder"], "float32", model["page"], num_blocks=64) as engine:
        out = engine.generate([prompt], SamplingParams(max_tokens=6, temperature=0.0, stop_token_ids=[free[2]]))[0]
    cut = free.index(free[2]) + 1
    assert out.new_token_ids == free[:cut] and out.finish_reason == "stop"


def test_too_large_prompt_is_refused(model):
    with make_engine(model["folder"], "float32", model["page"], num_blocks=2) as engine:
        with pytest.raises(ValueError, match="cache pages"):
            engine.add_request("big", tiny.random_tokens(model["vocab"], 5 * model["page"], 1))


def test_smoke_entry_point():
    import __graft_entry__

    __graft_entry__.smoke()


def test_decode_graphs_replay_like_eager(model):
    """Steps of single tokens are replayed as HIP graphs.  Every replay must equal the eager
    step: several replays of one graph with different data, eager work and synchronisation
    between them, batch sizes that are padded (3 -> 4) and exact, a request leaving the batch."""
    import json
    from pathlib import Path

    import trace_helpers as th
    from turboserve_amd.engine.replay import TraceReplayer

    config = json.loads((Path(model["folder"]) / "config.json").read_text())
    requests = {f"g{i}": tiny.random_tokens(config["vocab_size"], n, 900 + i) for i, n in enumerate([37, 21, 30])}
    steps = []
    for rid, tokens in requests.items():  # prompts whole, except the last 12 tokens
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": tokens[:-12], "want": []}], "end": []})
    for k in range(12):  # then all three decode together; g1 leaves after 8 tokens
        entries = [{"id": rid, "tokens": [tokens[len(tokens) - 12 + k]], "want": [0]}
                   for rid, tokens in requests.items() if not (rid == "g1" and k >= 8)]
        steps.append({"step": len(steps), "entries": entries, "end": ["g1"] if k == 7 else []})
    results = {}
    for dtype in ("float32", "bfloat16"):
        for use_graphs in (False, True):
            replayer = TraceReplayer(model["folder"], dtype=dtype, max_tokens=256, page_size=model["page"])
            if not use_graphs:
                replayer.runner.graphs = None
            outs = []
            for record in steps:
                logits = replayer.run_step(record)
                if logits.shape[0]:
                    outs.append(logits.float().cpu())
                    torch.cuda.synchronize()
                    _ = (torch.ones(64, 64, device="cuda") @ torch.ones(64, 64, device="cuda")).sum().item()  # eager work between replays
            results[(dtype, use_graphs)] = outs
            if use_graphs:
                assert replayer.runner.graphs.num_replays == 12
        for eager, graph in zip(results[(dtype, False)], results[(dtype, True)]):
            assert torch.equal(eager, graph), f"{dtype}: a graph replay differs from the eager step"


def test_recorded_steps_survive_the_growth_of_the_rotary_tables(tmp_path):
    """A recorded step holds the addresses of the rotary tables it was recorded with.  The
    tables of this model start at 48 positions: a short request decodes (its step is recorded
    against tables of 96), a 1,500-token prompt makes the tables grow, memory of the old tables'
    size is then filled with NaN (so a freed table would be overwritten), and a second short
    request decodes through the step recorded first.  Its logits are the plain
    implementation's, and bit for bit those of a run without recorded steps."""
    from turboserve_amd.engine.replay import TraceReplayer

    config = {**tiny.CONFIG_A, "max_position_embeddings": 48}
    folder = tiny.make_model_dir(tmp_path / "m", config, 11, torch.float32, std=tiny.WIDE_STD)
    raw, tensors = tiny.read_model_dir(folder)
    requests = {"s1": tiny.random_tokens(256, 14, 1), "long": tiny.random_tokens(256, 1503, 2),
                "s2": tiny.random_tokens(256, 17, 3)}

    def decode_tail(rid, count, end):
        tokens = requests[rid]
        return [{"entries": [{"id": rid, "tokens": [tokens[len(tokens) - count + k]], "want": [0]}],
                 "end": [rid] if end and k == count - 1 else []} for k in range(count)]

    steps = [{"entries": [{"id": "s1", "tokens": requests["s1"][:-4], "want": list(range(10))}], "end": []},
             *decode_tail("s1", 4, True),
             {"entries": [{"id": "long", "tokens": requests["long"][:-3], "want": [1499]}], "end": []},
             {"entries": [{"id": "s2", "tokens": requests["s2"][:-5], "want": list(range(12))}], "end": []},
             *decode_tail("s2", 5, True),
             *decode_tail("long", 3, True)]
    for index, record in enumerate(steps):
        record["step"] = index
    expected = {rid: plain.forward_logits(raw, tensors, tokens) for rid, tokens in requests.items()}
    results = {}
    for use_graphs in (False, True):
        replayer = TraceReplayer(folder, dtype="float32", max_tokens=64 + 1536 + 64, page_size=16)
        rope = replayer.model.blocks[0].mixer.position
        if not use_graphs:
            replayer.runner.graphs = None
        outs, junk = {}, []
        for record in steps:
            outs[record["step"]] = replayer.run_step(record).float().cpu()
            if record["entries"][0]["id"] == "long" and len(record["entries"][0]["tokens"]) > 1:
                assert rope.capacity >= 1500
                junk = [torch.full((rows, 8), float("nan"), device="cuda") for rows in (48, 96) for _ in range(64)]
                torch.cuda.synchronize()
        if use_graphs:
            assert replayer.runner.graphs.num_replays == 12
            assert len(replayer.runner.graphs._graphs) == 2, "s1 and s2 replay one recorded step, `long` another"
            assert len(rope.superseded) >= 1, "the tables grew after a step had been recorded"
        del junk
        results[use_graphs] = outs
        for rid, first in (("s1", 0), ("s2", 0), ("long", 1499)):
            got = torch.cat([outs[s["step"]] for s in steps if s["entries"][0]["id"] == rid])
            worst = float((got - expected[rid][first:]).abs().max())
            assert worst <= 1e-4, f"graphs={use_graphs} request {rid}: {worst:.3e}"
    for step in results[False]:
        assert torch.equal(results[False][step], results[True][step]), f"step {step}: recorded differs from eager"


_TIMED_WIDTHS = itertools.count()


def test_timed_library_products_and_the_dry_step(model, tmp_path):
    """An engine asked to time the BLAS library's kernels at start-up: the choices are written
    to the given file, nothing is timed once the engine serves, products below the size worth
    timing keep the library's default kernel, and the dry step the timing runs in leaves every
    cache page as it was.  A prompt longer than the 128 rows the engine's own products take (so
    that the library computes its projections) gives the plain implementation's
    log-probabilities."""
    from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
    from turboserve_amd.engine.llm_engine import LLMEngine
    from turboserve_amd.kernels.ops import Ops
    from turboserve_amd.sampling.params import SamplingParams

    prompt = tiny.random_tokens(model["vocab"], 200, 77)

    def engine_with_tuning(results):
        return LLMEngine(EngineConfig(
            model=str(model["bf16_folder"]), dtype="bfloat16", tune_gemm_tokens=(200,), gemm_tuning_file=str(results),
            scheduler=SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=256, block_size=model["page"], num_blocks=64),
        ))

    # This model's products are all below the size worth timing: nothing is chosen, nothing written.
    untouched = tmp_path / "none.csv"
    engine = engine_with_tuning(untouched)
    try:
        assert torch.cuda.tunable.is_enabled() and not torch.cuda.tunable.tuning_is_enabled()
        assert not untouched.exists() or "Gemm" not in untouched.read_text()
        before = [t.clone() for t in engine.storage.tensors()]
        engine.runner.dry_run(150)
        assert all(torch.equal(a, b) for a, b in zip(before, engine.storage.tensors()))
        out = engine.generate([prompt], SamplingParams(max_tokens=4, temperature=0.0, ignore_eos=True, logprobs=True))[0]
    finally:
        engine.close()
        torch.cuda.tunable.enable(False)
    sequence = prompt + out.new_token_ids
    logits = plain.forward_logits(model["bf16_raw"], model["bf16_tensors"], sequence)
    check_logprobs(logits[len(prompt) - 1:], out)
    # A product of a size worth timing (and of a regular shape: the library's candidates for
    # small odd shapes are not all sound) is timed inside the block, its choice is written to the
    # file and stays in use afterwards.
    from turboserve_amd.kernels.gemm_tuning import LibraryGemmTuning

    ops = Ops("cuda:0")
    ops.wide_default_rows = 0  # the library's product is the one under test here
    g = torch.Generator().manual_seed(3)
    # A width of its own for every run of this test: a shape that was timed before in this process
    # is not timed again, and nothing would be written.
    width = 1024 + 128 * next(_TIMED_WIDTHS)
    x = torch.randn(256, 1024, generator=g).bfloat16().to("cuda:0")
    w = (torch.randn(width, 1024, generator=g) / 32).bfloat16().to("cuda:0")
    assert x.shape[0] * w.shape[0] * w.shape[1] >= Ops.library_tuning_min_work
    results = tmp_path / "choices.csv"
    try:
        with LibraryGemmTuning(str(results), max_ms_per_candidate=5, max_iterations=5):
            timed = ops.linear(x, w)
        assert results.exists() and "Gemm" in results.read_text()
        assert torch.cuda.tunable.is_enabled() and not torch.cuda.tunable.tuning_is_enabled()
        again = ops.linear(x, w)
    finally:
        torch.cuda.tunable.enable(False)
    want = x.float() @ w.float().t()
    for got in (timed, again):
        torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2 * float(want.abs().max()))


def test_own_product_against_the_librarys_is_timed_once_and_remembered(tmp_path):
    """A product of many rows that is worth timing runs both ways when asked to, the faster one
    is kept, both give the product, and the next process (another ``Ops``) adopts the choice
    from the file unless the file is of another state of the sources."""
    import json

    from turboserve_amd.kernels.gemm_tuning import OwnProductChoices
    from turboserve_amd.kernels.ops import Ops

    g = torch.Generator().manual_seed(5)
    x = torch.randn(300, 1024, generator=g).bfloat16().to("cuda:0")
    w = (torch.randn(1152, 1024, generator=g) / 32).bfloat16().to("cuda:0")
    bias = torch.randn(1152, generator=g).bfloat16().to("cuda:0")
    want = x.float() @ w.float().t() + bias.float()
    ops = Ops("cuda:0")
    ops.time_wide_choices = True
    first = ops.linear(x, w, bias)
    key = (300, 1152, 1024, "one")
    assert set(ops.wide_timings) == {key} and all(0 < t < 50 for t in ops.wide_timings[key])
    assert ops.wide_choices[key] == (ops.wide_timings[key][0] <= ops.wide_timings[key][1])
    timings = dict(ops.wide_timings)
    results = [first]
    for forced in (True, False):
        ops.wide_choices[key] = forced
        results.append(ops.linear(x, w, bias))
    assert ops.wide_timings == timings, "a known product is not timed again"
    for got in results:
        assert got.shape == want.shape and got.dtype == torch.bfloat16
        torch.testing.assert_close(got.float().cpu(), want.cpu(), rtol=2e-2, atol=2e-2 * float(want.abs().max()))
    ops.wide_choices[key] = timings[key][0] <= timings[key][1]
    kept = OwnProductChoices(str(tmp_path / "choices.csv"), ops)
    kept.save()
    other = Ops("cuda:0")
    assert OwnProductChoices(str(tmp_path / "choices.csv"), other).load() == 1
    assert other.wide_choices == ops.wide_choices and other.wide_timings == ops.wide_timings
    assert OwnProductChoices(str(tmp_path / "choices.csv"), other).load() == 0  # nothing new the second time
    data = json.loads((tmp_path / "choices.csv.own.json").read_text())
    data["stamp"]["source"] = "another state of the sources"
    (tmp_path / "choices.csv.own.json").write_text(json.dumps(data))
    assert OwnProductChoices(str(tmp_path / "choices.csv"), Ops("cuda:0")).load() == 0
    assert OwnProductChoices(str(tmp_path / "absent.csv"), Ops("cuda:0")).load() == 0


def test_library_products_at_timed_step_sizes(model, tmp_path, monkeypatch):
    """An engine told to run the library's products at a few timed sizes: prompts of lengths
    between the sizes, alone and cut into portions beside decoded tokens, give the plain
    implementation's log-probabilities, and their products did run at the sizes.  (The engine's
    own product for steps of many rows is switched off: the library's is the one under test.)"""
    from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
    from turboserve_amd.engine.llm_engine import LLMEngine
    from turboserve_amd.kernels.ops import Ops
    from turboserve_amd.sampling.params import SamplingParams

    monkeypatch.setattr(Ops, "wide_default_rows", 0)

    prompts = [tiny.random_tokens(model["vocab"], length, 900 + length) for length in (131, 203, 250, 390)]
    sampling = SamplingParams(max_tokens=5, temperature=0.0, ignore_eos=True, logprobs=True)
    engine = LLMEngine(EngineConfig(
        model=str(model["bf16_folder"]), dtype="bfloat16", tune_gemm_step_sizes=True, gemm_tuning_file=str(tmp_path / "choices.csv"),
        scheduler=SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=300, block_size=model["page"], num_blocks=96),
    ))
    lengths = []
    mm, addmm = torch.mm, torch.addmm
    try:
        ops = engine.model.runtime.ops
        assert ops.library_buckets == (32, 64, 96, 128, 160, 192, 224, 256, 300)
        torch.mm = lambda a, *rest, **kw: (lengths.append(a.shape[0]), mm(a, *rest, **kw))[1]
        torch.addmm = lambda c, a, *rest, **kw: (lengths.append(a.shape[0]), addmm(c, a, *rest, **kw))[1]
        outs = engine.generate(prompts[:1], sampling) + engine.generate(prompts[1:2], sampling)
        assert set(lengths) == {160, 224}, "131 and 203 tokens, each at the next size up"
        outs += engine.generate(prompts[2:], sampling)
    finally:
        torch.mm, torch.addmm = mm, addmm
        engine.close()
        torch.cuda.tunable.enable(False)
    assert set(lengths) <= {32, 64, 96, 128, 160, 192, 224, 256, 300}, sorted(set(lengths))
    assert ops.library_buckets == (), "a closed engine leaves the model's kernels as it found them"
    for prompt, out in zip(prompts, outs):
        sequence = prompt + out.new_token_ids
        logits = plain.forward_logits(model["bf16_raw"], model["bf16_tensors"], sequence)
        check_logprobs(logits[len(prompt) - 1:], out)


@pytest.mark.parametrize("count", [40, 100])
def test_many_requests_decode_together(model, count):
    """40 and 100 requests decoding in one batch (recorded steps of 64 and 128 rows, the tiled
    product at both of its heights) give the plain implementation's log-probabilities."""
    from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
    from turboserve_amd.engine.llm_engine import LLMEngine
    from turboserve_amd.sampling.params import SamplingParams

    prompts = [tiny.random_tokens(model["vocab"], 3 + i % 9, 300 + i) for i in range(count)]
    sampling = SamplingParams(max_tokens=4, temperature=0.0, ignore_eos=True, logprobs=True)
    engine = LLMEngine(EngineConfig(
        model=str(model["bf16_folder"]), dtype="bfloat16",
        scheduler=SchedulerConfig(max_num_seqs=128, max_num_batched_tokens=2048, block_size=model["page"], num_blocks=512),
    ))
    try:
        outs = engine.generate(prompts, sampling)
        assert engine.runner.graphs.num_replays >= 3
    finally:
        engine.close()
    for prompt, out in zip(prompts, outs):
        sequence = prompt + out.new_token_ids
        check_logprobs(plain.forward_logits(model["bf16_raw"], model["bf16_tensors"], sequence)[len(prompt) - 1:], out)


def test_steps_launched_ahead_give_the_same_tokens(model):
    """With `run_ahead` every decode step is launched before the tokens of the step before it
    have been read (they are copied on the device into the recorded step's input): greedy in
    32-bit gives the plain implementation's tokens, with plenty of pages and with so few that
    requests are preempted; seeded temperature sampling gives the tokens it gives without
    running ahead; a stop token ends its request at the same place."""
    from turboserve_amd.sampling.params import SamplingParams

    new = 20
    prompts = model["prompts"]
    want = [plain.greedy_generate(model["wide_raw"], model["wide_tensors"], p, new) for p in prompts]
    longest = max(len(p) for p in prompts) + new
    few = -(-longest // model["page"])  # the longest request just fits alone; together they do not
    for blocks in (64, few):
        with make_engine(model["wide_folder"], "float32", model["page"], num_blocks=blocks, budget=64,
                         run_ahead=True) as engine:
            outputs = engine.generate(prompts, SamplingParams(max_tokens=new, temperature=0.0, ignore_eos=True))
            assert [o.new_token_ids for o in outputs] == want, f"{blocks} pages"
            assert engine.runner.graphs.num_replays > 0
            engine.scheduler.check_invariants()
            assert all(pool.num_in_use == 0 for pool in engine.scheduler.cache.pools)
            if blocks == few:
                assert engine.stats()["num_preemptions"] > 0
    stop = want[0][5]
    expected = want[0][: want[0].index(stop) + 1]
    with make_engine(model["wide_folder"], "float32", model["page"], num_blocks=64, run_ahead=True) as engine:
        outputs = engine.generate(prompts, [SamplingParams(max_tokens=new, temperature=0.0, ignore_eos=True,
                                                           stop_token_ids=(stop,) if i == 0 else ())
                                            for i in range(len(prompts))])
        assert outputs[0].new_token_ids == expected and outputs[0].finish_reason == "stop"
        assert [o.new_token_ids for o in outputs[1:]] == want[1:]
    sampling = [SamplingParams(max_tokens=new, temperature=0.8, top_p=0.9, seed=7 + i, ignore_eos=True, logprobs=True)
                for i in range(len(prompts))]
    results = []
    for ahead in (False, True):
        with make_engine(model["folder"], "bfloat16", model["page"], num_blocks=64, run_ahead=ahead) as engine:
            outputs = engine.generate(prompts, sampling)
            results.append([(o.new_token_ids, o.logprobs) for o in outputs])
    assert results[0] == results[1]


def test_truncated_and_penalised_sampling_through_the_engine(model):
    """top-k, top-p and the repetition penalty through ``LLMEngine`` (not only the kernel): every
    token a request draws is the one the plain sampler draws from the plain logits of the
    sequence so far, with the request's seed, draw number and history."""
    from turboserve_amd.sampling.params import SamplingParams

    new = 10
    settings = [dict(temperature=0.9, top_k=5), dict(temperature=1.1, top_p=0.6), dict(temperature=0.7, top_k=12, top_p=0.8),
                dict(temperature=1.0, repetition_penalty=1.7), dict(temperature=0.0, repetition_penalty=2.5)]
    prompts = [model["prompts"][i % len(model["prompts"])] for i in range(len(settings))]
    params = [SamplingParams(max_tokens=new, seed=31 + i, ignore_eos=True, **kw) for i, kw in enumerate(settings)]
    with make_engine(model["wide_folder"], "float32", model["page"], num_blocks=64, run_ahead=True) as engine:
        outputs = engine.generate(prompts, params)
    for i, (prompt, output, kw) in enumerate(zip(prompts, outputs, settings)):
        tokens = list(prompt)
        assert len(output.new_token_ids) == new
        for draw, token in enumerate(output.new_token_ids):
            logits = plain.forward_logits(model["wide_raw"], model["wide_tensors"], tokens)[-1]
            want, cdf = plain.sample_token(
                logits, temperature=kw["temperature"], seed=31 + i, draw_index=draw, top_k=kw.get("top_k", 0),
                top_p=kw.get("top_p", 1.0), penalty=kw.get("repetition_penalty", 1.0), history=tokens)
            if token != want:  # only a uniform that falls on the edge of two tokens' intervals may differ
                u = plain.philox_uniform(31 + i, draw)
                low = float(cdf[token - 1]) if token > 0 else 0.0
                assert cdf.numel() and low - 1e-5 <= u <= float(cdf[token]) + 1e-5, f"request {i} draw {draw}: {token} != {want}"
            tokens.append(token)


def test_a_penalised_request_that_stops_while_a_step_is_in_flight(model):
    """Steps launched ahead with a repetition penalty: the sampler counts the token that only the
    device knows yet into the history, and a request that hits a stop token while the next step
    is already in flight drops that step's result.  Tokens equal those of the loop that reads
    every step before it schedules the next, and the plain sampler's."""
    from turboserve_amd.sampling.params import SamplingParams

    new = 14
    prompts = model["prompts"]

    def params(stops):
        return [SamplingParams(max_tokens=new, temperature=0.0 if i % 2 else 0.9, seed=400 + i, ignore_eos=True,
                               repetition_penalty=1.6, stop_token_ids=stops.get(i, ()))
                for i in range(len(prompts))]

    with make_engine(model["wide_folder"], "float32", model["page"], num_blocks=64) as engine:
        free = [o.new_token_ids for o in engine.generate(prompts, params({}))]
    for i, (prompt, produced) in enumerate(zip(prompts, free)):  # the plain sampler's tokens, with the history
        tokens = list(prompt)
        for draw, token in enumerate(produced):
            logits = plain.forward_logits(model["wide_raw"], model["wide_tensors"], tokens)[-1]
            want, cdf = plain.sample_token(logits, temperature=0.0 if i % 2 else 0.9, seed=400 + i, draw_index=draw,
                                           penalty=1.6, history=tokens)
            if token != want:
                u = plain.philox_uniform(400 + i, draw)
                low = float(cdf[token - 1]) if token > 0 else 0.0
                assert cdf.numel() and low - 1e-5 <= u <= float(cdf[token]) + 1e-5, f"request {i} draw {draw}: {token} != {want}"
            tokens.append(token)
    # request 0 stops at its 6th token, the last request at its 9th: each while later steps are in flight
    stops = {0: (free[0][5],), len(prompts) - 1: (free[-1][8],)}
    results = []
    for ahead in (False, True):
        with make_engine(model["wide_folder"], "float32", model["page"], num_blocks=64, run_ahead=ahead) as engine:
            outputs = engine.generate(prompts, params(stops))
            results.append([(o.new_token_ids, o.finish_reason) for o in outputs])
            if ahead:
                assert engine.runner.graphs.num_replays > 0
            engine.scheduler.check_invariants()
            assert all(pool.num_in_use == 0 for pool in engine.scheduler.cache.pools)
    assert results[0] == results[1]
    for i, (tokens, reason) in enumerate(results[1]):
        if i in stops:
            cut = free[i].index(stops[i][0]) + 1
            assert tokens == free[i][:cut] and reason == "stop"
        else:
            assert tokens == free[i] and reason == "length"


def test_prompts_are_not_cut_when_chunking_is_off(model):
    """``enable_chunked_prefill=False``: a prompt runs whole or waits; one longer than the token
    budget is refused at arrival (src/turboserve/engine/core/scheduler.py:530-548, 663-667)."""
    from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
    from turboserve_amd.engine.llm_engine import LLMEngine
    from turboserve_amd.sampling.params import SamplingParams

    new = 6
    want = [plain.greedy_generate(model["wide_raw"], model["wide_tensors"], p, new) for p in model["prompts"]]
    budget = max(len(p) for p in model["prompts"]) + 2  # room for the longest prompt, not for two of them
    engine = LLMEngine(EngineConfig(model=str(model["wide_folder"]), dtype="float32", scheduler=SchedulerConfig(
        max_num_seqs=8, max_num_batched_tokens=budget, block_size=model["page"], num_blocks=64, enable_chunked_prefill=False)))
    with engine:
        seen = []
        original = engine.runner.step

        def watched(entries, **kw):
            seen.extend((entry.start, len(entry.tokens)) for entry in entries)
            return original(entries, **kw)

        engine.runner.step = watched
        outputs = engine.generate(model["prompts"], SamplingParams(max_tokens=new, temperature=0.0, ignore_eos=True))
        assert [o.new_token_ids for o in outputs] == want
        lengths = {len(p) for p in model["prompts"]}
        assert all(count in lengths for start, count in seen if start == 0), "a prompt was cut into portions"
        assert all(count == 1 for start, count in seen if start > 0)
        with pytest.raises(ValueError):
            engine.add_request("too-long", tiny.random_tokens(model["vocab"], budget + 1, 3))


def test_more_requests_decode_than_a_recorded_step_takes(model):
    """150 requests decoding at once: more than the 128 rows a recorded step takes, so the step
    runs eagerly (the decode attention without a device-side longest context)."""
    from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
    from turboserve_amd.engine.llm_engine import LLMEngine
    from turboserve_amd.sampling.params import SamplingParams

    count = 150
    prompts = [tiny.random_tokens(model["vocab"], 2 + i % 11, 700 + i) for i in range(count)]
    sampling = SamplingParams(max_tokens=3, temperature=0.0, ignore_eos=True, logprobs=True)
    results = {}
    for dtype in ("float32", "bfloat16"):
        folder = model["wide_folder"] if dtype == "float32" else model["bf16_folder"]
        engine = LLMEngine(EngineConfig(model=str(folder), dtype=dtype, scheduler=SchedulerConfig(
            max_num_seqs=256, max_num_batched_tokens=4096, block_size=model["page"], num_blocks=600)))
        with engine:
            results[dtype] = engine.generate(prompts, sampling)
            assert engine.runner.graphs.num_replays == 0
    for prompt, exact, fast in zip(prompts, results["float32"], results["bfloat16"]):
        assert exact.new_token_ids == plain.greedy_generate(model["wide_raw"], model["wide_tensors"], prompt, 3)
        sequence = prompt + fast.new_token_ids
        logits = plain.forward_logits(model["bf16_raw"], model["bf16_tensors"], sequence)
        for i, token in enumerate(fast.new_token_ids):
            row = logits[len(prompt) - 1 + i]
            assert float(row.max() - row[token]) <= 2e-2 * float(row.abs().max()), "not a near-argmax in bfloat16"


def test_text_prompts_stop_strings_and_the_tokenizers_end_token(model, tmp_path):
    """Text in, text out through a ``tokenizer.json`` (made here with the ``tokenizers`` library:
    one word per token id): the prompt is encoded without special tokens, a stop string ends a
    request and is cut from its text, and the end token that ``tokenizer_config.json`` names ends
    a request although the model's ``config.json`` does not list it (the reference joins both,
    src/turboserve/engine/runtime/engine.py:223-237)."""
    import json
    import shutil

    from tokenizers import Tokenizer
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import WhitespaceSplit

    from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
    from turboserve_amd.engine.llm_engine import LLMEngine
    from turboserve_amd.sampling.params import SamplingParams

    folder = tmp_path / "with_tokenizer"
    shutil.copytree(model["wide_folder"], folder)
    word = lambda token: f"w{token:04d}"  # one length for all, so no word is the start of another
    vocab = {word(i): i for i in range(model["vocab"])}
    tokenizer = Tokenizer(WordLevel(vocab, unk_token=word(0)))
    tokenizer.pre_tokenizer = WhitespaceSplit()
    tokenizer.save(str(folder / "tokenizer.json"))
    prompt_ids = model["prompts"][-1]
    text = " ".join(word(t) for t in prompt_ids)
    free = plain.greedy_generate(model["wide_raw"], model["wide_tensors"], prompt_ids, 10)
    assert len(set(free[:6])) == 6, "the continuation should not repeat a token early"
    scheduler = SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=64, block_size=model["page"], num_blocks=64)
    with LLMEngine(EngineConfig(model=str(folder), dtype="float32", scheduler=scheduler)) as engine:
        assert engine.tokenizer is not None and engine.encode(text) == prompt_ids
        plain_run = engine.generate([text], SamplingParams(max_tokens=10, temperature=0.0))[0]
        assert plain_run.new_token_ids == free and plain_run.finish_reason == "length"
        words = plain_run.text_delta.split()
        assert words == [word(t) for t in free]
        stopped = engine.generate([text], SamplingParams(max_tokens=10, temperature=0.0, stop=[word(free[3])]))[0]
        assert stopped.finish_reason == "stop" and stopped.new_token_ids == free[:4]
        assert stopped.text_delta.split() == [word(t) for t in free[:3]], "the stop string is cut from the text"
    (folder / "tokenizer_config.json").write_text(json.dumps({"eos_token": {"content": word(free[4])}}))
    with LLMEngine(EngineConfig(model=str(folder), dtype="float32", scheduler=scheduler)) as engine:
        assert free[4] in engine.eos_token_ids
        ended = engine.generate([text], SamplingParams(max_tokens=10, temperature=0.0))[0]
        assert ended.finish_reason == "stop" and ended.new_token_ids == free[:5]
        ignored = engine.generate([text], SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True))[0]
        assert ignored.new_token_ids == free


def test_command_line_generates_the_plain_tokens(tmp_path):
    """`turboserve engine random-model` writes a model folder and `turboserve engine generate
    --prompt-ids` (no tokenizer there) prints, per prompt, the greedy tokens of the plain
    implementation; `kv-size` prints its sizing as JSON."""
    import json
    import re
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    config_file = tmp_path / "config.json"
    config_file.write_text(json.dumps(tiny.CONFIG_A))
    folder = tmp_path / "model"
    run = lambda *args: subprocess.run([sys.executable, str(root / "bin" / "turboserve"), *args], capture_output=True,
                                       text=True, timeout=240)
    made = run("engine", "random-model", "--config", str(config_file), "--out", str(folder), "--seed", "3",
               "--dtype", "float32")
    assert made.returncode == 0, made.stderr
    raw, tensors = tiny.read_model_dir(folder)
    prompts = [[5, 17, 3, 200], [9, 9, 9, 9, 9, 9, 1]]
    out = run("engine", "generate", "--model", str(folder), "--dtype", "float32", "--max-tokens", "6", "--ignore-eos",
              "--num-blocks", "16", "--stats", *[a for p in prompts for a in ("--prompt-ids", ",".join(map(str, p)))])
    assert out.returncode == 0, out.stderr
    shown = [json.loads(m) for m in re.findall(r"^output \d+: (\[.*\])$", out.stdout, flags=re.M)]
    assert shown == [plain.greedy_generate(raw, tensors, p, 6) for p in prompts]
    assert "2 completions in" in out.stdout and "finish_reason=length" in out.stdout
    sizing = run("engine", "kv-size", "--model", str(folder), "--dtype", "float32", "--max-model-len", "64")
    assert sizing.returncode == 0, sizing.stderr
    assert min(json.loads(sizing.stdout[sizing.stdout.index("{"):])["num_blocks"]) >= 1  # one pool per cache group
