#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at the Qwen2.5-7B layer sizes on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Everything is measured through the engine's own entry point: requests are given to
``LLMEngine`` (scheduler, cache manager, step function, sampler) and the clock runs around
calls of ``LLMEngine.step()``, the loop ``generate()`` runs.  A "step" is one decode step: every
live request gets one token.  As always in the engine, a decode step is launched before the
host has read the tokens of the step before it.

The default run has the Qwen2.5-7B layer sizes (the benchmark's named configuration), random
weights (N(0, 0.02), norm gains 1) and 8 requests whose prompts of uniform-random token ids
are prefilled (chunked, by the engine) to a context of 8,192 tokens; then W untimed and K timed
decode steps.  One JSON line is printed: ``value`` is decoded tokens a second; ``prefill`` times
one 2,048-token prompt from arrival to its first token; ``roofline`` prices the decode step
against HBM bandwidth (against the published peak, and against what a kernel that only reads
gets from this device, ``read_probe``); ``points`` holds decode at batch 1 and 64 at the same
context, the benchmark's literal workload (prompts of 512 tokens, 256 generated,
end-of-sequence ignored, greedy) at 1, 8 and 64 requests, with the details of those runs under
``workload``, and further sizes, detailed under ``further``: prompts of 8,192 and 32,767 tokens
in portions of 2,048, decode at batch 1 and 8 with about 32 k tokens of context, and the
default decode step at the 14B and 32B shapes (all of their layers) and the 14B shape's mixed
step (32 decode tokens and one 2,048-token prompt).  A prefill's projections
are this engine's own product or the BLAS library's, whichever is the faster one for the shape:
both are timed once at the engine's start (``--no-gemm-tuning`` leaves the library's kernels to
its heuristic and the choice to a rule).
Peaks are the published MI355X figures: HBM 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s, fp32 157.3
TFLOP/s.

Other runs: ``--shape 14b --batch 32 --mixed-prefill 2048`` (every step holds the decode tokens
and one 2,048-token prompt), ``--shape 32b --batch 64 --fill-hbm`` (a cache pool of all the
free memory), ``--closed-loop C [--sampled]`` (the reference's serving profile driven offline: 256
requests of 128..1,024 tokens in and 64..512 out, C in flight; the library's products run at a
few step sizes that are all timed at start-up, about 70 s the first time), ``--attention-prefill T[,CTX]`` (the
prefill attention kernel alone), ``--sample-kernel ROWS`` (the sampling kernel alone), ``--hbm-read`` (a kernel that only reads: what the memory gives), ``--only-prefill [TOKENS]`` (one prompt's prefill alone, 2,048 tokens or TOKENS), ``--kernel-shares TRACE.csv`` (no GPU: the per-kernel table of a
``rocprofv3 --kernel-trace`` of any of these runs).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile
import time

HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}

#: The benchmark's named configuration: Qwen2.5-7B layer sizes.
SHAPE_7B = {
    "architectures": ["Qwen2ForCausalLM"],
    "model_type": "qwen2",
    "hidden_size": 3584,
    "num_hidden_layers": 28,
    "num_attention_heads": 28,
    "num_key_value_heads": 4,
    "head_dim": 128,
    "intermediate_size": 18944,
    "vocab_size": 152064,
    "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False,
    "use_sliding_window": False,
    "max_position_embeddings": 32768,
}
#: The 14B and 32B layer sizes of the same family: the other shapes a run can be asked for.
SHAPE_14B = dict(SHAPE_7B, hidden_size=5120, num_hidden_layers=48, num_attention_heads=40, num_key_value_heads=8,
                 intermediate_size=13824, rms_norm_eps=1e-5)
SHAPE_32B = dict(SHAPE_14B, num_hidden_layers=64, intermediate_size=27648)
SHAPES = {"7b": ("Qwen2.5-7B", SHAPE_7B), "14b": ("Qwen2.5-14B", SHAPE_14B), "32b": ("Qwen2.5-32B", SHAPE_32B)}
CONTEXT = 8192
LONG_CONTEXT = 32768
PREFILL_TOKENS = 2048
PAGE = 16
#: The benchmark's literal decode workload: prompt length and generated tokens.
WORKLOAD_PROMPT, WORKLOAD_NEW = 512, 256


def parse_args(argv: list[str] | None = None) -> argparse.Namespace:
    p = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=64)
    p.add_argument("--warmup", type=int, default=40,
                   help="untimed steps first; the clocks take some tens of milliseconds of load to settle")
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--context", type=int, default=CONTEXT)
    p.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (named in config)")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64 and the literal workload")
    p.add_argument("--no-prefill", action="store_true")
    p.add_argument("--no-gemm-tuning", action="store_true",
                   help="leave the choice of the BLAS library's prefill kernels to its heuristic")
    p.add_argument("--only-prefill", nargs="?", type=int, const=PREFILL_TOKENS, default=None, metavar="TOKENS",
                   help="run the prefill of one prompt alone (for profiling): 2,048 tokens, or TOKENS")
    p.add_argument("--shape", default="7b", choices=sorted(SHAPES), help="layer sizes (the default run is 7b)")
    p.add_argument("--fill-hbm", action="store_true", help="size the cache pool to the free device memory")
    p.add_argument("--mixed-prefill", type=int, default=0, metavar="N",
                   help="time steps that hold the batch's decode tokens and one whole N-token prompt")
    p.add_argument("--no-run-ahead", action="store_true",
                   help="read every step's tokens before the next is scheduled, as the reference's loop does")
    p.add_argument("--kernel-shares", metavar="TRACE.csv", default=None,
                   help="print the per-kernel table of a rocprofv3 kernel trace of a run of this program and exit")
    p.add_argument("--shares-steps", type=int, default=4, help="steps at the end of the trace that the table covers")
    p.add_argument("--closed-loop", type=int, default=0, metavar="C",
                   help="the reference's serving profile offline: 256 requests of 128..1024 input and 64..512 output "
                        "tokens, C of them live at a time; prints output tokens/s, time to first token and time between tokens")
    p.add_argument("--sampled", action="store_true",
                   help="with --closed-loop: temperature 0.7, top-p 0.8, top-k 20, repetition penalty 1.05 instead of greedy")
    p.add_argument("--sample-kernel", type=int, default=0, metavar="ROWS",
                   help="time the sampling kernel alone on ROWS rows of logits of the shape's vocabulary, and exit")
    p.add_argument("--hbm-read", action="store_true",
                   help="time a kernel that only reads, walking memory in several ways with plain and non-temporal "
                        "loads (what the memory gives: the practical ceiling of the decode step), and exit")
    p.add_argument("--no-further", action="store_true",
                   help="skip the further sizes: prefill of 8,192 and 32,767 tokens, decode at 32 k tokens of context, "
                        "the decode step at the 14B and 32B shapes")
    p.add_argument("--attention-prefill", metavar="TOKENS[,CONTEXT]", default=None,
                   help="time the prefill attention kernel alone on the shape's heads: one request that brings TOKENS "
                        "tokens and holds CONTEXT afterwards (default: TOKENS), and exit")
    return p.parse_args(argv)


def tuning_file() -> str:
    return os.path.join(tempfile.gettempdir(), f"turboserve_amd_bench_gemm_{os.getuid()}.csv")


def make_engine(model, config, *, max_num_seqs: int, budget: int, tokens_per_request: int, fill_hbm: bool = False,
                tune_tokens: tuple[int, ...] = (), run_ahead: bool = True, step_sizes: bool = False):
    """An ``LLMEngine`` around the already loaded model, with a cache pool for ``max_num_seqs``
    requests of ``tokens_per_request`` tokens (or, with ``fill_hbm``, 90% of the free memory)."""
    import torch

    from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
    from turboserve_amd.engine.llm_engine import LLMEngine

    num_blocks = max_num_seqs * -(-tokens_per_request // PAGE)
    if fill_hbm:
        free, _ = torch.cuda.mem_get_info()
        page_bytes = config.kv_bytes_per_token(model.runtime.dtype) * PAGE
        num_blocks = max(num_blocks, int(free * 0.9) // page_bytes)
    engine_config = EngineConfig(
        model="(random weights)", dtype="bfloat16" if model.runtime.dtype == torch.bfloat16 else "float32", seed=0,
        tune_gemm_tokens=tune_tokens, tune_gemm_step_sizes=step_sizes, gemm_tuning_file=tuning_file(), run_ahead=run_ahead,
        scheduler=SchedulerConfig(max_num_seqs=max_num_seqs, max_num_batched_tokens=budget, block_size=PAGE,
                                  num_blocks=num_blocks),
    )
    return LLMEngine(engine_config, model=model, model_config=config)


def random_prompts(config, count: int, length: int, seed: int) -> list[list[int]]:
    import torch

    generator = torch.Generator().manual_seed(seed)
    return [torch.randint(0, config.vocab_size, (length,), generator=generator).tolist() for _ in range(count)]


def run_decode(model, config, batch: int, prompt_len: int, *, steps: int, warmup: int, fill_hbm: bool = False,
               mixed_prefill: int = 0, tune: bool = False, run_ahead: bool = True) -> dict:
    """``batch`` requests with prompts of ``prompt_len`` uniform-random ids through
    ``LLMEngine``: prefill (chunked by the engine; requests whose prompt is done decode
    meanwhile), ``warmup`` untimed decode steps of the whole batch, ``steps`` timed ones.  With
    ``mixed_prefill`` every step also holds one new request's whole prompt of that many tokens
    (which ends after its first token)."""
    import torch

    from turboserve_amd.sampling.params import SamplingParams

    budget = max(PREFILL_TOKENS, mixed_prefill + batch, batch)
    # Tokens a request may have to produce: the steps of this run and those it decodes while the
    # others' prompts are still being prefilled, with a few to spare (no request may end inside the clock).
    max_new = warmup + steps + batch * -(-prompt_len // budget) + 8
    engine = make_engine(
        model, config, max_num_seqs=batch + (1 if mixed_prefill else 0), budget=budget,
        tokens_per_request=prompt_len + max_new + (-(-mixed_prefill // batch) if mixed_prefill else 0),
        fill_hbm=fill_hbm, tune_tokens=(mixed_prefill + batch,) if (mixed_prefill and tune) else (), run_ahead=run_ahead,
    )
    pool_tokens = min(engine.storage.num_pages) * PAGE
    decode = SamplingParams(max_tokens=max_new, temperature=0.0, ignore_eos=True)
    one = SamplingParams(max_tokens=1, temperature=0.0, ignore_eos=True)
    extra = random_prompts(config, 1, max(mixed_prefill, 1), 99)[0]
    sequences = [engine.add_request(f"r{index}", prompt, decode)
                 for index, prompt in enumerate(random_prompts(config, batch, prompt_len, 1234))]
    started = time.perf_counter()
    first_tokens = 0
    while first_tokens < batch:  # the prompts' portions, until every request has its first token
        first_tokens += sum(1 for out in engine.step() if out.output_tokens == 1)
    torch.cuda.synchronize()
    prefill_seconds = time.perf_counter() - started
    arrivals = 0

    def step() -> None:
        nonlocal arrivals
        if mixed_prefill:
            engine.add_request(f"p{arrivals}", extra, one)
            arrivals += 1
        engine.step()

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    context_before = sum(seq.num_tokens for seq in sequences) / batch
    started = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    seconds = time.perf_counter() - started
    stats = engine.stats()
    assert not any(seq.is_finished for seq in sequences), "a request ended inside the timed steps"
    for index in range(batch):
        engine.abort(f"r{index}")
    engine.close()
    return {"tokens_per_s": batch * steps / seconds, "step_seconds": seconds / steps, "prefill_seconds": prefill_seconds,
            "mean_context": context_before + steps / 2, "pool_tokens": pool_tokens,
            "preemptions": int(stats["num_preemptions"])}


def run_workload(model, config, batch: int, prompt_len: int, new_tokens: int, run_ahead: bool = True) -> dict:
    """The benchmark's literal decode workload through ``LLMEngine``'s loop (the loop the
    reference times, src/turboserve/engine/runtime/engine.py:414-448): ``batch`` prompts of
    ``prompt_len`` uniform-random ids, ``new_tokens`` generated each, greedy, end-of-sequence
    ignored.  Decoding is priced over the steps in which the whole batch decodes: from the
    moment the last request has its first token to the moment the first request ends."""
    from turboserve_amd.sampling.params import SamplingParams

    engine = make_engine(model, config, max_num_seqs=batch, budget=PREFILL_TOKENS,
                         tokens_per_request=prompt_len + new_tokens + 1, run_ahead=run_ahead)
    sampling = SamplingParams(max_tokens=new_tokens, temperature=0.0, ignore_eos=True)
    sequences = [engine.add_request(f"w{index}", prompt, sampling)
                 for index, prompt in enumerate(random_prompts(config, batch, prompt_len, 777))]
    started = time.perf_counter()
    first_tokens = finished = tokens = calls = 0
    window_start = window_end = None
    context_at_start = 0.0
    while engine.has_unfinished():
        outputs = engine.step()
        now = time.perf_counter()
        if window_start is not None and window_end is None:
            calls += 1
            tokens += sum(len(out.new_token_ids) for out in outputs)
        first_tokens += sum(1 for out in outputs if out.output_tokens == 1)
        finished += sum(1 for out in outputs if out.finished)
        if window_start is None and first_tokens == batch:
            window_start = now
            context_at_start = sum(seq.num_tokens for seq in sequences) / batch
        if window_end is None and finished > 0:
            window_end = now
    total = time.perf_counter() - started
    engine.close()
    assert all(seq.num_output_tokens == new_tokens for seq in sequences)
    window = window_end - window_start
    return {"tokens_per_s": tokens / window, "step_seconds": window / calls, "steps": calls,
            "mean_context": context_at_start + calls / 2, "first_tokens_seconds": window_start - started,
            "total_seconds": total, "total_tokens_per_s": batch * new_tokens / total}


def run_prefill(model, config, tokens: int, repeats: int = 3, tune: bool = True, budget: int | None = None) -> float:
    """Seconds (best of ``repeats``) from the arrival of a ``tokens``-long prompt to its first
    token on the host, through ``LLMEngine`` with a step budget that takes the prompt whole, or
    with ``budget`` tokens a step (the prompt then runs in portions, as it does in serving)."""
    import torch

    from turboserve_amd.sampling.params import SamplingParams

    budget = min(tokens, budget or tokens)
    engine = make_engine(model, config, max_num_seqs=1, budget=budget, tokens_per_request=tokens + 1,
                         tune_tokens=(budget,) if tune else ())
    prompt = random_prompts(config, 1, tokens, 4321)[0]
    best = float("inf")
    for attempt in range(repeats + 1):
        torch.cuda.synchronize()
        started = time.perf_counter()
        engine.add_request(f"p{attempt}", prompt, SamplingParams(max_tokens=1, temperature=0.0, ignore_eos=True))
        outputs = []
        while not outputs:
            outputs = engine.step()
        torch.cuda.synchronize()
        best = min(best, time.perf_counter() - started)
        assert outputs[0].finished and len(outputs[0].new_token_ids) == 1
    engine.close()
    return best


def run_closed_loop(model, config, concurrency: int, *, sampled: bool, requests: int = 256, tune: bool = True) -> dict:
    """The workload shape of the reference's serving benchmark (configs/bench/profiles.yaml:26-40:
    256 requests, 128 to 1,024 input tokens, 64 to 512 output tokens, a fixed number in flight),
    driven offline: a request is added the moment one ends.  Lengths and token ids are seeded
    uniform draws; every request runs to its output length."""
    import random

    import torch

    from turboserve_amd.sampling.params import SamplingParams

    rng = random.Random(1)
    shapes = [(rng.randint(128, 1024), rng.randint(64, 512)) for _ in range(requests)]
    engine = make_engine(model, config, max_num_seqs=concurrency, budget=PREFILL_TOKENS,
                         tokens_per_request=1024 + 512 + PAGE, step_sizes=tune)
    prompts = [random_prompts(config, 1, length, 100 + index)[0] for index, (length, _) in enumerate(shapes)]

    def params(index: int) -> "SamplingParams":
        if sampled:
            return SamplingParams(max_tokens=shapes[index][1], temperature=0.7, top_p=0.8, top_k=20,
                                  repetition_penalty=1.05, seed=index, ignore_eos=True)
        return SamplingParams(max_tokens=shapes[index][1], temperature=0.0, ignore_eos=True)

    sequences, live, produced, steps = [], 0, 0, 0

    def admit() -> None:
        nonlocal live
        while live < concurrency and len(sequences) < requests:
            index = len(sequences)
            sequences.append(engine.add_request(f"r{index}", prompts[index], params(index)))
            live += 1

    admit()
    torch.cuda.synchronize()
    started = time.perf_counter()
    while engine.has_unfinished():
        for output in engine.step():
            produced += len(output.new_token_ids)
            live -= bool(output.finished)
        admit()
        steps += 1
    torch.cuda.synchronize()
    seconds = time.perf_counter() - started
    preemptions = int(engine.stats()["num_preemptions"])
    engine.close()

    def median(values: list[float]) -> float:
        ordered = sorted(values)
        return ordered[len(ordered) // 2]

    first = [seq.timing.t_first_token - seq.timing.t_arrival for seq in sequences]
    between = [(seq.timing.t_finished - seq.timing.t_first_token) / max(1, seq.num_output_tokens - 1) for seq in sequences]
    return {"metric": f"closed loop, {requests} requests of 128..1024 in / 64..512 out, {concurrency} in flight "
                      f"(through LLMEngine, {'sampled' if sampled else 'greedy'})",
            "value": round(produced / seconds, 1), "unit": "output tokens/s", "seconds": round(seconds, 2), "steps": steps,
            "ms_per_step": round(seconds / steps * 1e3, 3), "output_tokens": produced,
            "input_tokens": sum(length for length, _ in shapes), "first_token_ms_p50": round(median(first) * 1e3, 1),
            "between_tokens_ms_p50": round(median(between) * 1e3, 2), "preemptions": preemptions}


def run_attention_prefill(shape: dict, tokens: int, context: int, launches: int = 15) -> dict:
    """The prefill attention kernel alone (no model): ``tokens`` rows of one request at the end of
    ``context`` keys on scrambled pages, random queries, keys and values; the best of ``launches``
    launches by device events.  Flops: causal attention of the rows over what they see."""
    import torch

    from turboserve_amd.kernels.ops import Ops

    heads, kv_heads = shape["num_attention_heads"], shape["num_key_value_heads"]
    dim = shape["hidden_size"] // heads
    ops = Ops("cuda:0")
    pages = -(-context // PAGE)
    generator = torch.Generator(device="cuda").manual_seed(0)
    k_pages = torch.randn(pages, kv_heads, PAGE, dim, device="cuda", generator=generator).bfloat16()
    v_pages = torch.randn(pages, kv_heads, dim, PAGE, device="cuda", generator=generator).bfloat16()
    q = torch.randn(tokens, heads * dim, device="cuda", generator=generator).bfloat16()
    table = torch.randperm(pages, device="cuda", generator=generator).int().view(1, -1)
    starts = torch.tensor([0, tokens], dtype=torch.int32, device="cuda")
    contexts = torch.tensor([context], dtype=torch.int32, device="cuda")
    rows = ops.prefill_block_rows(dim, heads, kv_heads)
    blocks = ops.prefill_blocks([tokens], [context], rows, heads=heads, kv_heads=kv_heads, head_dim=dim, block_size=PAGE)
    out = torch.empty(tokens, heads * dim, dtype=torch.bfloat16, device="cuda")
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for _ in range(launches):
        start.record()
        ops.attention_prefill(out, q, heads * dim, k_pages, v_pages, table, starts, contexts, blocks, heads, dim ** -0.5,
                              None, context, rows)
        stop.record()
        stop.synchronize()
        best = min(best, start.elapsed_time(stop) * 1e-3)
    flops = 4.0 * heads * dim * (tokens * (context - tokens) + tokens * tokens / 2)
    return {"kernel": "prefill attention", "tokens": tokens, "context": context, "heads": heads, "kv_heads": kv_heads,
            "head_dim": dim, "us": round(best * 1e6, 1), "tflops": round(flops / best / 1e12, 1),
            "frac": round(flops / best / PEAK_FLOPS["bf16"], 4)}


def run_sample_kernel(shape: dict, rows: int, launches: int = 20) -> dict:
    """The sampling kernel alone on ``rows`` rows of logits of the shape's vocabulary, of a language
    model's kind (N(0, 2.5) with thirty tokens at 12 to 24): microseconds a launch by device
    events, the host's preparation of the launch included, for several settings."""
    import torch

    from turboserve_amd.kernels.ops import Ops
    from turboserve_amd.sampling.params import SamplingParams
    from turboserve_amd.sampling.sampler import Sampler

    vocab = shape["vocab_size"]
    sampler = Sampler(Ops("cuda:0"))
    generator = torch.Generator(device="cuda").manual_seed(0)
    logits = torch.randn(rows, vocab, device="cuda", generator=generator) * 2.5
    spots = torch.randint(0, vocab, (rows, 30), device="cuda", generator=generator)
    logits.scatter_(1, spots, torch.rand(rows, 30, device="cuda", generator=generator) * 12 + 12)
    settings = {
        "greedy": dict(temperature=0.0),
        "temperature 0.8": dict(temperature=0.8),
        "temperature 0.7, top-k 20, top-p 0.8": dict(temperature=0.7, top_k=20, top_p=0.8),
        "the same with repetition penalty 1.05 over 800 tokens": dict(temperature=0.7, top_k=20, top_p=0.8, repetition_penalty=1.05),
        "temperature 0.8, top-p 0.9": dict(temperature=0.8, top_p=0.9),
        "temperature 0.8, top-k 50": dict(temperature=0.8, top_k=50),
    }
    histories = [list(range(100, 900)) for _ in range(rows)]
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    result = {"kernel": "sampling", "rows": rows, "vocab": vocab, "us": {}}
    for name, kwargs in settings.items():
        params = [SamplingParams(**kwargs) for _ in range(rows)]
        for _ in range(3):
            sampler.launch(logits, params, list(range(rows)), [3] * rows, histories)
        torch.cuda.synchronize()
        start.record()
        for _ in range(launches):
            sampler.launch(logits, params, list(range(rows)), [3] * rows, histories)
        stop.record()
        stop.synchronize()
        result["us"][name] = round(start.elapsed_time(stop) / launches * 1e3, 1)
    return result


def run_hbm_read(launches: int = 12) -> dict:
    """What the memory gives a kernel that only reads (``csrc/probe.hip``), in GB/s, for a few ways
    of walking 272 MB (the 7B shape's gate|up matrix; five copies in turn, so that no cache holds
    them): the rows as a checkpoint stores them in tiles of 160, 64 and 32 rows as the decode
    products walk them, the same bytes with every workgroup's iteration contiguous, and one long
    contiguous stream per workgroup; each with plain and with non-temporal loads."""
    import torch

    from turboserve_amd.kernels.ops import Ops

    ops = Ops("cuda:0")
    n, k = 37888, 3584
    row_bytes, iters, copies = 2 * k, k // 128, 5
    size = (n + 512) * row_bytes
    buffers = [torch.randint(0, 2 ** 31 - 1, (size // 4,), dtype=torch.int32, device="cuda") for _ in range(copies)]
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def rate(iterations: int, **walk) -> float:
        read = walk["workgroups"] * 16 * walk["pieces"] * iterations * 256
        for buffer in buffers:
            ops.hbm_read(buffer, iters=iterations, **walk)
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(3):
            start.record()
            for _ in range(max(1, launches // copies)):
                for buffer in buffers:
                    ops.hbm_read(buffer, iters=iterations, **walk)
            stop.record()
            stop.synchronize()
            best = min(best, start.elapsed_time(stop) * 1e-3 / (max(1, launches // copies) * copies))
        return round(read / best / 1e9, 1)

    table: dict[str, float] = {}
    for once in (False, True):
        tag = "non-temporal" if once else "plain"
        for pieces, ahead in ((10, 2), (4, 2), (2, 1)):
            rows = 16 * pieces
            table[f"rows as stored, {rows} a workgroup, {tag}"] = rate(
                iters, workgroups=-(-n // rows), pieces=pieces, ahead=ahead, wg_stride=rows * row_bytes, it_stride=256,
                blk_rows=rows, blk_stride=0, row_stride=row_bytes, non_temporal=once)
            table[f"iteration contiguous, {rows} rows a workgroup, {tag}"] = rate(
                iters, workgroups=-(-n // rows), pieces=pieces, ahead=ahead, wg_stride=iters * rows * 256,
                it_stride=rows * 256, blk_rows=rows, blk_stride=0, row_stride=256, non_temporal=once)
        for workgroups in (256, 1024):
            chunk = 16 * 4 * 256
            count = n * row_bytes // (workgroups * chunk)
            table[f"one contiguous stream a workgroup, {workgroups} workgroups, {tag}"] = rate(
                count, workgroups=workgroups, pieces=4, ahead=2, wg_stride=count * chunk, it_stride=chunk, blk_rows=64,
                blk_stride=0, row_stride=256, non_temporal=once)
    return {"kernel": "read-only probe", "bytes": n * row_bytes, "unit": "GB/s", "rates": table,
            "best": max(table.values()), "peak": HBM_PEAK_GBS}


def decode_bytes(config, layers: int, batch: int, context: float, itemsize: int) -> float:
    """Bytes a decode step has to read: every weight it uses once (all but the embedding
    table, of which it reads one row per request) and the cache of the live requests."""
    h, i, v = config.hidden_size, config.intermediate_size, config.vocab_size
    qkv = config.q_proj_size + 2 * config.kv_proj_size
    per_layer = h * qkv + qkv + config.q_proj_size * h + 3 * h * i + 2 * h
    weights = (layers * per_layer + h + v * h + batch * h) * itemsize
    cache = batch * context * 2 * layers * config.kv_proj_size * itemsize
    return float(weights + cache)


def prefill_flops(config, layers: int, tokens: int) -> float:
    """Flops of one whole-prompt step: the projections (2 flops per weight per token), causal
    attention (4 * Hq * D * T^2 / 2 per layer) and one head row."""
    h, i = config.hidden_size, config.intermediate_size
    qkv = config.q_proj_size + 2 * config.kv_proj_size
    linear = layers * (h * qkv + config.q_proj_size * h + 3 * h * i)
    attention = layers * 4 * config.q_proj_size * tokens * tokens / 2
    return 2.0 * tokens * linear + attention + 2.0 * config.vocab_size * h


def main(argv: list[str] | None = None) -> int:
    args = parse_args(argv)
    if args.kernel_shares:
        from turboserve_amd.profiling import format_shares, step_shares

        print(format_shares(step_shares(args.kernel_shares, steps=args.shares_steps)))
        return 0
    if args.sample_kernel:
        print(json.dumps(run_sample_kernel(SHAPES[args.shape][1], args.sample_kernel)))
        return 0
    if args.hbm_read:
        print(json.dumps(run_hbm_read()))
        return 0
    if args.attention_prefill:
        sizes = [int(v) for v in args.attention_prefill.split(",")]
        print(json.dumps(run_attention_prefill(SHAPES[args.shape][1], sizes[0], sizes[-1])))
        return 0
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine (single-GPU by design)")
        return 2
    import torch

    from turboserve_amd.engine.loading import build_model, make_runtime, resolve_run_dtype
    from turboserve_amd.hwinfo import brief
    from turboserve_amd.weights.random_init import random_tensors_on_device

    shape_name, shape = SHAPES[args.shape]
    shape = dict(shape)
    full_layers = shape["num_hidden_layers"]
    if args.layers is not None:
        shape["num_hidden_layers"] = args.layers
    dtype = resolve_run_dtype(args.dtype)
    runtime = make_runtime(dtype, "cuda:0")
    config, model = build_model(shape, runtime)
    random_tensors_on_device(model, seed=0)
    layers = config.num_hidden_layers
    itemsize = 2 if dtype == torch.bfloat16 else 4
    dtype_key = "bf16" if dtype == torch.bfloat16 else "fp32"
    tune = not args.no_gemm_tuning and dtype == torch.bfloat16
    run_ahead = not args.no_run_ahead

    if args.closed_loop:
        record = run_closed_loop(model, config, args.closed_loop, sampled=args.sampled, tune=tune)
        record.update({"dtype": dtype_key, "layers": layers, "model": f"{shape_name} shape"})
        print(json.dumps(record))
        return 0
    if args.only_prefill:
        seconds = run_prefill(model, config, args.only_prefill, tune=tune)
        ops = model.runtime.ops
        # What the start-up timing found for the step's products (device time of one launch).
        products = {f"{n}x{k} at {rows} rows, {kind}": {"own_us": round(own * 1e3, 1), "library_us": round(library * 1e3, 1)}
                    for (rows, n, k, kind), (own, library) in sorted(ops.wide_timings.items())
                    if rows == ops.library_rows(args.only_prefill)}
        print(json.dumps({"prefill_ms": round(seconds * 1e3, 3), "tokens": args.only_prefill, "layers": layers,
                          "tokens_per_s": round(args.only_prefill / seconds, 1),
                          "frac": round(prefill_flops(config, layers, args.only_prefill) / seconds / PEAK_FLOPS[dtype_key], 4),
                          "products": products}))
        return 0

    main_run = run_decode(model, config, args.batch, args.context - 1, steps=args.steps, warmup=args.warmup,
                          fill_hbm=args.fill_hbm, mixed_prefill=args.mixed_prefill, tune=tune, run_ahead=run_ahead)
    step_seconds = main_run["step_seconds"]
    if args.mixed_prefill:
        # A mixed step is priced by its products' flops, not by bytes: say what ran and stop there.
        flops = (prefill_flops(config, layers, args.mixed_prefill)
                 + 2.0 * args.batch * decode_bytes(config, layers, 0, 0, 1)  # every weight once per decode token
                 + 4.0 * args.batch * layers * config.q_proj_size * args.context)  # and its attention
        print(json.dumps({
            "metric": f"mixed step: {args.batch} decode tokens + one {args.mixed_prefill}-token prompt "
                      f"({shape_name} shape, one MI355X, through LLMEngine)",
            "value": round((args.batch + args.mixed_prefill) / step_seconds, 1), "unit": "tokens/s",
            "decode_tokens_per_s": round(main_run["tokens_per_s"], 2), "ms_per_step": round(step_seconds * 1e3, 3),
            "steps": args.steps, "warmup": args.warmup, "dtype": dtype_key, "decode_context": args.context,
            "layers": layers, "kv_pool_tokens": main_run["pool_tokens"],
            "flops_frac": round(flops / step_seconds / PEAK_FLOPS[dtype_key], 4),
        }))
        return 0
    read = decode_bytes(config, layers, args.batch, main_run["mean_context"], itemsize)
    achieved = read / step_seconds / 1e9
    result = {
        "metric": f"decode tok/s ({shape_name} shape, paged cache, one MI355X)",
        "value": round(main_run["tokens_per_s"], 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_seconds * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype_key,
        "data": "synthetic: random weights N(0,0.02), uniform-random token ids; prompts prefilled by the engine",
        "config": {
            "model": f"{shape_name} shape (Qwen2ForCausalLM)",
            "global_batch": args.batch,
            "seq_len": args.context,
            "parallelism": "single GPU",
            "layers": layers,
            "layers_of_shape": full_layers,
            "hidden_size": config.hidden_size,
            "num_attention_heads": config.num_attention_heads,
            "num_key_value_heads": config.num_key_value_heads,
            "head_dim": config.head_dim,
            "intermediate_size": config.intermediate_size,
            "vocab_size": config.vocab_size,
            "rope_theta": config.rope_theta,
            "rms_norm_eps": config.rms_norm_eps,
            "tie_word_embeddings": config.tie_word_embeddings,
            "page_size": PAGE,
            "kv_pool_tokens": main_run["pool_tokens"],
            "prefill_tokens": PREFILL_TOKENS,
            "path": "LLMEngine.step (scheduler, cache manager, step function, sampler)" + ("" if run_ahead else ", no run-ahead"),
            "sampling": "greedy",
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
        },
    }
    if not args.no_prefill:
        seconds = run_prefill(model, config, PREFILL_TOKENS, tune=tune)
        flops = prefill_flops(config, layers, PREFILL_TOKENS)
        result["prefill"] = {
            "value": round(PREFILL_TOKENS / seconds, 1),
            "tokens": PREFILL_TOKENS,
            "ms": round(seconds * 1e3, 3),
            "frac": round(flops / seconds / PEAK_FLOPS[dtype_key], 4),
        }
    if not args.no_points:
        points, workload = {}, {}
        for batch in (1, 64):
            run = run_decode(model, config, batch, args.context - 1, steps=max(8, args.steps // 2),
                             warmup=max(2, args.warmup // 2), run_ahead=run_ahead)
            points[f"decode_b{batch}"] = round(run["tokens_per_s"], 2)
        # The benchmark's literal workload: prompts of 512 ids, 256 generated, 1 / 8 / 64 requests.
        for batch in (1, 8, 64):
            run = run_workload(model, config, batch, WORKLOAD_PROMPT, WORKLOAD_NEW, run_ahead=run_ahead)
            read = decode_bytes(config, layers, batch, run["mean_context"], itemsize)
            points[f"decode_b{batch}_prompt{WORKLOAD_PROMPT}_new{WORKLOAD_NEW}"] = round(run["tokens_per_s"], 2)
            workload[f"b{batch}"] = {
                "ms_per_step": round(run["step_seconds"] * 1e3, 4), "steps": run["steps"],
                "mean_context": round(run["mean_context"], 1),
                "hbm_frac": round(read / run["step_seconds"] / 1e9 / HBM_PEAK_GBS, 4),
                "first_tokens_ms": round(run["first_tokens_seconds"] * 1e3, 2),
                "whole_run_tokens_per_s": round(run["total_tokens_per_s"], 2),
            }
        result["points"] = points
        result["workload"] = workload
    if not args.no_further and not args.no_points and args.shape == "7b" and full_layers == layers:
        # Further sizes and contexts: long prompts in portions of the step budget, and decode steps
        # whose requests hold about 32 k tokens (the shape's max_position_embeddings).
        further = {}
        for tokens in (8192, LONG_CONTEXT - 1):
            seconds = run_prefill(model, config, tokens, repeats=2, tune=tune, budget=PREFILL_TOKENS)
            result.setdefault("points", {})[f"prefill_{tokens}"] = round(tokens / seconds, 1)
            further[f"prefill_{tokens}"] = {"ms": round(seconds * 1e3, 2), "budget": PREFILL_TOKENS,
                                            "frac": round(prefill_flops(config, layers, tokens) / seconds / PEAK_FLOPS[dtype_key], 4)}
        for batch in (1, 8):
            steps, warmup = 24, 12
            run = run_decode(model, config, batch, LONG_CONTEXT - 1 - steps - warmup - 16, steps=steps, warmup=warmup,
                             run_ahead=run_ahead)
            read = decode_bytes(config, layers, batch, run["mean_context"], itemsize)
            result["points"][f"decode_b{batch}_ctx{LONG_CONTEXT}"] = round(run["tokens_per_s"], 2)
            further[f"decode_b{batch}_ctx{LONG_CONTEXT}"] = {
                "ms_per_step": round(run["step_seconds"] * 1e3, 4), "mean_context": round(run["mean_context"], 1),
                "hbm_frac": round(read / run["step_seconds"] / 1e9 / HBM_PEAK_GBS, 4)}
        # The same decode step at the two wider shapes of the family (all of their layers), so that
        # their figures are taken by whoever runs this, not only quoted.
        del model
        for other in ("14b", "32b"):
            other_name, other_shape = SHAPES[other]
            torch.cuda.empty_cache()
            other_config, other_model = build_model(dict(other_shape), runtime)
            random_tensors_on_device(other_model, seed=0)
            steps, warmup = 16, 8
            run = run_decode(other_model, other_config, args.batch, args.context - 1, steps=steps, warmup=warmup,
                             run_ahead=run_ahead)
            read = decode_bytes(other_config, other_config.num_hidden_layers, args.batch, run["mean_context"], itemsize)
            result["points"][f"decode_b{args.batch}_{other}"] = round(run["tokens_per_s"], 2)
            further[f"decode_b{args.batch}_{other}"] = {
                "model": f"{other_name} shape", "layers": other_config.num_hidden_layers,
                "ms_per_step": round(run["step_seconds"] * 1e3, 4), "mean_context": round(run["mean_context"], 1),
                "hbm_frac": round(read / run["step_seconds"] / 1e9 / HBM_PEAK_GBS, 4)}
            if other == "14b":
                # The 14B shape's mixed step: 32 decode tokens (context as above) and one whole
                # 2,048-token prompt in every step.
                mixed_batch = 32
                run = run_decode(other_model, other_config, mixed_batch, args.context - 1, steps=12, warmup=4,
                                 mixed_prefill=PREFILL_TOKENS, tune=tune, run_ahead=run_ahead)
                other_layers = other_config.num_hidden_layers
                flops = (prefill_flops(other_config, other_layers, PREFILL_TOKENS)
                         + 2.0 * mixed_batch * decode_bytes(other_config, other_layers, 0, 0, 1)
                         + 4.0 * mixed_batch * other_layers * other_config.q_proj_size * args.context)
                result["points"][f"mixed_b{mixed_batch}_prompt{PREFILL_TOKENS}_{other}"] = round(
                    (mixed_batch + PREFILL_TOKENS) / run["step_seconds"], 1)
                further[f"mixed_b{mixed_batch}_prompt{PREFILL_TOKENS}_{other}"] = {
                    "model": f"{other_name} shape", "ms_per_step": round(run["step_seconds"] * 1e3, 3),
                    "flops_frac": round(flops / run["step_seconds"] / PEAK_FLOPS[dtype_key], 4)}
            del other_model
        result["further"] = further
    if not args.no_points:
        # What a kernel that only reads gets from this device's memory: the decode step's practical ceiling.
        probe = run_hbm_read(launches=10)
        result["roofline"]["read_probe"] = probe["best"]
        result["roofline"]["frac_of_read_probe"] = round(achieved / probe["best"], 4)
    result["hw"] = brief()
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
