#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at the Qwen2.5-7B layer sizes on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one decode step of the whole engine path: the step function over a batch of
single tokens against the paged cache, logits, greedy sampling, tokens back on the host.  As
in the engine's own loop a step is launched before the host has read the tokens of the step
before it (its token ids are copied from the sampler's result on the device); every step's
tokens are read, one step later, and the clock stops after the last are.
The default run has the Qwen2.5-7B layer sizes (the benchmark's named configuration), random weights
(N(0, 0.02), norm gains 1), a batch of 8 requests each holding a context of 8,192 tokens
(cache filled with random keys and values; what is timed is real decode steps on top of it).
One JSON line is printed: ``value`` is decoded tokens a second; ``prefill`` times one
2,048-token prompt; ``roofline`` prices the decode step against HBM bandwidth; ``points``
holds decode at batch 1 and 64.  The prefill's projections are BLAS-library products; which
of the library's kernels runs each is timed once before the measurement
(``--no-gemm-tuning`` leaves it to the library's heuristic).  Peaks are the published MI355X
figures: HBM 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s, fp32 157.3 TFLOP/s.
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
PREFILL_TOKENS = 2048
PAGE = 16


def parse_args() -> argparse.Namespace:
    p = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=64)
    p.add_argument("--warmup", type=int, default=40,
                   help="untimed steps first; the clocks take some tens of milliseconds of load to settle")
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--context", type=int, default=CONTEXT)
    p.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (named in config)")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64")
    p.add_argument("--no-prefill", action="store_true")
    p.add_argument("--no-gemm-tuning", action="store_true",
                   help="leave the choice of the BLAS library's prefill kernels to its heuristic")
    p.add_argument("--only-prefill", action="store_true", help="run the 2,048-token prefill alone (for profiling)")
    p.add_argument("--shape", default="7b", choices=sorted(SHAPES), help="layer sizes (the default run is 7b)")
    p.add_argument("--fill-hbm", action="store_true",
                   help="size the cache pool to the free device memory and interleave the requests' pages in it")
    p.add_argument("--mixed-prefill", type=int, default=0, metavar="N",
                   help="time steps that hold the batch's decode tokens and one N-token portion of a prompt")
    return p.parse_args()


class DecodeBench:
    """Requests with a given context already in the cache, decoded one token per step through
    the engine's own cache manager, step function and sampler."""

    def __init__(self, model, config, batch: int, context: int, steps_total: int, *, fill_hbm: bool = False,
                 extra_tokens: int = 0) -> None:
        import torch

        from turboserve_amd.cache.manager import CacheManager
        from turboserve_amd.engine.loading import build_storage
        from turboserve_amd.engine.runner import ModelRunner
        from turboserve_amd.sampling.sampler import Sampler

        self.torch = torch
        self.batch = batch
        self.context = context
        self.vocab_size = config.vocab_size
        pages_per_request = -(-(context + steps_total + 1) // PAGE)
        num_pages = batch * pages_per_request + -(-extra_tokens // PAGE)
        if fill_hbm:
            # As many pages as 90% of what is free holds (at least what the requests need).
            free, _ = torch.cuda.mem_get_info()
            page_bytes = config.kv_bytes_per_token(model.runtime.dtype) * PAGE
            num_pages = max(num_pages, int(free * 0.9) // page_bytes)
        self.num_pages = num_pages
        self.storage = build_storage(model, num_pages, PAGE, batch + 1)
        for pages in self.storage.pages:
            for member in pages:  # piecewise: a 200 GB pool is not filled in one launch's temporaries
                member.normal_(0.0, 0.5)
        self.manager = CacheManager(self.storage.layout.windows(), num_pages, PAGE, batch + 1)
        self.runner = ModelRunner(model, self.storage, check=False)
        self.sampler = Sampler(model.runtime.ops)
        self.pending = None  # the sampler's result of a step whose tokens have not been read yet
        generator = torch.Generator().manual_seed(1234)
        self.tokens = torch.randint(0, config.vocab_size, (batch,), generator=generator).tolist()
        self.portion = torch.randint(0, config.vocab_size, (max(extra_tokens, 1),), generator=generator).tolist()
        for request in range(batch):
            self.manager.admit(request)
        if fill_hbm:
            # Page by page in turn, as requests that grow together get them: interleaved tables.
            remaining = [context - 1] * batch
            while any(remaining):
                for request in range(batch):
                    take = min(PAGE, remaining[request])
                    if take:
                        self.manager.append(request, take)
                        remaining[request] -= take
        else:
            for request in range(batch):
                self.manager.append(request, context - 1)  # the context's last token is decoded below

    def step(self, portion_tokens: int = 0) -> None:
        """One decode step of the batch; with ``portion_tokens`` the step also holds the first
        portion, that long, of a new request's prompt (its pages are given back afterwards)."""
        from turboserve_amd.engine.batch import StepEntry
        from turboserve_amd.sampling.params import SamplingParams

        entries = []
        if portion_tokens:
            held = self.manager.admit("portion")
            slots = self.manager.append("portion", portion_tokens)
            entries.append(StepEntry(request="portion", tokens=self.portion[:portion_tokens], start=0,
                                     tables=held.tables, slots=slots, state_slot=held.state_slot, want=[]))
        for request in range(self.batch):
            held = self.manager.get(request)
            start = held.num_tokens
            slots = self.manager.append(request, 1)
            entries.append(StepEntry(request=request, tokens=[self.tokens[request]], start=start,
                                     tables=held.tables, slots=slots, state_slot=held.state_slot, want=[0]))
        greedy = SamplingParams(temperature=0.0)
        if portion_tokens or not self.runner.takes_tokens_from(self.batch):
            # A step with a portion of a prompt does not replay as a graph: its tokens are read
            # before the next step is built, as the engine does for such steps.
            self.finish()
            logits = self.runner.step(entries)
            out = self.sampler.sample(logits, [greedy] * self.batch, [0] * self.batch, [0] * self.batch)
            self.tokens = out.token_ids
        else:
            # As the engine's loop does (LLMEngine._run_ahead): the step is launched with its token
            # ids taken on the device from what the step before sampled, and that step's tokens
            # are read only afterwards, so the GPU does not wait while the host builds a step.
            before = self.pending
            if before is not None:
                for entry in entries:
                    entry.tokens = [-1]
                logits = self.runner.step(entries, tokens_from=(before.tokens, {i: i for i in range(self.batch)}))
            else:
                logits = self.runner.step(entries)
            self.pending = self.sampler.launch(logits, [greedy] * self.batch, [0] * self.batch, [0] * self.batch)
            if before is not None:
                self.tokens = before.read().token_ids
        if portion_tokens:
            self.manager.free("portion")

    def finish(self) -> None:
        """Read the tokens of the step that is still in flight, if one is."""
        if self.pending is not None:
            self.tokens = self.pending.read().token_ids
            self.pending = None

    def run(self, steps: int, warmup: int, portion_tokens: int = 0) -> float:
        """Seconds for ``steps`` steps after ``warmup`` untimed ones."""
        torch = self.torch
        for _ in range(warmup):
            self.step(portion_tokens)
        self.finish()
        torch.cuda.synchronize()
        started = time.perf_counter()
        for _ in range(steps):
            self.step(portion_tokens)
        self.finish()
        torch.cuda.synchronize()
        return time.perf_counter() - started

    def close(self) -> None:
        self.runner.release()
        self.storage = None
        self.torch.cuda.empty_cache()


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


def run_prefill(model, config, tokens: int, repeats: int = 3, tune: bool = True) -> float:
    """Seconds (best of ``repeats``) for one step over a ``tokens``-long prompt, to its last
    position's logits on the host.  With ``tune`` the BLAS library's kernels for the step's
    products are timed first in a dry step and the fastest kept, as an engine started with
    ``tune_gemm_tokens`` does."""
    import torch

    from turboserve_amd.cache.manager import CacheManager
    from turboserve_amd.engine.batch import StepEntry
    from turboserve_amd.engine.loading import build_storage
    from turboserve_amd.engine.runner import ModelRunner

    num_pages = -(-tokens // PAGE)
    storage = build_storage(model, num_pages, PAGE, 1)
    manager = CacheManager(storage.layout.windows(), num_pages, PAGE, 1)
    runner = ModelRunner(model, storage, check=False)
    if tune and model.runtime.dtype == torch.bfloat16:
        from turboserve_amd.kernels.gemm_tuning import LibraryGemmTuning

        with LibraryGemmTuning(os.path.join(tempfile.gettempdir(), f"turboserve_amd_bench_gemm_{os.getuid()}.csv")):
            runner.dry_run(tokens)
    generator = torch.Generator().manual_seed(4321)
    prompt = torch.randint(0, config.vocab_size, (tokens,), generator=generator).tolist()
    best = float("inf")
    for _ in range(repeats + 1):
        held = manager.admit("p")
        slots = manager.append("p", tokens)
        entry = StepEntry(request="p", tokens=prompt, start=0, tables=held.tables, slots=slots,
                          state_slot=held.state_slot, want=[tokens - 1])
        torch.cuda.synchronize()
        started = time.perf_counter()
        logits = runner.step([entry])
        logits.argmax(dim=-1).tolist()
        torch.cuda.synchronize()
        best = min(best, time.perf_counter() - started)
        manager.free("p")
    runner.release()
    del storage
    torch.cuda.empty_cache()
    return best


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine (single-GPU by design)")
        return 2
    import torch

    from turboserve_amd.engine.loading import build_model, make_runtime, resolve_run_dtype
    from turboserve_amd.hwinfo import collect
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

    pool_tokens = 0

    def decode_rate(batch: int, steps: int, warmup: int) -> tuple[float, float]:
        nonlocal pool_tokens
        bench = DecodeBench(model, config, batch, args.context, steps + warmup, fill_hbm=args.fill_hbm,
                            extra_tokens=args.mixed_prefill)
        pool_tokens = bench.num_pages * PAGE
        if args.mixed_prefill and not args.no_gemm_tuning and dtype == torch.bfloat16:
            from turboserve_amd.kernels.gemm_tuning import LibraryGemmTuning

            with LibraryGemmTuning(os.path.join(tempfile.gettempdir(), f"turboserve_amd_bench_gemm_{os.getuid()}.csv")):
                bench.runner.dry_run(args.mixed_prefill + batch)
        seconds = bench.run(steps, warmup, args.mixed_prefill)
        bench.close()
        return batch * steps / seconds, seconds / steps

    if args.only_prefill:
        seconds = run_prefill(model, config, PREFILL_TOKENS, tune=not args.no_gemm_tuning)
        print(json.dumps({"prefill_ms": round(seconds * 1e3, 3), "tokens": PREFILL_TOKENS, "layers": layers}))
        return 0

    value, step_seconds = decode_rate(args.batch, args.steps, args.warmup)
    if args.mixed_prefill:
        # A mixed step is priced by its products' flops, not by bytes: say what ran and stop there.
        flops = (prefill_flops(config, layers, args.mixed_prefill)
                 + 2.0 * args.batch * decode_bytes(config, layers, 0, 0, 1)  # every weight once per decode token
                 + 4.0 * args.batch * layers * config.q_proj_size * args.context)  # and its attention
        print(json.dumps({
            "metric": f"mixed step: {args.batch} decode tokens + one {args.mixed_prefill}-token prompt portion "
                      f"({shape_name} shape, one MI355X)",
            "value": round((args.batch + args.mixed_prefill) / step_seconds, 1), "unit": "tokens/s",
            "decode_tokens_per_s": round(value, 2), "ms_per_step": round(step_seconds * 1e3, 3),
            "steps": args.steps, "warmup": args.warmup, "dtype": dtype_key, "decode_context": args.context,
            "layers": layers, "kv_pool_tokens": pool_tokens,
            "flops_frac": round(flops / step_seconds / PEAK_FLOPS[dtype_key], 4),
        }))
        return 0
    mean_context = args.context + args.warmup + args.steps / 2
    read = decode_bytes(config, layers, args.batch, mean_context, itemsize)
    achieved = read / step_seconds / 1e9
    result = {
        "metric": f"decode tok/s ({shape_name} shape, paged cache, one MI355X)",
        "value": round(value, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_seconds * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype_key,
        "data": "synthetic: random weights N(0,0.02), uniform-random token ids, cache pre-filled with random keys/values",
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
            "kv_pool_tokens": pool_tokens,
            "prefill_tokens": PREFILL_TOKENS,
            "prefill_gemm_choice": "library heuristic" if args.no_gemm_tuning else "library candidates timed at start-up",
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
        seconds = run_prefill(model, config, PREFILL_TOKENS, tune=not args.no_gemm_tuning)
        flops = prefill_flops(config, layers, PREFILL_TOKENS)
        result["prefill"] = {
            "value": round(PREFILL_TOKENS / seconds, 1),
            "tokens": PREFILL_TOKENS,
            "ms": round(seconds * 1e3, 3),
            "frac": round(flops / seconds / PEAK_FLOPS[dtype_key], 4),
        }
    if not args.no_points:
        points = {}
        for batch in (1, 64):
            rate, _ = decode_rate(batch, max(8, args.steps // 2), max(2, args.warmup // 2))
            points[f"decode_b{batch}"] = round(rate, 2)
        result["points"] = points
    info = collect()
    result["hw"] = {"gpu": info["gpu_name"], "torch": info["torch"]["version"], "hip": info["torch"]["hip_version"],
                    "git": (info["git"]["sha"] or "")[:12]}
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
