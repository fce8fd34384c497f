"""Command line in the reference's manner (src/turboserve/cli.py:43-95,
src/turboserve/engine/runtime/engine.py:515-641)::

    turboserve [--log-level L] engine generate PROMPT... --model DIR [options]
    turboserve engine kv-size --model DIR [options]
    turboserve engine random-model --config FILE --out DIR --seed N
    turboserve engine replay --model DIR --dtype D --out DIR --max-tokens N    (bin/trace_run's arguments)
    turboserve engine bench [bench.py's arguments]
    turboserve version | hwinfo [--indent N]

Option names, defaults and meanings are the reference's where it has them (``--max-tokens 64``,
``--temperature 0`` = greedy, ``--max-num-seqs 8`` for ``generate`` and 64 for ``kv-size``,
...).  Added here: ``--prompt-ids`` (prompts as comma-separated token ids, so no tokenizer is
needed), ``--top-k``, ``--repetition-penalty`` and the ``random-model``, ``replay`` and ``bench``
commands (the last two hand their arguments to the trace replay program and to ``bench.py`` in
the checkout, which stay programs of their own as well).  The
reference's ``--offline`` and ``--no-prefix-caching`` are accepted and change nothing (there is
no download and no prefix cache); ``--prefix-caching`` is refused with that reason.
"""

from __future__ import annotations

import argparse
import json
import logging
import os
import sys
import time


def _add_engine_options(p: argparse.ArgumentParser, *, max_num_seqs: int) -> None:
    p.add_argument("--model", "-m", default=os.environ.get("TURBOSERVE_MODEL", ""), help="model folder (config.json + safetensors)")
    p.add_argument("--device", default="auto", help="auto or cuda[:N]")
    p.add_argument("--dtype", default="auto", help="auto, bfloat16 or float32")
    p.add_argument("--block-size", type=int, default=16)
    p.add_argument("--max-num-seqs", type=int, default=max_num_seqs)
    p.add_argument("--max-num-batched-tokens", type=int, default=2048)
    p.add_argument("--offline", action="store_true", help="accepted for the reference's command lines: nothing is ever downloaded")
    p.add_argument("--prefix-caching", dest="prefix_caching", action="store_true",
                   help="refused: this engine has no prefix cache")
    p.add_argument("--no-prefix-caching", dest="prefix_caching", action="store_false", help="accepted: the only mode")
    p.set_defaults(prefix_caching=False)
    p.add_argument("--tune-gemm", action="store_true",
                   help="time the BLAS library's kernels for a full step of prompt tokens at start-up and keep the fastest")
    p.add_argument("--tune-gemm-step-sizes", action="store_true",
                   help="run every step's BLAS products at one of a few sizes and time the library's kernels at all of them "
                        "at start-up (a minute or two the first time; kept in a per-user file)")
    p.add_argument("--run-ahead", dest="run_ahead", action="store_true",
                   help="launch each decode step before the host has read the tokens of the step before it (the default)")
    p.add_argument("--no-run-ahead", dest="run_ahead", action="store_false",
                   help="read every step's tokens before the next step is scheduled, as the reference does")
    p.set_defaults(run_ahead=True)


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="turboserve", description="Qwen2 inference engine for one MI355X.")
    parser.add_argument("--log-level", default=os.environ.get("TURBOSERVE_LOG_LEVEL", "INFO"))
    top = parser.add_subparsers(dest="command", required=True)
    top.add_parser("version", help="print the version")
    hw = top.add_parser("hwinfo", help="print the hardware and software record")
    hw.add_argument("--indent", type=int, default=2)

    engine = top.add_parser("engine", help="run the engine directly").add_subparsers(dest="engine_command", required=True)
    gen = engine.add_parser("generate", help="complete one or more prompts and print the results")
    gen.add_argument("prompt", nargs="*", help="text prompts (need a tokenizer.json in the model folder)")
    gen.add_argument("--prompt-ids", action="append", default=[], help="a prompt as comma-separated token ids; repeatable")
    _add_engine_options(gen, max_num_seqs=8)
    gen.add_argument("--max-tokens", type=int, default=64)
    gen.add_argument("--temperature", type=float, default=0.0)
    gen.add_argument("--top-p", type=float, default=1.0)
    gen.add_argument("--top-k", type=int, default=0)
    gen.add_argument("--repetition-penalty", type=float, default=1.0)
    gen.add_argument("--seed", type=int, default=None, help="seed for stochastic sampling")
    gen.add_argument("--num-blocks", type=int, default=None, help="explicit cache pool size; skips memory sizing")
    gen.add_argument("--ignore-eos", action="store_true")
    gen.add_argument("--stats", dest="stats", action="store_true")
    gen.add_argument("--no-stats", dest="stats", action="store_false")
    gen.set_defaults(stats=False)

    kv = engine.add_parser("kv-size", help="report how many cache blocks a configuration would get, and why")
    _add_engine_options(kv, max_num_seqs=64)
    kv.add_argument("--gpu-memory-utilization", type=float, default=0.9)
    kv.add_argument("--max-model-len", type=int, default=None)

    rnd = engine.add_parser("random-model", help="write a model folder with random weights from a config.json")
    rnd.add_argument("--config", required=True, help="a config.json")
    rnd.add_argument("--out", required=True)
    rnd.add_argument("--seed", type=int, default=0)
    rnd.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])

    replay = engine.add_parser("replay", add_help=False,
                               help="feed given token ids through a model step by step and write logits (bin/trace_run)")
    replay.set_defaults(passes_on=True)  # everything behind the command's name goes to that program's own parser
    bench = engine.add_parser("bench", add_help=False, help="the measurements of bench.py in the checkout")
    bench.set_defaults(passes_on=True)
    return parser


def _generate(args: argparse.Namespace) -> int:
    from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
    from turboserve_amd.engine.llm_engine import LLMEngine
    from turboserve_amd.sampling.params import SamplingParams

    prompts: list = list(args.prompt) + [[int(t) for t in ids.split(",") if t.strip()] for ids in args.prompt_ids]
    if not prompts:
        print("no prompt given", file=sys.stderr)
        return 2
    if not args.model:
        print("--model is required", file=sys.stderr)
        return 2
    config = EngineConfig(
        model=args.model, device=args.device, dtype=args.dtype, seed=args.seed,
        tune_gemm_tokens=(args.max_num_batched_tokens,) if args.tune_gemm else (),
        tune_gemm_step_sizes=getattr(args, "tune_gemm_step_sizes", False),
        run_ahead=getattr(args, "run_ahead", True),
        scheduler=SchedulerConfig(
            max_num_seqs=args.max_num_seqs, max_num_batched_tokens=args.max_num_batched_tokens,
            block_size=args.block_size, num_blocks=args.num_blocks, enable_prefix_caching=args.prefix_caching,
        ),
    )
    sampling = SamplingParams(
        max_tokens=args.max_tokens, temperature=args.temperature, top_p=args.top_p, top_k=args.top_k,
        repetition_penalty=args.repetition_penalty, seed=args.seed, ignore_eos=args.ignore_eos,
    )
    with LLMEngine(config) as engine:
        started = time.perf_counter()
        outputs = engine.generate(prompts, sampling)
        elapsed = time.perf_counter() - started
        for index, output in enumerate(outputs):
            print(f"prompt {index}: {prompts[index]}")
            shown = output.text_delta if engine.tokenizer is not None else output.new_token_ids
            print(f"output {index}: {shown}")
            print(f"  {output.output_tokens} tokens, finish_reason={output.finish_reason}")
        print(f"{len(outputs)} completions in {elapsed:.2f}s")
        if args.stats:
            print(json.dumps(engine.stats(), indent=2))
    return 0


def _kv_size(args: argparse.Namespace) -> int:
    import torch

    from turboserve_amd.cache.layout import CacheLayout
    from turboserve_amd.cache.sizing import activation_headroom_bytes, size_cache
    from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
    from turboserve_amd.config.model_config import read_config_json
    from turboserve_amd.weights.random_init import describe_model

    config = EngineConfig(
        model=args.model, device=args.device, dtype=args.dtype,
        gpu_memory_utilization=args.gpu_memory_utilization, max_model_len=args.max_model_len,
        scheduler=SchedulerConfig(
            max_num_seqs=args.max_num_seqs, max_num_batched_tokens=args.max_num_batched_tokens,
            block_size=args.block_size, enable_prefix_caching=args.prefix_caching,
        ),
    )
    _, model = describe_model(read_config_json(config.model))
    itemsize = 2 if config.resolved_dtype() == "bfloat16" else 4
    activation = activation_headroom_bytes(model, config.scheduler, itemsize)
    if not torch.cuda.is_available():
        print("no GPU is visible: the sizing needs the device's memory", file=sys.stderr)
        return 1
    sizing = size_cache(
        CacheLayout.from_model(model), config.scheduler, itemsize=itemsize, activation_bytes=activation,
        gpu_memory_utilization=config.gpu_memory_utilization, max_model_len=config.max_model_len,
        device=config.resolved_device(),
    )
    print(json.dumps(sizing.to_dict(), indent=2))
    return 0


def _random_model(args: argparse.Namespace) -> int:
    import torch

    from turboserve_amd.weights.random_init import write_random_model

    with open(args.config, encoding="utf-8") as handle:
        data = json.load(handle)
    dtype = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    print(write_random_model(data, args.out, seed=args.seed, dtype=dtype))
    return 0


def _bench(rest: list[str]) -> int:
    """``bench.py`` of the checkout this package lies in, with the given arguments."""
    import importlib.util
    from pathlib import Path

    path = Path(__file__).resolve().parent.parent / "bench.py"
    if not path.is_file():
        print(f"no bench.py beside the package ({path}): the measurements live in the checkout", file=sys.stderr)
        return 2
    spec = importlib.util.spec_from_file_location("turboserve_bench", path)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return int(module.main(rest) or 0)


def main(argv: list[str] | None = None) -> int:
    parser = build_parser()
    args, rest = parser.parse_known_args(argv)
    if rest and not getattr(args, "passes_on", False):
        parser.error("unrecognized arguments: " + " ".join(rest))
    logging.basicConfig(level=getattr(logging, str(args.log_level).upper(), logging.INFO),
                        format="%(asctime)s %(levelname)s %(name)s: %(message)s")
    if args.command == "version":
        from turboserve_amd import __version__

        print(f"turboserve_amd {__version__}")
        return 0
    if args.command == "hwinfo":
        from turboserve_amd.hwinfo import collect

        print(json.dumps(collect(), indent=args.indent or None, sort_keys=True))
        return 0
    if args.engine_command == "generate":
        return _generate(args)
    if args.engine_command == "kv-size":
        return _kv_size(args)
    if args.engine_command == "replay":
        from turboserve_amd.engine.replay import main as replay_main

        return replay_main(rest)
    if args.engine_command == "bench":
        return _bench(rest)
    return _random_model(args)


if __name__ == "__main__":  # pragma: no cover
    sys.exit(main())
