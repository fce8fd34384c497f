"""Replay on the GPU against the plain implementation: every way of cutting the same requests
(whole, a long prefix then token by token, portions of changing size, mixed with other
requests on so few pages that they are used again), in true 32-bit and in bfloat16."""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import pytest
import torch

import tiny
import trace_helpers as th
from plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parent.parent

#: 32-bit engine against the 32-bit plain implementation: both are exact up to the order of
#: additions (the reference allows 1e-4 against its oracle, tests/unit/test_model_parity.py:181).
ATOL_F32 = 1e-4
#: Between two cuttings of the same request in 32-bit (test_model_parity.py:246).
ATOL_F32_CUTS = 1e-5
#: bfloat16 engine against the plain implementation run in 32-bit on the same (bfloat16-valued)
#: weights: activations are rounded to 8 bits of mantissa once per op, so the bound is relative
#: to the largest logit (the reference uses 1e-2 for its half-precision kernel,
#: tests/gpu/test_triton_attention.py:117).
RTOL_BF16 = 2e-2


def lengths_for(name: str) -> list[int]:
    return {"A": [5, 17, 33, 70, 50], "B": [1, 9, 24, 40, 75, 66], "C": [3, 45, 97, 130, 64]}[name]


@pytest.fixture(scope="module", params=["A", "B", "C"])
def case(request, tmp_path_factory):
    name = request.param
    config, seed, page = tiny.TINY[name]
    folders = {}
    for dtype_name, dtype in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        folders[dtype_name] = tiny.make_model_dir(tmp_path_factory.mktemp(f"tiny{name}_{dtype_name}"), config, seed, dtype,
                                                  std=tiny.WIDE_STD if dtype == torch.float32 else 0.02)
    requests = {f"r{i}": tiny.random_tokens(config["vocab_size"], n, 100 + i) for i, n in enumerate(lengths_for(name))}
    expected = {d: {rid: tiny.plain_logits(folders[d], toks) for rid, toks in requests.items()} for d in folders}
    return {"name": name, "page": page, "folders": folders, "requests": requests, "expected": expected}


def run_trace(folder: Path, dtype: str, page: int, steps: list[dict], max_tokens: int | None = None):
    from turboserve_amd.engine.replay import TraceReplayer

    replayer = TraceReplayer(folder, dtype=dtype, max_tokens=max_tokens or th.peak_tokens(steps), page_size=page)
    outputs = {}
    for record in steps:
        logits = replayer.run_step(record)
        if logits.shape[0]:
            outputs[record["step"]] = logits.float().cpu()
    replayer.manager.check_invariants()
    assert all(pool.num_in_use == 0 for pool in replayer.manager.pools), "pages were not given back"
    return outputs


def check(got: dict[str, torch.Tensor], expected: dict[str, torch.Tensor], dtype: str, what: str) -> None:
    for rid, want in expected.items():
        diff = (got[rid] - want).abs()
        scale = float(want.abs().max())
        worst = float(diff.max())
        bound = ATOL_F32 if dtype == "float32" else RTOL_BF16 * scale
        if worst > bound:
            row = int(diff.max(dim=1).values.argmax())
            first = int((diff.max(dim=1).values > bound).nonzero()[0])
            raise AssertionError(
                f"{what} {dtype} request {rid}: max |diff| {worst:.3e} > {bound:.3e} (logit scale {scale:.3f}); "
                f"worst position {row}, first wrong position {first} of {want.shape[0]}"
            )


CUTS = {
    "whole": lambda reqs: th.whole(reqs),
    "prefix_then_single": lambda reqs: th.prefix_then_single(reqs, 32),
    "portions": lambda reqs: th.portions(reqs, [7, 5, 3, 2, 2, 11, 4]),
    "mixed": lambda reqs: th.mixed(reqs, [7, 2, 13, 3, 5], max_live=4, decode_tail=6),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", list(CUTS))
def test_replay_matches_plain(case, dtype, cut):
    steps = CUTS[cut](case["requests"])
    outputs = run_trace(case["folders"][dtype], dtype, case["page"], steps)
    got = th.collect(steps, outputs, case["requests"])
    check(got, case["expected"][dtype], dtype, f"tiny {case['name']} {cut}")


def test_cuttings_agree_in_float32(case):
    """Logits at a position do not depend on how the tokens were cut into steps."""
    results = {}
    for cut, make in CUTS.items():
        steps = make(case["requests"])
        results[cut] = th.collect(steps, run_trace(case["folders"]["float32"], "float32", case["page"], steps), case["requests"])
    for cut, got in results.items():
        for rid, ref in results["whole"].items():
            worst = float((got[rid] - ref).abs().max())
            assert worst <= ATOL_F32_CUTS, f"tiny {case['name']} {cut} vs whole, request {rid}: {worst:.3e}"


def test_mixed_reuses_pages(case):
    """The mixed trace runs on a pool so small that finished requests' pages go to later ones."""
    steps = CUTS["mixed"](case["requests"])
    total = sum(-(-len(t) // 64) * 64 for t in case["requests"].values())
    assert th.peak_tokens(steps) < total


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(case, dtype, tmp_path):
    """The program itself: JSON lines on stdin, ``done <step>`` lines on stdout, .f32 files."""
    if case["name"] != "B":
        pytest.skip("one configuration is enough for the subprocess test")
    steps = CUTS["mixed"](case["requests"])
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(case["folders"][dtype]), "--dtype", dtype,
         "--out", str(out), "--max-tokens", str(th.peak_tokens(steps)), "--page-size", str(case["page"])],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600,
    )
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [line for line in proc.stdout.splitlines() if line.startswith("done ")] == [f"done {s['step']}" for s in steps]
    vocab = tiny.TINY[case["name"]][0]["vocab_size"]
    outputs = {}
    for record in steps:
        wanted = sum(len(e["want"]) for e in record["entries"])
        path = out / f"{record['step']}.f32"
        if wanted:
            import numpy as np

            outputs[record["step"]] = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(wanted, vocab).copy())
        else:
            assert not path.exists()
    check(th.collect(steps, outputs, case["requests"]), case["expected"][dtype], dtype, "trace_run mixed")


@pytest.mark.parametrize("trial", range(10))
def test_random_configurations_replay_like_plain(trial, tmp_path):
    """Seeded random configurations beyond the three fixed ones: head sizes that are and are not
    multiples of 16 or 32, one to sixteen query heads per KV head (every attention kernel variant),
    page sizes 8 to 64, windows, tied and untied heads; mixed and portion-wise cutting, both dtypes."""
    import random

    rng = random.Random(9000 + trial)
    kv_heads = rng.choice([1, 1, 2, 3, 4])
    group = rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 16])
    heads = kv_heads * group if kv_heads * group <= 32 else kv_heads * (32 // kv_heads)
    window = rng.choice([None, None, 12, 33, 70])
    config = {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": rng.choice([64, 72, 96, 136, 200]),
        "num_hidden_layers": rng.choice([1, 2, 3]), "num_attention_heads": heads, "num_key_value_heads": kv_heads,
        "head_dim": rng.choice([16, 32, 48, 64, 80, 96, 128, 256, 24, 40]),
        "intermediate_size": rng.choice([64, 104, 200, 264]), "vocab_size": rng.choice([97, 256, 1000, 5003]),
        "rope_theta": rng.choice([1e4, 1e6]), "rms_norm_eps": rng.choice([1e-6, 1e-5]),
        "tie_word_embeddings": rng.random() < 0.5, "use_sliding_window": window is not None,
        "max_position_embeddings": 512,
    }
    if window is not None:
        config["sliding_window"] = window
        config["max_window_layers"] = rng.choice([0, 1])
    page = rng.choice([8, 16, 32, 64])
    lengths = [rng.choice([3, 17, 40, 75, 130, 200]) for _ in range(rng.choice([2, 3, 5]))]
    folder = tiny.make_model_dir(tmp_path, config, trial, torch.float32)
    raw, tensors = tiny.read_model_dir(folder)
    requests = {f"r{i}": tiny.random_tokens(config["vocab_size"], n, 500 + i) for i, n in enumerate(lengths)}
    expected = {rid: plain.forward_logits(raw, plain.as_float32(tensors), toks) for rid, toks in requests.items()}
    for cut in ("mixed", "portions"):
        steps = CUTS[cut](requests)
        for dtype in ("float32", "bfloat16"):
            got = th.collect(steps, run_trace(folder, dtype, page, steps), requests)
            check(got, expected, dtype, f"trial {trial} {config} page {page} {cut}")


def test_7b_layer_sizes_float32_and_bfloat16_paths_agree():
    """Two layers of the Qwen2.5-7B sizes (hidden 3584, 28 heads on 4 KV heads of 128, 18944
    wide, 152064 tokens) holding the same bfloat16-rounded random weights, stepped by the
    32-bit path (its own product and attention kernels) and by the bfloat16 path (skinny and
    library products, matrix-core attention): a 300- and a 77-token prompt in one step, then
    four decode steps of both.  The logits agree to bfloat16 accuracy and pick the same token."""
    from turboserve_amd.cache.manager import CacheManager
    from turboserve_amd.engine.batch import StepEntry
    from turboserve_amd.engine.loading import build_model, build_storage, make_runtime
    from turboserve_amd.engine.runner import ModelRunner

    shape = {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": 3584, "num_hidden_layers": 2,
        "num_attention_heads": 28, "num_key_value_heads": 4, "head_dim": 128, "intermediate_size": 18944,
        "vocab_size": 152064, "rope_theta": 1e6, "rms_norm_eps": 1e-6, "tie_word_embeddings": False,
        "max_position_embeddings": 32768,
    }
    generator = torch.Generator().manual_seed(5)
    requests = {name: torch.randint(0, shape["vocab_size"], (n,), generator=generator).tolist()
                for name, n in (("a", 300), ("b", 77))}
    logits = {}
    for dtype in (torch.float32, torch.bfloat16):
        runtime = make_runtime(dtype, "cuda:0")
        _, model = build_model(shape, runtime)
        draw = torch.Generator(device="cuda:0")
        draw.manual_seed(3)
        tensors = {}
        for name, spec in model.tensor_specs().items():
            if spec.init == "ones":
                values = torch.ones(spec.shape, device="cuda:0")
            else:
                values = torch.empty(spec.shape, device="cuda:0").normal_(0.0, 0.02, generator=draw)
            tensors[name] = values.bfloat16().to(dtype)  # the same numbers in both runs
        model.load(tensors)
        del tensors
        storage = build_storage(model, 64, 16, 4)
        manager = CacheManager(storage.layout.windows(), 64, 16, 4)
        runner = ModelRunner(model, storage)
        rows = []
        entries = []
        for name, tokens in requests.items():
            held = manager.admit(name)
            slots = manager.append(name, len(tokens) - 4)
            entries.append(StepEntry(request=name, tokens=tokens[:-4], start=0, tables=held.tables, slots=slots,
                                     state_slot=held.state_slot, want=[len(tokens) - 5]))
        rows.append(runner.step(entries).float().cpu())
        for k in range(4):
            entries = []
            for name, tokens in requests.items():
                held = manager.get(name)
                start = held.num_tokens
                slots = manager.append(name, 1)
                entries.append(StepEntry(request=name, tokens=[tokens[len(tokens) - 4 + k]], start=start,
                                         tables=held.tables, slots=slots, state_slot=held.state_slot, want=[0]))
            rows.append(runner.step(entries).float().cpu())
        logits[dtype] = torch.cat(rows)
        runner.release()
        del model, storage, runner
        torch.cuda.empty_cache()
    exact, fast = logits[torch.float32], logits[torch.bfloat16]
    assert exact.shape == (10, shape["vocab_size"])
    assert float((exact - fast).abs().max()) <= RTOL_BF16 * float(exact.abs().max())
    assert torch.equal(exact.argmax(-1), fast.argmax(-1))
