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
#: weights: activations are rounded to 8 bits of mantissa once per op, so the bound is relative,
#: row by row, to the largest logit of that position (the reference uses 1e-2 for its
#: half-precision kernel, tests/gpu/test_triton_attention.py:117).  Both precisions run models
#: with a wide spread of weights (``tiny.std_for``), in which every layer and every cached key
#: matters to the logits: ``test_a_fault_in_the_last_layers_cache_is_seen`` shows that a fault in
#: one layer's cache exceeds these bounds more than tenfold.  Measured on these models: up to
#: 1.6% (``tiny.BF16_STD`` has the figures, also for the reference's own formulas in bfloat16).
RTOL_BF16 = 2e-2
#: The same for steps of more than 128 rows, whose projections the BLAS library computes: it
#: rounds the q|k|v and gate|up projections to bfloat16 where this engine's own products hand
#: 32-bit sums to their consumers, so such a step carries more rounding: 140 short requests as
#: one step are off by up to 2.3% where each alone is off by up to 1.7% (mean 0.6%), and the
#: reference's own formulas in bfloat16 by up to 2.8%.  A fault moves the logits by 24% or more.
RTOL_BF16_LIBRARY = 3e-2


def lengths_for(name: str) -> list[int]:
    return {"A": [5, 17, 33, 70, 50], "B": [1, 9, 24, 40, 75, 66], "C": [3, 45, 97, 130, 64], "D": [2, 31, 80, 49, 112]}[name]


@pytest.fixture(scope="module", params=["A", "B", "C", "D"])
def case(request, tmp_path_factory):
    name = request.param
    config, seed, page = tiny.TINY[name]
    folders = {}
    for dtype_name, dtype in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        folders[dtype_name] = tiny.make_model_dir(tmp_path_factory.mktemp(f"tiny{name}_{dtype_name}"), config, seed, dtype,
                                                  std=tiny.std_for(dtype, config["hidden_size"]))
    requests = {f"r{i}": tiny.random_tokens(config["vocab_size"], n, 100 + i) for i, n in enumerate(lengths_for(name))}
    expected = {d: {rid: tiny.plain_logits(folders[d], toks) for rid, toks in requests.items()} for d in folders}
    return {"name": name, "page": page, "folders": folders, "requests": requests, "expected": expected}


def run_trace(folder: Path, dtype: str, page: int, steps: list[dict], max_tokens: int | None = None):
    from turboserve_amd.engine.replay import TraceReplayer

    # The pool is what the trace needs at its peak counted in whole pages (the program's own
    # rounding to 64 tokens comes on top), so that pages run out and are used again.
    replayer = TraceReplayer(folder, dtype=dtype, max_tokens=max_tokens or th.peak_tokens(steps, rounding=page), page_size=page)
    outputs = {}
    for record in steps:
        logits = replayer.run_step(record)
        if logits.shape[0]:
            outputs[record["step"]] = logits.float().cpu()
    replayer.manager.check_invariants()
    assert all(pool.num_in_use == 0 for pool in replayer.manager.pools), "pages were not given back"
    return outputs


def excess(got: torch.Tensor, want: torch.Tensor, dtype: str, rtol_bf16: float = RTOL_BF16) -> torch.Tensor:
    """Per position: the largest |difference| of its logits divided by the bound for that
    position (above 1: out of bounds).  32-bit: ``ATOL_F32`` times the size of the logits where
    that is above 1; bfloat16: ``rtol_bf16`` times the position's largest |logit|."""
    diff = (got - want).abs().max(dim=1).values
    scale = want.abs().max(dim=1).values
    bound = ATOL_F32 * scale.clamp(min=1.0) if dtype == "float32" else rtol_bf16 * scale
    return diff / bound


def check(got: dict[str, torch.Tensor], expected: dict[str, torch.Tensor], dtype: str, what: str,
          rtol_bf16: float = RTOL_BF16) -> None:
    for rid, want in expected.items():
        ratio = excess(got[rid], want, dtype, rtol_bf16)
        if float(ratio.max()) > 1.0:
            row = int(ratio.argmax())
            first = int((ratio > 1.0).nonzero()[0])
            raise AssertionError(
                f"{what} {dtype} request {rid}: position {row} is off by {float(ratio[row]):.2f} times its bound "
                f"(largest |logit| there {float(want[row].abs().max()):.3f}); first wrong position {first} of {want.shape[0]}"
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
    """The mixed trace runs on a pool so small that finished requests' pages go to later ones:
    in the run itself, some page id turns up in the block tables of two different requests."""
    from turboserve_amd.engine.replay import TraceReplayer

    steps = CUTS["mixed"](case["requests"])
    total = sum(-(-len(t) // 64) * 64 for t in case["requests"].values())
    assert th.peak_tokens(steps) < total
    replayer = TraceReplayer(case["folders"]["float32"], dtype="float32", max_tokens=th.peak_tokens(steps, rounding=case["page"]),
                             page_size=case["page"])
    holders: dict[tuple[int, int], set[str]] = {}
    for record in steps:
        live = [entry["id"] for entry in record["entries"]]
        replayer.run_step({**record, "end": []})
        for rid in live:
            for group, table in enumerate(replayer.manager.get(rid).tables):
                for page in table:
                    if page >= 0:
                        holders.setdefault((group, page), set()).add(rid)
        for rid in record["end"]:
            replayer.manager.free(rid)
    shared = [key for key, rids in holders.items() if len(rids) > 1]
    assert shared, "no page was handed to a second request"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_fault_in_the_last_layers_cache_is_seen(case, dtype):
    """The comparisons above would catch a fault in the cache of any one layer.  After a prompt
    of 64 tokens, in the LAST layer only, either the values of the request's last full page are
    lost (zeroed, as a block-table entry that points at a page never written would have it) or
    the values of its last two pages are swapped (the keys stay: a page misplaced for the values
    alone; the reference checks paging with reversed block ids, tests/unit/test_model_parity.py:
    249-274).  The eight tokens decoded after that miss their bounds more than tenfold for the
    lost page and more than fivefold for the swap, and without a fault they are inside them.
    (Swapping keys AND values of two pages a request sees in full must change nothing, and does
    not: attention does not depend on the order of its keys.)"""
    from turboserve_amd.engine.replay import TraceReplayer

    tokens = tiny.random_tokens(tiny.TINY[case["name"]][0]["vocab_size"], 72, 4242)
    want = tiny.plain_logits(case["folders"][dtype], tokens)[64:]
    worst = {}
    for fault in ("none", "lost", "swapped", "swapped with keys"):
        replayer = TraceReplayer(case["folders"][dtype], dtype=dtype, max_tokens=128, page_size=case["page"])
        replayer.run_step({"entries": [{"id": "r", "tokens": tokens[:64], "want": []}]})
        unit = replayer.storage.layout.entry_units[-1]
        assert unit[0] == "pages"
        _, group, member = unit
        table = replayer.manager.get("r").tables[group]
        a, b = table[64 // case["page"] - 2], table[64 // case["page"] - 1]
        assert a >= 0 and b >= 0 and a != b
        keys = replayer.storage.key_pages[group][member]  # [pages, kv heads, page x head size]
        values = replayer.storage.value_pages[group][member]
        if fault == "lost":
            values[b] = 0
        elif fault.startswith("swapped"):
            for pages in (keys, values) if fault.endswith("keys") else (values,):
                kept = pages[a].clone()
                pages[a] = pages[b]
                pages[b] = kept
        rows = [replayer.run_step({"entries": [{"id": "r", "tokens": [t], "want": [0]}]}).float().cpu() for t in tokens[64:]]
        worst[fault] = float(excess(torch.cat(rows), want, dtype).max())
    assert worst["none"] <= 1.0, f"the undisturbed run is off by {worst['none']:.2f} times its bound"
    assert worst["lost"] > 10.0, f"a lost page in the last layer moves the logits by only {worst['lost']:.2f} times the bound"
    assert worst["swapped"] > 5.0, f"swapped values in the last layer move the logits by only {worst['swapped']:.2f} times the bound"
    if replayer.storage.layout.groups[group].window is None:
        assert worst["swapped with keys"] <= 1.0, "the order of a request's pages should not matter when keys and values move together"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_portions_beside_more_single_tokens_than_a_recorded_step_takes(case, dtype):
    """Steps that hold 140 single tokens and portions of two prompts: a two-token portion, one
    that ends just past a page's edge, one that starts just before one.  More rows than a
    recorded step or the decode products take, so the decode attention runs without the
    device-side longest context beside the prefill attention, and the bfloat16 projections are
    the library's."""
    page = case["page"]
    vocab = tiny.TINY[case["name"]][0]["vocab_size"]
    many = {f"d{i}": tiny.random_tokens(vocab, 4 + i % 9, 6000 + i) for i in range(140)}
    long = {"p": tiny.random_tokens(vocab, 2 * page + 9, 6500), "q": tiny.random_tokens(vocab, page + 6, 6501)}
    requests = {**many, **long}
    steps: list[dict] = []
    names = list(many)
    for first in range(0, len(names), 35):  # the prompts of the many, 35 requests a step, all but their last two tokens
        steps.append({"step": len(steps), "end": [], "entries": [
            {"id": rid, "tokens": many[rid][:-2], "want": list(range(len(many[rid]) - 2))} for rid in names[first:first + 35]]})
    cuts = {"p": [(0, 2), (2, page + 1), (page + 1, 2 * page + 9)], "q": [(0, page + 3), (page + 3, page + 5), (page + 5, page + 6)]}
    for k in range(3):
        entries = []
        if k < 2:
            entries += [{"id": rid, "tokens": [many[rid][len(many[rid]) - 2 + k]], "want": [0]} for rid in names]
        for rid in ("q", "p") if k % 2 else ("p", "q"):
            lo, hi = cuts[rid][k]
            entries.insert(len(entries) // 2, {"id": rid, "tokens": long[rid][lo:hi], "want": list(range(hi - lo))})
        steps.append({"step": len(steps), "entries": entries, "end": names if k == 1 else (["p", "q"] if k == 2 else [])})
    from turboserve_amd.engine.replay import TraceReplayer

    replayer = TraceReplayer(case["folders"][dtype], dtype=dtype, max_tokens=th.peak_tokens(steps, rounding=max(64, page)),
                             page_size=page, max_live=len(requests))
    outputs = {}
    for record in steps:
        outputs[record["step"]] = replayer.run_step(record).float().cpu()
    if replayer.runner.graphs is not None:
        assert replayer.runner.graphs.num_replays == 0
    replayer.manager.check_invariants()
    raw, tensors = tiny.read_model_dir(case["folders"][dtype])
    expected = {rid: plain.forward_logits(raw, tensors, tokens) for rid, tokens in requests.items()}
    got = th.collect(steps, outputs, requests)
    check(got, expected, dtype, f"tiny {case['name']} portions beside 140 single tokens", RTOL_BF16_LIBRARY)
    # ... and all but a few positions inside the bound of the engine's own products
    ratios = torch.cat([excess(got[rid], want, dtype) for rid, want in expected.items()])
    assert float((ratios > 1.0).float().mean()) <= 0.005, f"{int((ratios > 1.0).sum())} of {ratios.numel()} positions"


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
def test_random_configurations_replay_like_plain(trial, tmp_path, monkeypatch):
    """Seeded random configurations beyond the three fixed ones: head sizes that are and are not
    multiples of 16 or 32, one to sixteen query heads per KV head (every attention kernel variant),
    page sizes 8 to 64, windows, tied and untied heads; mixed and portion-wise cutting, both dtypes.
    Every other trial shares out the keys of every attention block that has two windows of keys
    or more (serving does so only for long contexts)."""
    import random

    from turboserve_amd.kernels.ops import Ops

    if trial % 2:
        monkeypatch.setattr(Ops, "prefill_share_min_windows", 1)
        monkeypatch.setattr(Ops, "prefill_share_combine_cost", 0)

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
    requests = {f"r{i}": tiny.random_tokens(config["vocab_size"], n, 500 + i) for i, n in enumerate(lengths)}
    for dtype_name, dtype in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        folder = tiny.make_model_dir(tmp_path / dtype_name, config, trial, dtype, std=tiny.std_for(dtype, config["hidden_size"]))
        raw, tensors = tiny.read_model_dir(folder)
        expected = {rid: plain.forward_logits(raw, tensors, toks) for rid, toks in requests.items()}
        for cut in ("mixed", "portions"):
            steps = CUTS[cut](requests)
            got = th.collect(steps, run_trace(folder, dtype_name, page, steps), requests)
            check(got, expected, dtype_name, f"trial {trial} {config} page {page} {cut}")


@pytest.mark.parametrize("trial", range(3))
def test_long_requests_in_large_portions_replay_like_plain(trial, tmp_path, monkeypatch):
    """Requests of hundreds to thousands of tokens in portions of up to 2,048 (and of two), on
    narrow layers so that the plain implementation stays quick: the attention kernels' forms for
    many keys (several blocks of rows per request, windows of a thousand keys, portions behind a
    long context, decoding far into a request), which the tiny requests above never reach.  The
    second trial shares out every block of four windows of keys or more."""
    import random

    from turboserve_amd.kernels.ops import Ops

    rng = random.Random(7000 + trial)
    if trial == 1:
        monkeypatch.setattr(Ops, "prefill_share_min_windows", 4)
        monkeypatch.setattr(Ops, "prefill_share_combine_cost", 0)
    kv_heads, group = [(2, 7), (1, 8), (4, 5)][trial]
    window = [None, 1025, 300][trial]
    config = {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": rng.choice([64, 96, 136]),
        "num_hidden_layers": 2, "num_attention_heads": kv_heads * group, "num_key_value_heads": kv_heads,
        "head_dim": [128, 64, 128][trial], "intermediate_size": rng.choice([64, 104]), "vocab_size": rng.choice([97, 256]),
        "rope_theta": rng.choice([1e4, 1e6]), "rms_norm_eps": 1e-6, "tie_word_embeddings": trial == 1,
        "use_sliding_window": window is not None, "max_position_embeddings": 8192,
    }
    if window is not None:
        config["sliding_window"] = window
        config["max_window_layers"] = trial - 1  # trial 2: one layer sees everything, one the window
    page = [16, 32, 64][trial]
    lengths = [[3300, 700, 150], [1900, 5000, 700], [150, 1900, 3300]][trial]
    requests = {f"r{i}": tiny.random_tokens(config["vocab_size"], n, 500 + i) for i, n in enumerate(lengths)}
    cuts = {
        "portions": lambda reqs: th.portions(reqs, [512, 37, 1024, 2, 300, 2048]),
        "mixed": lambda reqs: th.mixed(reqs, [256, 33, 700, 2, 1500], max_live=3, decode_tail=6),
    }
    for dtype_name, dtype in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        folder = tiny.make_model_dir(tmp_path / dtype_name, config, trial, dtype, std=tiny.std_for(dtype, config["hidden_size"]))
        raw, tensors = tiny.read_model_dir(folder)
        expected = {rid: plain.forward_logits(raw, tensors, toks) for rid, toks in requests.items()}
        for cut, make in cuts.items():
            steps = make(requests)
            got = th.collect(steps, run_trace(folder, dtype_name, page, steps), requests)
            check(got, expected, dtype_name, f"long trial {trial} {config} page {page} {cut}")


LAYER_SHAPES = {
    "7b": dict(hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, intermediate_size=18944, rms_norm_eps=1e-6),
    "14b": dict(hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, intermediate_size=13824, rms_norm_eps=1e-5),
    "32b": dict(hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, intermediate_size=27648, rms_norm_eps=1e-5),
}


@pytest.mark.parametrize("shape", list(LAYER_SHAPES))
def test_real_layer_sizes_match_plain(shape):
    """Two layers of the Qwen2.5 7B, 14B and 32B sizes (28 heads on 4 KV heads and 40 on 8, of
    128; 18944, 13824 and 27648 wide; 152064 tokens) with random weights N(0, 0.02) that are
    bfloat16 numbers: the plain implementation on the CPU against the 32-bit path and the
    bfloat16 path, for one prompt of 300 tokens fed whole, in portions of 7, 5, 3 and 2 tokens,
    and with its last 32 tokens one by one (the reference's whole-model check,
    tests/unit/test_model_parity.py:171-181, 233-246).  The bfloat16 path runs a second time with
    the keys of its attention blocks shared out over several workgroups wherever a block has two
    windows of keys or more (what serving does for short portions behind long contexts)."""
    from turboserve_amd.cache.manager import CacheManager
    from turboserve_amd.engine.batch import StepEntry
    from turboserve_amd.engine.loading import build_model, build_storage, make_runtime
    from turboserve_amd.engine.runner import ModelRunner

    config = {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 2, "head_dim": 128,
        "vocab_size": 152064, "rope_theta": 1e6, "tie_word_embeddings": False, "max_position_embeddings": 32768,
        **LAYER_SHAPES[shape],
    }
    generator = torch.Generator().manual_seed(5)
    tokens = torch.randint(0, config["vocab_size"], (300,), generator=generator).tolist()
    # Rows whose logits are compared: the first tokens, places around page edges and portion
    # starts, the last 32.
    wanted = sorted({0, 1, 2, 15, 16, 17, 100, 127, 128, 255, 256, *range(268, 300)})
    portions, left = [], 300
    while left:
        portions.append(min((7, 5, 3, 2)[len(portions) % 4], left))
        left -= portions[-1]
    cuts = {"whole": [300], "portions": portions, "tail": [268] + [1] * 32}
    assert all(sum(sizes) == 300 for sizes in cuts.values()), {k: sum(v) for k, v in cuts.items()}
    want = None
    for dtype in (torch.float32, torch.bfloat16):
        runtime = make_runtime(dtype, "cuda:0")
        _, model = build_model(config, runtime)
        draw = torch.Generator(device="cuda:0")
        draw.manual_seed(3)
        tensors = {}
        for name, spec in model.tensor_specs().items():
            if spec.init == "ones":
                values = torch.ones(spec.shape, device="cuda:0")
            else:
                values = torch.empty(spec.shape, device="cuda:0").normal_(0.0, 0.02, generator=draw)
            tensors[name] = values.bfloat16().to(dtype)  # the same numbers in both runs
        if want is None:
            want = plain.forward_logits(config, {name: t.float().cpu() for name, t in tensors.items()}, tokens)[wanted]
            assert float(want.abs().max()) > 1.0
        model.load(tensors)
        del tensors
        storage = build_storage(model, 32, 16, 2)
        runner = ModelRunner(model, storage)
        passes = [(cut, sizes, False) for cut, sizes in cuts.items()]
        if dtype == torch.bfloat16:
            passes += [(cut, sizes, True) for cut, sizes in cuts.items()]
        ops = model.runtime.ops
        lists_with_shares = 0
        for cut, sizes, shared_out in passes:
            if shared_out and ops.prefill_share_min_windows != 1:
                ops.prefill_share_min_windows, ops.prefill_share_combine_cost = 1, 0
                made = ops.prefill_blocks

                def counting(*args, **kwargs):
                    nonlocal lists_with_shares
                    work = made(*args, **kwargs)
                    lists_with_shares += work.ranges is not None
                    return work

                ops.prefill_blocks = counting
            manager = CacheManager(storage.layout.windows(), 32, 16, 2)
            held = manager.admit("r")
            rows, start = [], 0
            for size in sizes:
                slots = manager.append("r", size)
                rows.append(runner.step([StepEntry(
                    request="r", tokens=tokens[start:start + size], start=start, tables=held.tables, slots=slots,
                    state_slot=held.state_slot, want=[p - start for p in wanted if start <= p < start + size])]).float().cpu())
                start += size
            got = torch.cat(rows)
            if dtype == torch.float32:
                ratio = excess(got, want, "float32")
                assert torch.equal(got.argmax(-1), want.argmax(-1))
            else:
                # Relative to the whole row of 152,064 logits (the largest difference of so many
                # is an extreme value) and to its largest logit.  Measured: up to 1.8% and 2.2%;
                # the reference's own formulas evaluated in bfloat16 (the plain implementation on
                # bfloat16 tensors) differ from their 32-bit evaluation by 1.9% and 2.3% here.
                difference = got - want
                ratio = torch.maximum(difference.norm(dim=1) / want.norm(dim=1) / 2.5e-2,
                                      difference.abs().max(dim=1).values / want.abs().max(dim=1).values / 3e-2)
            assert float(ratio.max()) <= 1.0, (
                f"{shape} {dtype} {cut} shared out {shared_out}: position {wanted[int(ratio.argmax())]} is off by "
                f"{float(ratio.max()):.2f} times its bound")
        assert dtype == torch.float32 or lists_with_shares >= 40, lists_with_shares
        runner.release()
        del model, storage, runner
        torch.cuda.empty_cache()
