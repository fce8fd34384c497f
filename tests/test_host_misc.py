"""Host-side pieces that need no GPU: the batch builder, sequences, the detokeniser and stop
strings, the command line's options, the model plan as data."""

from __future__ import annotations

import pytest

from turboserve_amd.cli import build_parser
from turboserve_amd.engine.batch import StepEntry, build_context, validate_entries
from turboserve_amd.engine.detokenizer import IncrementalDetokenizer, StopStringMatcher, StreamingDecoder
from turboserve_amd.engine.sequence import Sequence
from turboserve_amd.models.decoder import LayerCall, LayerSpec, ModelPlan
from turboserve_amd.parts.base import PartSpec
from turboserve_amd.sampling.params import FinishReason, SamplingParams


def entry(rid, tokens, start, table, want=()):
    slots = [[table[min(p // 4, len(table) - 1)] * 4 + p % 4 for p in range(start, start + len(tokens))]]
    return StepEntry(request=rid, tokens=tokens, start=start, tables=[table], slots=slots, want=list(want))


def test_batch_is_packed_with_multi_token_entries_first():
    entries = [entry("d1", [9], 6, [5, 1], [0]), entry("p", [1, 2, 3, 4, 5], 0, [2, 0], [4, 0]), entry("d2", [8], 2, [7], [0])]
    ctx = build_context(entries, num_groups=1, page_size=4, device="cpu")
    assert ctx.token_ids.tolist() == [1, 2, 3, 4, 5, 9, 8]
    assert ctx.positions.tolist() == [0, 1, 2, 3, 4, 6, 2]
    assert ctx.token_seq.tolist() == [0, 0, 0, 0, 0, 1, 2]
    assert ctx.query_start_loc.tolist() == [0, 5, 6, 7] and ctx.context_lens.tolist() == [5, 7, 3]
    assert ctx.logit_rows.tolist() == [5, 4, 0, 6]  # in the order the entries were given, and of their `want`
    assert ctx.block_tables[0].tolist() == [[2, 0], [5, 1], [7, -1]]
    assert ctx.slot_mapping[0].tolist() == [8, 9, 10, 11, 0, 6, 30]
    assert (ctx.num_prefill_seqs, ctx.num_decode_seqs, ctx.num_prefill_tokens) == (1, 2, 5)
    assert (ctx.max_query_len, ctx.max_context_len, ctx.max_decode_context_len) == (5, 7, 7)
    assert ctx.prefill_blocks.tolist() == [[0, 0]]
    long = build_context([entry("a", list(range(40)), 8, list(range(12))), entry("b", list(range(20)), 0, list(range(12, 17)))],
                         num_groups=1, page_size=4, device="cpu")
    assert long.prefill_blocks.tolist() == [[0, 32], [0, 16], [0, 0], [1, 56], [1, 40]]  # those that see most keys first


def test_batch_validation():
    """src/turboserve/engine/core/types.py:335-398 in the reference."""
    with pytest.raises(ValueError, match="appears twice"):
        validate_entries([entry("a", [1], 0, [0]), entry("a", [2], 1, [0])], 1, 4)
    with pytest.raises(ValueError, match="brings no token"):
        validate_entries([entry("a", [], 0, [0])], 1, 4)
    with pytest.raises(ValueError, match="does not cover"):
        validate_entries([entry("a", [1, 2], 3, [0])], 1, 4)
    with pytest.raises(ValueError, match="wanted place"):
        validate_entries([entry("a", [1, 2], 0, [0], [2])], 1, 4)
    bad = entry("a", [1, 2], 0, [0])
    bad.slots = [[0]]
    with pytest.raises(ValueError, match="slots for 2 tokens"):
        validate_entries([bad], 1, 4)


def test_sequence_accounting():
    """One formula for prompt, portion and decode (src/turboserve/engine/core/sequence.py:231-241)."""
    seq = Sequence(seq_id=0, request_id="r", prompt_token_ids=[1, 2, 3, 4, 5], sampling=SamplingParams(max_tokens=2))
    assert seq.num_new_tokens_to_compute(100) == 5 and seq.num_new_tokens_to_compute(3) == 3
    seq.advance_computed(3)
    assert seq.num_new_tokens_to_compute(100) == 2
    seq.advance_computed(2)
    assert seq.num_new_tokens_to_compute(100) == 0
    seq.append_token(9)
    assert seq.num_new_tokens_to_compute(100) == 1 and seq.tokens_in_range(3, 6) == [4, 5, 9]
    assert seq.check_stop(9) is None
    seq.append_token(8)
    assert seq.check_stop(8) is FinishReason.LENGTH
    with pytest.raises(ValueError):
        seq.advance_computed(5)
    seq.reset_for_recompute()
    assert seq.num_computed_tokens == 0 and seq.output_token_ids == [9, 8] and seq.num_preemptions == 1
    seq.finish(FinishReason.LENGTH)
    with pytest.raises(ValueError):
        seq.append_token(1)


class FakeTokenizer:
    """Token i decodes to a letter; 99 is half a two-token character."""

    def decode(self, ids, skip_special_tokens=True):
        out = ""
        i = 0
        while i < len(ids):
            if ids[i] == 99:
                if i + 1 < len(ids) and ids[i + 1] == 100:
                    out += "é"
                    i += 2
                    continue
                out += "�"
            else:
                out += chr(ord("a") + ids[i] % 26)
            i += 1
        return out


def test_incremental_detokenizer_holds_back_half_characters():
    """src/turboserve/engine/runtime/streaming.py:142-171."""
    detok = IncrementalDetokenizer(FakeTokenizer())
    assert detok.append([0, 1]) == "ab"
    assert detok.append([99]) == ""  # incomplete character: nothing yet
    assert detok.append([100]) == "é"
    assert detok.append([2] * 20) == "c" * 20
    assert detok.text == "abé" + "c" * 20
    detok.append([99])
    assert detok.flush() == "�"  # at the end what is left is emitted


def test_stop_strings():
    """src/turboserve/engine/runtime/streaming.py:193-262."""
    matcher = StopStringMatcher(["</s>", "END"])
    assert matcher.feed("hello <").text == "hello "  # "<" could still grow into a stop string
    assert matcher.feed("b").text == "<b"
    assert matcher.feed("x</").text == "x"
    delta = matcher.feed("s>tail")
    assert delta.stop == "</s>" and delta.text == "" and delta.stopped
    assert StopStringMatcher([]).feed("anything").text == "anything"
    decoder = StreamingDecoder(FakeTokenizer(), ["cd"])
    assert decoder.feed([0, 1]).text == "ab"
    assert decoder.feed([2]).text == ""
    delta = decoder.feed([3])
    assert delta.stopped and decoder.text == "ab"
    silent = StreamingDecoder(None, ["x"])
    assert silent.feed([1, 2]).text == "" and silent.finish() == ""


def test_command_line_options_are_the_references():
    """src/turboserve/engine/runtime/engine.py:522-547, 589-605."""
    args = build_parser().parse_args(["engine", "generate", "hi", "--model", "m"])
    assert (args.max_tokens, args.temperature, args.top_p, args.seed) == (64, 0.0, 1.0, None)
    assert (args.device, args.dtype, args.num_blocks) == ("auto", "auto", None)
    assert (args.max_num_seqs, args.max_num_batched_tokens, args.block_size, args.stats) == (8, 2048, 16, False)
    args = build_parser().parse_args(["--log-level", "DEBUG", "engine", "generate", "--prompt-ids", "1,2,3", "-m", "m", "--stats"])
    assert args.prompt_ids == ["1,2,3"] and args.stats and args.log_level == "DEBUG"
    kv = build_parser().parse_args(["engine", "kv-size", "--model", "m"])
    assert (kv.max_num_seqs, kv.gpu_memory_utilization, kv.max_model_len, kv.block_size) == (64, 0.9, None, 16)
    assert build_parser().parse_args(["hwinfo"]).indent == 2
    assert build_parser().parse_args(["version"]).command == "version"
    # the reference's flags for what is not built: accepted switched off, refused switched on
    off = build_parser().parse_args(["engine", "generate", "hi", "-m", "m", "--offline", "--no-prefix-caching"])
    assert off.offline and off.prefix_caching is False
    assert build_parser().parse_args(["engine", "kv-size", "-m", "m", "--offline"]).prefix_caching is False
    from turboserve_amd.cli import main

    with pytest.raises(ValueError, match="no prefix cache"):
        main(["engine", "generate", "--prompt-ids", "1", "-m", "m", "--prefix-caching"])


def test_the_run_order_is_data():
    norm = PartSpec("rmsnorm", {"size": 8, "eps": 1e-6})
    layers = (LayerSpec("model.layers.0", PartSpec("prenorm", {})), LayerSpec("model.layers.1", PartSpec("prenorm", {})))
    plan = ModelPlan(vocab_size=10, hidden_size=8, layers=layers, final_norm=norm, tie_head=True,
                     schedule=(LayerCall(0), LayerCall(1), LayerCall(0), LayerCall(1, cache_of=1)))
    assert [c.layer for c in plan.schedule] == [0, 1, 0, 1]  # a layer may run twice, or read an earlier call's cache
    with pytest.raises(ValueError, match="not earlier"):
        ModelPlan(10, 8, layers, (LayerCall(0, cache_of=0),), norm, True)
    with pytest.raises(ValueError, match="names layer"):
        ModelPlan(10, 8, layers, (LayerCall(2),), norm, True)
    with pytest.raises(ValueError, match="owns none"):
        ModelPlan(10, 8, layers, (LayerCall(0), LayerCall(1, cache_of=0), LayerCall(0, cache_of=1)), norm, True)


def test_bench_contract_on_the_host():
    """What of bench.py can be checked without a GPU: more than one GPU is refused with one
    line and exit code 2; the byte and flop counts behind `roofline` and `prefill.frac` are the
    7B shape's by hand; the other shapes differ only where the 14B and 32B layer sizes do."""
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    sys.path.insert(0, str(root))
    import bench
    from turboserve_amd.config.registry import parse_model_config

    refused = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert refused.returncode == 2 and len(refused.stdout.strip().splitlines()) == 1
    config = parse_model_config(dict(bench.SHAPE_7B))
    h, i, v, layers = 3584, 18944, 152064, 28
    per_layer = h * 4608 + 4608 + h * h + 3 * h * i + 2 * h  # qkv + bias, o, gate/up/down, two norms
    weights = layers * per_layer + h + v * h
    assert bench.decode_bytes(config, layers, 0, 0, 2) == 2 * weights
    cache_8 = 8 * 8192 * 2 * layers * 512 * 2  # batch 8, context 8192, K and V, 4 KV heads x 128, bf16
    assert bench.decode_bytes(config, layers, 8, 8192, 2) == 2 * (weights + 8 * h) + cache_8
    linear = layers * (h * 4608 + h * h + 3 * h * i)
    assert bench.prefill_flops(config, layers, 2048) == 2.0 * 2048 * linear + layers * 4 * h * 2048 * 2048 / 2 + 2.0 * v * h
    assert bench.SHAPES["14b"][1]["num_hidden_layers"] == 48 and bench.SHAPES["32b"][1]["intermediate_size"] == 27648
    assert bench.PEAK_FLOPS["bf16"] == 2.5e15 and bench.PEAK_FLOPS["fp32"] == 157.3e12 and bench.HBM_PEAK_GBS == 8000.0
