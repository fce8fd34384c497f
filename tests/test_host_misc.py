"""Host-side pieces that need no GPU: the batch builder, sequences, the detokeniser and stop
strings, the command line's options, the model plan as data."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from turboserve_amd.cli import build_parser
from turboserve_amd.engine.batch import StepEntry, StepLayout, StepLimits, build_context, check_packed, pack_step, validate_entries
from turboserve_amd.engine.detokenizer import StopAutomaton, TextStream
from turboserve_amd.engine.sequence import Sequence
from turboserve_amd.models.decoder import LayerCall, LayerSpec, ModelPlan
from turboserve_amd.parts.base import PartSpec
from turboserve_amd.parts.ends import standard_ends
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
    assert int(ctx.max_decode_context_dev[0]) == 7 and ctx.token_source.tolist() == [-1] * 7
    # what a part derives from a step is made once and shared by its layers
    made = []
    assert ctx.derive("k", lambda step: made.append(step.num_tokens) or "x") == "x" and ctx.derive("k", None) == "x"
    assert made == [7]
    # the prefill attention's work list: blocks of 16 rows, those that see most keys first
    from turboserve_amd.kernels.ops import prefill_block_list

    assert prefill_block_list([5], [5], 16) == [[0, 0]]
    assert prefill_block_list([40, 20], [48, 20], 16) == [[0, 32], [0, 16], [0, 0], [1, 56], [1, 40]]


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


def test_packed_step_is_checked_against_the_pools():
    """What a kernel would turn into an address is refused on the host
    (src/turboserve/engine/core/types.py:388-397, src/turboserve/engine/model/attention.py:105-112)."""
    limits = StepLimits(num_pages=[8], windows=[None], vocab_size=50, num_state_slots=4)
    build = lambda entries, lim=limits: build_context(entries, num_groups=1, page_size=4, device="cpu", limits=lim)
    build([entry("ok", [1, 2, 3, 4, 5], 3, [7, 0])])
    with pytest.raises(ValueError, match="page id 8 at index 1 .* outside the pool of 8 pages"):
        build([entry("a", [1, 2, 3, 4, 5], 0, [2, 8])])
    with pytest.raises(ValueError, match="page id -2"):
        build([entry("a", [1], 0, [-2])])
    with pytest.raises(ValueError, match="'a': no page at index 0 .* inside the keys 0..5"):
        build([entry("a", [1, 2], 4, [-1, 3])])
    with pytest.raises(ValueError, match="token id 50 is outside the vocabulary of 50"):
        build([entry("a", [1, 50], 0, [2])])
    with pytest.raises(ValueError, match="token id -1"):
        build([entry("b", [7], 0, [2]), entry("a", [-1], 0, [3])])
    wrong = entry("a", [1, 2, 3], 2, [5, 6])
    wrong.slots = [[22, 23, 25]]  # position 4 lies in page 6: slot 24
    with pytest.raises(ValueError, match="'a': slot 25 of group 0 is not where its block table puts position 4"):
        build([wrong])
    wrong.slots = [[22, -1, 24]]  # the skip mark is always allowed
    build([wrong])
    wrong.slots = [[22, 23, 32]]
    with pytest.raises(ValueError, match="slot 32"):
        build([wrong])
    bad_state = entry("a", [1], 0, [1])
    bad_state.state_slot = 5
    with pytest.raises(ValueError, match="state slot 5 is outside the 4 slots"):
        build([bad_state])
    # A windowed group: pages wholly below the lowest key of the step's first query may be gone.
    windowed = StepLimits(num_pages=[8], windows=[6], vocab_size=50)
    build([entry("w", [1, 2], 13, [-1, -1, 3, 4])], windowed)       # first query at 13 reads keys 8..13: pages 2, 3
    with pytest.raises(ValueError, match="no page at index 2 .* inside the keys 8..14"):
        build([entry("w", [1, 2], 13, [-1, -1, -1, 4])], windowed)
    with pytest.raises(ValueError, match="no page at index 1"):
        build([entry("w", [1, 2], 13, [0, -1, 3, 4])], StepLimits(num_pages=[8], windows=[None]))
    # unchecked steps (measurements) pack whatever they are given
    build_context([entry("a", [1, 2, 3, 4, 5], 0, [2, 8])], num_groups=1, page_size=4, device="cpu", check=False, limits=limits)


def test_one_packer_fills_exact_and_padded_shapes():
    """A recorded step's buffer is the same packed layout with more rows: what lies beyond the
    entries is padding that reads page 0, writes nothing and uses the padding state slot."""
    entries = [entry("x", [9], 6, [5, 1]), entry("y", [8], 2, [7]), entry("z", [3], 0, [4])]
    entries[1].state_slot = 2
    layout = StepLayout.make(4, 4, 4, (4,))
    data = np.full(layout.total, 77, dtype=np.int32)
    pack_step(data, layout, entries, range(4), pad_state_slot=9, token_sources={1: 0}, recorded=True)
    field = lambda name: layout.view(data, name).tolist()
    assert field("token_ids") == [9, 8, 3, 0] and field("positions") == [6, 2, 0, 0]
    assert field("token_seq") == [0, 1, 2, 3] and field("query_start_loc") == [0, 1, 2, 3, 4]
    assert field("context_lens") == [7, 3, 1, 1] and field("state_slots") == [0, 2, 0, 9]
    assert field("token_source") == [-1, 0, -1, -1] and field("logit_rows") == [0, 1, 2, 3]
    assert field("max_decode_context") == [7]
    assert field("slot_mapping0") == [6, 30, 16, -1]
    assert layout.view(data, "block_table0").reshape(4, 4).tolist() == [[5, 1, 0, 0], [7, 0, 0, 0], [4, 0, 0, 0], [0, 0, 0, 0]]
    check_packed(data, layout, entries, 4, StepLimits(num_pages=[8], windows=[None], vocab_size=10, num_state_slots=9))
    # the fill of unused table entries follows the kind of step, not whether every row is a request
    exact = StepLayout.make(3, 3, 3, (4,))
    filled = np.zeros(exact.total, dtype=np.int32)
    pack_step(filled, exact, entries, range(3), recorded=True)
    assert exact.view(filled, "block_table0").reshape(3, 4).tolist() == [[5, 1, 0, 0], [7, 0, 0, 0], [4, 0, 0, 0]]
    pack_step(filled, exact, entries, range(3))
    assert exact.view(filled, "block_table0").reshape(3, 4).tolist() == [[5, 1, -1, -1], [7, -1, -1, -1], [4, -1, -1, -1]]
    # a request whose own table is too short for its context is refused whatever the fill
    short = [entry("x", [9], 6, [5, 1]), entry("y", [8], 4, [7])]
    pack_step(filled, exact, [*short, entries[2]], range(3), recorded=True)
    with pytest.raises(ValueError, match="'y': its block table of group 0 holds 1 pages, 5 tokens need 2"):
        check_packed(filled, exact, [*short, entries[2]], 4, StepLimits(num_pages=[8], windows=[None]))
    with pytest.raises(ValueError, match="'y': token id 8"):  # a token taken from the device is not known: only 'y' is checked here
        pack_step(data, layout, entries, range(4), pad_state_slot=9, token_sources={0: 0})
        check_packed(data, layout, entries, 4, StepLimits(num_pages=[8], windows=[None], vocab_size=8))
    with pytest.raises(ValueError, match="do not fit"):
        pack_step(data, layout, [*entries, entry("p", [1, 2], 0, [1])], range(4))
    # every field starts on 16 bytes and the same layout serves a portion beside single tokens
    assert all(start % 4 == 0 for start, _ in layout.offsets.values())
    mixed = [entry("p", [1, 2, 3], 4, [2, 6]), entry("x", [9], 6, [5, 1])]
    layout = StepLayout.make(4, 2, 2, (2,))
    data = np.zeros(layout.total, dtype=np.int32)
    pack_step(data, layout, mixed, [2, 3])
    assert layout.view(data, "positions").tolist() == [4, 5, 6, 6] and layout.view(data, "token_seq").tolist() == [0, 0, 0, 1]
    assert layout.view(data, "query_start_loc").tolist() == [0, 3, 4] and layout.view(data, "max_decode_context").tolist() == [7]


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


class PlainText:
    """A stand-in tokenizer whose tokens are characters."""

    def decode(self, ids, skip_special_tokens=True):
        return "".join(ids)


def test_text_is_released_when_certain_and_half_characters_are_held_back():
    """src/turboserve/engine/runtime/streaming.py:142-171: the behaviour, not the method."""
    stream = TextStream(FakeTokenizer())
    assert stream.push([0, 1]).text == "ab"
    assert stream.push([99]).text == ""  # incomplete character: nothing yet
    assert stream.push([100]).text == "é"
    assert stream.push([2] * 20).text == "c" * 20
    assert stream.text == "abé" + "c" * 20
    for token in range(60):  # far past the point where the early tokens stop being decoded again
        assert stream.push([token]).text == chr(ord("a") + token % 26)
    assert len(stream._tail) <= TextStream.RESEAL_TOKENS + 1
    assert stream.push([99]).text == ""
    assert stream.close() == "\ufffd"  # at the end what is left is emitted
    assert stream.text == "abé" + "c" * 20 + "".join(chr(ord("a") + t % 26) for t in range(60)) + "\ufffd"
    # a half character that is completed across a reseal
    stream = TextStream(FakeTokenizer())
    stream.push(list(range(TextStream.RESEAL_TOKENS)))
    assert stream.push([3, 99]).text == "d" and stream.push([100, 4]).text == "ée"
    # the same text whatever the pieces
    ids = [5, 99, 100, 7, 99, 100, 99, 100, 1, 2] * 9
    whole = TextStream(FakeTokenizer())
    whole.push(ids)
    pieces = TextStream(FakeTokenizer())
    for i in range(0, len(ids), 3):
        pieces.push(ids[i:i + 3])
    assert whole.text + whole.close() == pieces.text + pieces.close() == FakeTokenizer().decode(ids)


def test_stop_strings():
    """src/turboserve/engine/runtime/streaming.py:193-262: text that may still become a stop
    string is held back, a completed one ends the request and is cut."""
    stream = TextStream(PlainText(), ["</s>", "END"])
    assert stream.push("hello <").text == "hello "  # "<" could still grow into a stop string
    assert stream.push("b").text == "<b"
    assert stream.push("x</").text == "x"
    delta = stream.push("s>tail")
    assert delta.stop == "</s>" and delta.text == "" and delta.stopped and stream.stopped_by == "</s>"
    assert stream.push("more").text == "" and stream.close() == "" and stream.text == "hello <bx"
    assert TextStream(PlainText(), []).push("anything").text == "anything"
    # held text is released when the request ends otherwise
    stream = TextStream(PlainText(), ["END"])
    assert stream.push("the EN").text == "the " and stream.close() == "EN" and stream.text == "the EN"
    # one stop string inside another, overlapping beginnings, and the same result however the text arrives
    for text in ("xxabcdyy", "ababcab", "aENENDb", "abcabcabd", "no stop here ab"):
        results = set()
        for size in (1, 2, 3, 100):
            stream = TextStream(PlainText(), ["abcd", "bc", "END", "abd"])
            for i in range(0, len(text), size):
                stream.push(text[i:i + size])
            results.add((stream.text + stream.close(), stream.stopped_by))
        assert len(results) == 1, (text, results)
        out, stop = results.pop()
        firsts = [(text.find(s) + len(s), -len(s), s) for s in ("abcd", "bc", "END", "abd") if s in text]
        if firsts:  # the stop string that is complete first (the longest of those that end there)
            end, _, which = min(firsts)
            assert stop == which and out == text[:end - len(which)]
        else:
            assert stop is None and out == text
    automaton = StopAutomaton(["</s>", "END", ""])
    assert automaton.stops == ("</s>", "END")
    state = 0
    for char, held in zip("a</</s", (0, 1, 2, 1, 2, 3)):
        state = automaton.step(state, char)
        assert automaton.held(state) == held and automaton.ended(state) is None
    assert automaton.ended(automaton.step(state, ">")) == "</s>"
    decoder = TextStream(FakeTokenizer(), ["cd"])
    assert decoder.push([0, 1]).text == "ab"
    assert decoder.push([2]).text == ""
    delta = decoder.push([3])
    assert delta.stopped and decoder.text == "ab"
    silent = TextStream(None, ["x"])
    assert silent.push([1, 2]).text == "" and silent.close() == ""


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
    ends = standard_ends(10, 8, norm, tie_head=True)
    assert ends["head"].params["tied_to"] == "model.embed_tokens.weight"
    plan = ModelPlan(vocab_size=10, hidden_size=8, layers=layers, **ends,
                     schedule=(LayerCall(0), LayerCall(1), LayerCall(0), LayerCall(1, cache_of=1)))
    assert [c.layer for c in plan.schedule] == [0, 1, 0, 1]  # a layer may run twice, or read an earlier call's cache
    with pytest.raises(ValueError, match="not earlier"):
        ModelPlan(10, 8, layers, (LayerCall(0, cache_of=0),), **ends)
    with pytest.raises(ValueError, match="names layer"):
        ModelPlan(10, 8, layers, (LayerCall(2),), **ends)
    with pytest.raises(ValueError, match="owns none"):
        ModelPlan(10, 8, layers, (LayerCall(0), LayerCall(1, cache_of=0), LayerCall(0, cache_of=1)), **ends)


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


def test_end_tokens_are_the_configs_and_the_tokenizers(tmp_path):
    """The set of ids that end a generation joins ``config.json``'s and the tokenizer's
    (src/turboserve/engine/runtime/engine.py:223-237); a ``tokenizer.json`` gets its end token
    from the ``tokenizer_config.json`` beside it."""
    import json
    from types import SimpleNamespace

    from tokenizers import Tokenizer
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import WhitespaceSplit

    from turboserve_amd.engine.detokenizer import get_tokenizer
    from turboserve_amd.engine.llm_engine import LLMEngine

    tokenizer = Tokenizer(WordLevel({"a": 0, "b": 1, "<end>": 2, "<turn>": 3}, unk_token="a"))
    tokenizer.pre_tokenizer = WhitespaceSplit()
    tokenizer.save(str(tmp_path / "tokenizer.json"))
    assert get_tokenizer(tmp_path).eos_token_id is None and get_tokenizer(tmp_path / "nothing") is None
    (tmp_path / "tokenizer_config.json").write_text(json.dumps({"eos_token": "<turn>"}))
    loaded = get_tokenizer(tmp_path)
    assert loaded.eos_token_id == 3 and loaded.encode("b a <end>") == [1, 0, 2]
    (tmp_path / "tokenizer_config.json").write_text(json.dumps({"eos_token": {"content": "<end>", "lstrip": False}}))
    assert get_tokenizer(tmp_path).eos_token_id == 2
    resolve = lambda config_ids, tok: LLMEngine._resolve_eos_token_ids(
        SimpleNamespace(model_config=SimpleNamespace(eos_token_ids=config_ids), tokenizer=tok))
    assert resolve((2,), loaded) == frozenset({2, 3})
    assert resolve((), None) == frozenset() and resolve((7, 9), None) == frozenset({7, 9})
    assert resolve((1,), SimpleNamespace(eos_token_id=[4, 5])) == frozenset({1, 4, 5})
    assert LLMEngine._resolve_eos_token_ids(SimpleNamespace(model_config={"no": "attribute"}, tokenizer=loaded)) == frozenset({3})


def test_kernel_shares_of_a_trace(tmp_path):
    """The per-kernel table of a ``rocprofv3 --kernel-trace`` CSV: the last steps of the trace,
    a step ending with the marker kernel; kernels grouped by short name and grid."""
    from turboserve_amd.profiling import format_shares, short_name, step_shares

    assert short_name("void (anonymous namespace)::gemm_tiled_kernel<5, 2>(float*, unsigned short*)") == "gemm_tiled_kernel<5, 2>"
    assert short_name("(anonymous namespace)::decode_kernel(float*, int)") == "decode_kernel"
    assert short_name("void at::native::vectorized_elementwise_kernel<8, at::native::FillFunctor<c10::BFloat16>, std::array<char*, 1ul> >(int)"
                      ).startswith("at::native::vectorized_elementwise_kernel<8, at::native::FillFunctor")
    header = ("Kind,Agent_Id,Queue_Id,Stream_Id,Thread_Id,Dispatch_Id,Kernel_Id,Kernel_Name,Correlation_Id,Start_Timestamp,"
              "End_Timestamp,LDS_Block_Size,Scratch_Size,VGPR_Count,Accum_VGPR_Count,SGPR_Count,Workgroup_Size_X,"
              "Workgroup_Size_Y,Workgroup_Size_Z,Grid_Size_X,Grid_Size_Y,Grid_Size_Z")
    rows, clock = [], 1000

    def kernel(name, grid, duration):
        nonlocal clock
        rows.append(f'"KERNEL_DISPATCH","Agent 1",1,0,1,{len(rows)},1,"{name}",0,{clock},{clock + duration},0,0,8,0,16,64,1,1,{grid},1,1')
        clock += duration + 100

    kernel("void setup_kernel(int)", 64, 50_000)  # before the steps: not counted
    for step in range(3):
        for _ in range(2):
            kernel("void (anonymous namespace)::gemm_tiled_kernel<5, 2>(float*)", 60672, 50_000)
            kernel("void (anonymous namespace)::gemm_tiled_kernel<5, 2>(float*)", 243456, 10_000)  # same kernel, another product
        kernel("void argmax_rows_kernel(int*, float const*, int const*)", 512, 5_000)
    trace = tmp_path / "1_kernel_trace.csv"
    trace.write_text(header + "\n" + "\n".join(rows) + "\n")
    result = step_shares(trace, steps=2)
    assert result.steps == 2 and result.kernels_per_step == 5 and abs(result.busy_us - 125.0) < 1e-9
    first, second, third = result.rows
    assert (first.name, first.grid, first.calls_per_step, first.average_us, first.per_step_us) == (
        "gemm_tiled_kernel<5, 2>", (60672, 1, 1), 2, 50.0, 100.0)
    assert second.grid == (243456, 1, 1) and second.per_step_us == 20.0 and third.name == "argmax_rows_kernel"
    assert abs(first.share - 0.8) < 1e-9
    text = format_shares(result, top=2)
    assert "| `gemm_tiled_kernel<5, 2>` | 60672, 1, 1 | 2 | 50.0 | 100.0 | 80.0% |" in text and "1 other kernels" in text
    with pytest.raises(ValueError, match="not enough"):
        step_shares(trace, steps=3)


def test_tiled_product_plans_are_the_ones_measured_best():
    """The cost model of the tiled decode product is fitted to measurements on a device of 256
    compute units; these are the grids that were fastest inside the step there ((iterations of
    128 per range of K, ranges, tile)), so that a change to the model that loses one shows."""
    from turboserve_amd.kernels.ops import Ops

    class Planner(Ops):
        def __init__(self):  # the plan needs the device's size only
            self.compute_units = 256
            self._tiled_plans = {}

    plan = Planner()._tiled_plan
    h7, i7, h14, i14 = 3584, 18944, 5120, 13824
    assert plan(8, 2 * i7, h7, None) == (28, 1, 5)        # 7B gate+up: one workgroup of 160 rows a unit, one range
    assert plan(8, h7, i7, None) == (17, 9, 2)            # 7B down: pairs of small workgroups, nine ranges
    assert plan(64, h7, i7, None) == (17, 9, 4)           # at 64 rows a pair is no longer ahead of a tile of 128
    assert plan(8, 152064, h7, 1) == (28, 1, 5)           # the head: one range, in rounds
    assert plan(8, h14, i14, None)[1:] in ((6, 2), (8, 5))  # 14B down: six ranges in pairs or eight of 160 rows, not three
    assert plan(8, 7168, h14, None) == (10, 4, 2)         # 14B qkv: four ranges, two workgroups a unit
    assert plan(8, 2 * i14, h14, None) == (40, 1, 2)      # 14B gate+up: 432 small workgroups
    assert plan(128, h7, i7, None)[2] != 2                # above 64 rows LDS holds one workgroup: no pairs to count on
    assert plan(8, 2 * 27648, 5120, None) == (40, 1, 4)   # 32B gate+up: 432 tiles of 128 (1.7 rounds), not 864 of 64
    assert plan(8, 2 * 29568, 8192, None) == (64, 1, 8)   # 72B gate+up: 231 tiles of 256, one round
    assert plan(8, 152064, 8192, 1)[2] != 8 and plan(8, h7, i7, None)[2] != 8  # tiles of 256: one range in one round only
    assert plan(40, 2 * 29568, 8192, None)[2] != 8        # and up to 32 rows
    # The wide kernel's tile for one range of K at 17 to 128 rows: what was fastest of all tiles
    # for the gate|up matrices of the 7B, 14B, 32B and 72B shapes.
    tile = Planner()._one_range_tile
    assert [tile(n, 64) for n in (2 * i7, 2 * i14, 2 * 27648, 2 * 29568)] == [5, 4, 8, 8]
    wide = Planner()._wide_plan_few_rows
    assert wide(64, 2 * i7, h7, 1) == (28, 1, 5, 64, 8, 128) and wide(128, 2 * i7, h7, 1) == (56, 1, 5, 128, 8, 64)
    assert wide(64, 2 * 27648, 5120, 1) == (80, 1, 8, 64, 8, 64)  # tiles of 256 weight rows are 64 deep
    assert wide(64, 152064, h7, 1)[2:] == (5, 64, 8, 64)          # the head: several rounds, 64 deep
    assert wide(64, h7, i7, None) == (17, 9, 4, 64, 8, 128)       # down: ranges of K, tiles of 128


def test_library_products_run_at_a_few_sizes():
    """The sizes at which the BLAS library's products are run when they are all timed: a step is
    at most a quarter longer than it had to be, the token budget is a size itself, decode-sized
    steps keep their own size, and a buffer is seen longer only if its storage reaches that far."""
    from turboserve_amd.kernels.ops import Ops

    class Sized(Ops):
        def __init__(self, sizes):
            self.library_buckets = sizes

    sizes = Ops.bucket_sizes(2000)
    assert sizes[-1] == 2000 and list(sizes) == sorted(set(sizes))
    assert {32, 256, 320, 512, 640, 1024, 1280, 1792}.issubset(sizes) and 288 not in sizes and 576 not in sizes
    assert Ops.bucket_sizes(100) == (32, 64, 96, 100)
    ops = Sized(sizes)
    assert ops.library_rows(1) == 1 and ops.library_rows(128) == 128, "decode-sized steps use the engine's own products"
    for rows in range(129, 2001):
        at = ops.library_rows(rows)
        assert at in sizes and rows <= at <= rows * 1.25
    assert ops.library_rows(2001) == 2001, "beyond the largest size a step keeps its own"
    assert Sized(()).library_rows(777) == 777
    buffer = ops.rows_buffer(130, 8, torch.float32, "cpu")
    assert buffer.shape == (130, 8) and buffer.is_contiguous()
    seen = Ops._with_room(buffer, 160)
    assert seen.shape == (160, 8) and seen.data_ptr() == buffer.data_ptr()
    assert Ops._with_room(torch.empty(130, 8), 160) is None, "no room behind it"
    assert Ops._with_room(torch.empty(160, 16)[:130, :8], 160) is None, "rows that are not dense"
    assert Ops._with_room(torch.empty(4, 160, 8)[1, :130], 160).shape == (160, 8)
    assert Ops._with_room(torch.empty(4, 160, 8)[3, 10:140], 160) is None, "it would run past the end"


def test_prefill_work_list_shares_out_long_blocks():
    """The planner of the prefill attention's work list: every window of every block is taken by
    exactly one entry, shares of a block lie in consecutive slots, nothing is shared out where
    the device is busy anyway or a block is short, and what it picks is no slower, played
    through, than whole blocks."""
    from turboserve_amd.kernels.ops import prefill_block_list, prefill_block_windows, prefill_share_list

    assert prefill_block_windows(0, 32, 0) == 1 and prefill_block_windows(31, 2, 0) == 2
    assert prefill_block_windows(2016, 32, 0) == 64 and prefill_block_windows(2016, 32, 100) == 5
    assert prefill_block_windows(100, 1, 33) == 2  # keys 68..100: windows 64.. and 96..

    def check(query_lens, context_lens, window, per_block, places, min_windows=16):
        blocks, ranges, combine = prefill_share_list(query_lens, context_lens, 32, window, per_block, places, min_windows)
        if not ranges:
            assert blocks == prefill_block_list(query_lens, context_lens, 32) and combine == []
            return blocks, ranges, combine
        assert len(blocks) == len(ranges)
        taken, first_row, sizes = {}, 0, []
        starts = []
        for count in query_lens:
            starts.append(first_row)
            first_row += count
        for (request, row), (first, windows, slot) in zip(blocks, ranges):
            offset = row - starts[request]
            here = min(32, query_lens[request] - offset)
            total = prefill_block_windows(context_lens[request] - query_lens[request] + offset, here, window)
            span = range(total) if slot < 0 else range(first, first + windows)
            assert slot >= 0 or (first, windows) == (0, 0)
            assert windows >= 1 or slot < 0
            sizes.append(len(span))
            for w in span:
                assert 0 <= w < total and (request, row, w) not in taken
                taken[(request, row, w)] = slot
        covered = sum(prefill_block_windows(c - q + o, min(32, q - o), window)
                      for q, c in zip(query_lens, context_lens) for o in range(0, q, 32))
        assert len(taken) == covered
        assert sizes == sorted(sizes, reverse=True), "the longest entries start first"
        slots_seen = sorted(slot for _, _, slot in ranges if slot >= 0)
        assert slots_seen == list(range(len(slots_seen)))
        for row, rows, first_slot, shares in combine:
            assert 2 <= shares <= 16 and 1 <= rows <= 32
            members = [(b, r) for b, r in zip(blocks, ranges) if first_slot <= r[2] < first_slot + shares]
            assert len(members) == shares and all(b[1] == row for b, _ in members)
            assert sorted(r[0] for _, r in members) == [r[0] for _, r in sorted(members, key=lambda m: m[1][2])]
        assert sum(c[3] for c in combine) == len(slots_seen)
        return blocks, ranges, combine

    # a short portion at the end of a long context: every block several times, all at once
    blocks, ranges, combine = check([512], [8192], 0, 4, 256)
    assert len(combine) == 16 and all(c[3] == 4 for c in combine) and len(blocks) * 4 == 256
    blocks, ranges, combine = check([128], [16384], 0, 4, 256)
    assert len(combine) == 4 and all(c[3] == 16 for c in combine)
    # whole blocks that fill the device stay whole (a second workgroup's start costs more than
    # the shorter blocks save), and so do blocks too short to be worth putting together
    assert check([2048], [2048], 0, 4, 256)[1] == []
    assert check([8192], [8192], 0, 4, 256)[1] == []
    assert check([2048], [8192], 0, 4, 256)[1] == []
    assert check([600, 40], [600, 900], 0, 4, 256)[1] == []
    # a sliding window makes every block short
    assert check([512], [8192], 128, 4, 256)[1] == []
    # shares and whole blocks of several requests; a window that leaves long blocks
    blocks, ranges, combine = check([300, 100, 33], [4000, 150, 2000], 0, 8, 512, min_windows=4)
    assert combine and any(r[2] < 0 for r in ranges)
    assert check([64, 64], [3000, 4000], 1024, 4, 256, min_windows=8)[1]
    check([5], [5], 0, 4, 256)
    check([], [], 0, 4, 256)
    # the same invariants on seeded random steps: any mix of portions, contexts, windows, grids
    import random

    rng = random.Random(5)
    shared_out = 0
    for _ in range(400):
        requests = rng.randint(1, 5)
        query_lens = [rng.choice([1, 2, 31, 32, 33, 64, 100, 300, 700]) for _ in range(requests)]
        context_lens = [q + rng.choice([0, 0, 5, 200, 3000, 20000]) for q in query_lens]
        _, ranges, _ = check(query_lens, context_lens, rng.choice([0, 0, 33, 500, 4096]), rng.choice([1, 2, 4, 8, 16]),
                             rng.choice([64, 256, 512]), min_windows=rng.choice([1, 4, 16]))
        shared_out += bool(ranges)
    assert shared_out > 40


def test_the_kept_token_array_follows_the_lists():
    """``Sequence.token_array`` is ``token_ids`` at every moment: through appended tokens, places
    taken for unread tokens and filled or dropped later, growth beyond what the array held, and a
    reset for recomputation."""
    import random

    rng = random.Random(3)
    seq = Sequence(seq_id=1, request_id="a", prompt_token_ids=[rng.randrange(1000) for _ in range(70)],
                   sampling=SamplingParams(max_tokens=10_000))
    assert seq.token_array().tolist() == seq.token_ids and seq.token_array().dtype == np.int32
    pending = None
    for turn in range(400):
        action = rng.random()
        if pending is not None and action < 0.6:
            seq.set_unread_token(pending, rng.randrange(1000))
            pending = None
        elif pending is not None and action < 0.65:
            seq.drop_unread_token(pending)
            pending = None
        elif pending is None and action < 0.8:
            pending = seq.append_unread_token()
        elif pending is None:
            seq.append_token(rng.randrange(1000))
        if turn % 3 == 0:  # not looked at every turn: several changes meet one call
            assert seq.token_array().tolist() == seq.token_ids, turn
        if turn == 250:
            seq.reset_for_recompute()
    assert seq.token_array().tolist() == seq.token_ids and seq.num_output_tokens > 100


def test_an_attention_geometry_no_kernel_takes_is_refused_when_the_model_is_put_together():
    """A head size above what the attention kernels take, or an odd one, is refused when the part
    is built (from the configuration alone, on the host), not at the first step after the weights
    have been read."""
    import tiny
    from turboserve_amd.kernels.ops import ATTENTION_MAX_HEAD_DIM, attention_geometry_error
    from turboserve_amd.parts.attention import GroupedQueryAttention
    from turboserve_amd.parts.base import Runtime
    from turboserve_amd.weights.random_init import describe_model

    describe_model({**tiny.CONFIG_A, "head_dim": ATTENTION_MAX_HEAD_DIM})
    with pytest.raises(ValueError, match="model.layers.0.self_attn: a head size of 520 is above"):
        describe_model({**tiny.CONFIG_A, "head_dim": ATTENTION_MAX_HEAD_DIM + 8})
    assert attention_geometry_error(28, 4, 128) is None and attention_geometry_error(5, 1, 20) is None
    assert "not a multiple" in attention_geometry_error(6, 4, 64)
    assert "not even" in attention_geometry_error(4, 2, 33)
    runtime = Runtime(device=torch.device("cpu"), dtype=torch.float32, ops=None)
    common = dict(hidden_size=64, scale=1.0, qkv_bias=False, out_bias=False, window=None, position=PartSpec("none"))
    with pytest.raises(ValueError, match="not even"):
        GroupedQueryAttention("m", runtime, num_heads=4, num_kv_heads=2, head_dim=7, **common)
    with pytest.raises(ValueError, match="not a multiple"):
        GroupedQueryAttention("m", runtime, num_heads=5, num_kv_heads=2, head_dim=8, **common)


def test_a_parts_own_step_field_travels_in_the_packed_buffer():
    """A field a part asks for (``Part.step_fields``) lies behind the engine's own in the packed
    buffer, is filled from the entries in row order, padded in a recorded shape, and reaches the
    part as ``ctx.extras[name]``."""
    from turboserve_amd.engine.batch import StepField, merge_step_fields

    age = StepField("request_start", lambda t, s, n: s, lambda entries: [e.start for e in entries], pad=-7)
    parity = StepField("token_parity", lambda t, s, n: t, lambda entries: [tok % 2 for e in entries for tok in e.tokens])
    fields = merge_step_fields([age, parity, age])
    assert fields == (age, parity)
    with pytest.raises(ValueError, match="different step fields named 'request_start'"):
        merge_step_fields([age, StepField("request_start", age.length, age.fill, pad=0)])
    for taken in ("positions", "block_table0", "slot_mapping12"):
        with pytest.raises(ValueError, match="one of the engine's own"):
            merge_step_fields([StepField(taken, age.length, age.fill)])
    entries = [entry("x", [9], 6, [5, 1]), entry("p", [1, 2, 3], 4, [2, 6]), entry("z", [3], 0, [4], want=[0])]
    ctx = build_context(entries, num_groups=1, page_size=4, device="cpu", extra_fields=fields)
    assert ctx.extras["request_start"].tolist() == [4, 6, 0]  # the portion first, then the single tokens as given
    assert ctx.extras["token_parity"].tolist() == [1, 0, 1, 1, 1]
    assert ctx.token_ids.tolist() == [1, 2, 3, 9, 3] and ctx.logit_rows.tolist() == [4]
    # the same fields in a recorded shape of four rows: padding behind the three entries
    single = [entry("x", [9], 6, [5, 1]), entry("y", [8], 2, [7]), entry("z", [3], 0, [4])]
    layout = StepLayout.make(4, 4, 4, (2,), fields)
    data = np.full(layout.total, 77, dtype=np.int32)
    pack_step(data, layout, single, range(4), recorded=True)
    assert layout.view(data, "request_start").tolist() == [6, 2, 0, -7]
    assert layout.view(data, "token_parity").tolist() == [1, 0, 1, 0]
    assert all(start % 4 == 0 for start, _ in layout.offsets.values())
    with pytest.raises(ValueError, match="'request_start': 5 values for a field of 4"):
        pack_step(data, StepLayout.make(4, 4, 4, (2,), [StepField("request_start", age.length, lambda entries: [0] * 5)]),
                  single, range(4))


def test_replay_and_bench_are_commands_of_the_one_command_line(capsys):
    """``turboserve engine replay`` and ``turboserve engine bench`` hand their arguments to the
    trace replay program and to ``bench.py``; every other command still refuses what it does not
    know.  The measurement's record names the code by a digest of the sources where there is no
    git checkout."""
    from turboserve_amd import cli
    from turboserve_amd.hwinfo import brief, git_info, source_digest

    assert cli.main(["engine", "bench", "--gpus", "2"]) == 2
    assert "measures one GPU" in capsys.readouterr().out
    with pytest.raises(SystemExit) as stop:
        cli.main(["engine", "replay", "--help"])
    assert stop.value.code == 0 and "--max-tokens" in capsys.readouterr().out
    with pytest.raises(SystemExit) as stop:
        cli.main(["engine", "replay", "--model", "nowhere"])  # trace_run's own parser: the other arguments are required
    assert stop.value.code == 2
    capsys.readouterr()
    with pytest.raises(SystemExit):
        cli.main(["engine", "kv-size", "--bogus"])
    assert "unrecognized arguments: --bogus" in capsys.readouterr().err
    facts = brief()
    assert set(facts) == {"gpu", "arch", "torch", "hip", "rocm", "git", "source"}
    assert len(facts["source"]) == 12 and facts["source"] == source_digest()[:12] == git_info()["source_digest"][:12]
