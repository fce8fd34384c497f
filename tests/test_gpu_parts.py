"""The parts of a model, alone and recombined: each built-in part against the plain
implementation; a toy mixer with state of its own, a toy feed-forward with routing, two toy
position encodings (one added to queries and keys, one a bias inside the scores), a toy
embedding, a toy head and a toy architecture made of them, all defined here and registered
without touching the framework; a run order that names a layer twice and lets a
layer read another layer's cache; long decoding and the first tokens of a sequence."""

from __future__ import annotations

import json
from pathlib import Path

import pytest
import torch

import tiny
import trace_helpers as th
from plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def make_runtime(dtype):
    from turboserve_amd.engine.loading import make_runtime

    return make_runtime(dtype, DEV)


def assert_matches(got: torch.Tensor, want: torch.Tensor, dtype) -> None:
    """32-bit: 1e-4 absolute.  bfloat16 against the plain implementation in 32-bit: relative to
    the largest value, the criterion of the replay tests."""
    worst = float((got - want).abs().max())
    bound = 1e-4 if dtype == torch.float32 else 2e-2 * float(want.abs().max())
    assert worst <= bound, f"max |diff| {worst:.3e} > {bound:.3e}"


def one_request_context(tokens: int, page: int, start: int = 0, groups: int = 1):
    """A step context for one request bringing ``tokens`` tokens at ``start``, pages 0, 1, ..."""
    from turboserve_amd.engine.batch import StepEntry, build_context

    pages = list(range(-(-(start + tokens) // page)))
    slots = [pages[p // page] * page + p % page for p in range(start, start + tokens)]
    entry = StepEntry(request="r", tokens=[0] * tokens, start=start, tables=[pages] * groups, slots=[slots] * groups,
                      want=list(range(tokens)))
    return build_context([entry], num_groups=groups, page_size=page, device=DEV)


# -- built-in parts alone ----------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    from turboserve_amd.parts.base import PartSpec, ResidualStream
    from turboserve_amd.parts.registry import build_part

    runtime = make_runtime(dtype)
    norm = build_part("norm", PartSpec("rmsnorm", {"size": 72, "eps": 3e-6}), "n", runtime)
    assert list(norm.tensor_specs()) == ["n.weight"] and norm.tensor_specs()["n.weight"].init == "ones"
    g = torch.Generator().manual_seed(0)
    w = (1 + 0.1 * torch.randn(72, generator=g)).to(dtype)
    norm.load({"n.weight": w.to(DEV)})
    x = torch.randn(5, 72, generator=g).to(dtype)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(norm.forward(x.to(DEV)).float().cpu(), plain.rms_norm(x.float(), w.float(), 3e-6), **tol)
    stream = ResidualStream(torch.randn(5, 72, generator=g).to(DEV), x.to(DEV))
    before = stream.residual.clone()
    y = norm.forward_residual(stream)
    assert stream.pending is None
    torch.testing.assert_close(stream.residual.cpu(), before.cpu() + x.float(), rtol=0, atol=1e-6)
    torch.testing.assert_close(y.float().cpu(), plain.rms_norm(before.cpu() + x.float(), w.float(), 3e-6), **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [None, 5])
def test_attention_and_feed_forward_and_block_parts(dtype, window):
    """One attention mixer, one SwiGLU and one pre-norm block built from specs with sizes of
    their own (not a model's), stepped in two portions, against the plain functions."""
    from turboserve_amd.parts.base import PagedKVView, PartSpec, ResidualStream
    from turboserve_amd.parts.registry import build_part

    runtime = make_runtime(dtype)
    hidden, heads, kv_heads, dim, inter, page, eps = 48, 6, 2, 16, 40, 8, 1e-5
    position = PartSpec("rope", {"head_dim": dim, "theta": 5000.0, "scaling_factor": 1.0, "max_positions": 64})
    mixer_spec = PartSpec("gqa_attention", {
        "hidden_size": hidden, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": dim, "scale": dim ** -0.5,
        "qkv_bias": True, "out_bias": False, "window": window, "position": position})
    ff_spec = PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": inter})
    norm_spec = PartSpec("rmsnorm", {"size": hidden, "eps": eps})
    block = build_part("block", PartSpec("prenorm", {"mixer": mixer_spec, "feed_forward": ff_spec,
                                                     "mixer_norm": norm_spec, "ff_norm": norm_spec}), "model.layers.0", runtime)
    from turboserve_amd.parts.base import PagedKV

    assert block.mixer.cache_need() == PagedKV(kv_heads, dim, window)
    g = torch.Generator().manual_seed(1)
    tensors = {}
    for name, spec in block.tensor_specs().items():
        t = torch.ones(spec.shape) + 0.1 * torch.randn(spec.shape, generator=g) if spec.init == "ones" else 0.2 * torch.randn(spec.shape, generator=g)
        tensors[name] = t.to(dtype)
    block.load({k: v.to(DEV) for k, v in tensors.items()})
    cfg = {"hidden_size": hidden, "num_hidden_layers": 1, "num_attention_heads": heads, "num_key_value_heads": kv_heads,
           "head_dim": dim, "intermediate_size": inter, "vocab_size": 8, "rms_norm_eps": eps, "rope_theta": 5000.0,
           "use_sliding_window": window is not None, "sliding_window": window, "max_window_layers": 0}
    values = plain.cfg_values(cfg)
    ftensors = {k: v.float() for k, v in tensors.items()}
    tokens = 13
    h = torch.randn(tokens, hidden, generator=g).to(dtype)
    want = plain.decoder_layer(h.float(), ftensors, 0, values, torch.arange(tokens))
    kpages = torch.zeros(4, kv_heads, page, dim, dtype=dtype, device=DEV)
    vpages = torch.zeros(4, kv_heads, dim, page, dtype=dtype, device=DEV)
    cache = PagedKVView(kpages, vpages, group=0, block_size=page, window=window)
    got = []
    for start, count in ((0, 9), (9, 4)):
        ctx = one_request_context(count, page, start)
        stream = block.forward(ResidualStream(h[start:start + count].float().to(DEV)), ctx, cache)
        total = stream.residual + runtime.ops.dense(stream.pending, dtype).float()
        got.append(total.cpu())
    assert_matches(torch.cat(got), want, dtype)
    # the mixer alone, and the feed-forward alone
    x = plain.rms_norm(h.float(), ftensors["model.layers.0.input_layernorm.weight"], eps)
    attn_want = plain.attention_block(x, ftensors, "model.layers.0.self_attn", values, torch.arange(tokens), window)
    ctx = one_request_context(tokens, page)
    kpages.zero_(); vpages.zero_()
    attn = runtime.ops.dense(block.mixer.forward(x.to(dtype).to(DEV), ctx, cache), dtype).float().cpu()
    assert_matches(attn, attn_want, dtype)
    ff_want = plain.swiglu_mlp(x, *(ftensors[f"model.layers.0.mlp.{p}_proj.weight"] for p in ("gate", "up", "down")))
    ff = runtime.ops.dense(block.feed_forward.forward(x.to(dtype).to(DEV), ctx), dtype).float().cpu()
    assert_matches(ff, ff_want, dtype)


# -- a toy mixer with state of its own, and a toy architecture ---------------------------------------


def _position_buckets(entries):
    return [(entry.start + i) // 5 for entry in entries for i in range(len(entry.tokens))]


def _make_position_bucket_field():
    from turboserve_amd.engine.batch import StepField

    return StepField("position_bucket", lambda tokens, requests, wanted: tokens, _position_buckets, pad=0)


#: The step field of the toy mixer below: defined once, so that every layer of the kind names the same one.
POSITION_BUCKET = _make_position_bucket_field()


def register_toy_architecture():
    """Everything a new mixer and a new architecture need, using only the public registries."""
    from turboserve_amd.config import registry as arch_registry
    from turboserve_amd.models.decoder import LayerCall, LayerSpec, ModelPlan
    from turboserve_amd.parts import registry as part_registry
    from turboserve_amd.parts.base import (Embedding, FeedForward, FixedState, Head, Mixer, PartSpec, PositionEncoding,
                                           TensorSpec)

    if "running_mean" not in part_registry.MIXERS:

        @part_registry.register_mixer("running_mean")
        class RunningMean(Mixer):
            """out_t = W * mean(x_0 .. x_t): per request a running sum [H] and a count."""

            def __init__(self, prefix, runtime, *, hidden_size):
                super().__init__(prefix, runtime)
                self.hidden = hidden_size
                self.weight = None

            def cache_need(self):
                return FixedState((self.hidden + 1,), torch.float32)

            def tensor_specs(self):
                return {self.name("mix.weight"): TensorSpec((self.hidden, self.hidden))}

            def load(self, tensors):
                self.weight = tensors[self.name("mix.weight")]

            def forward(self, x, ctx, cache):
                out = torch.empty_like(x)
                row = 0
                for s, count in enumerate(ctx.query_lens):
                    slot = ctx.state_slots[s:s + 1].long()
                    state = cache.state.index_select(0, slot)[0]
                    sums = state[: self.hidden] + torch.cumsum(x[row:row + count].float(), dim=0)
                    counts = state[self.hidden] + torch.arange(1, count + 1, device=x.device, dtype=torch.float32)
                    mean = (sums / counts[:, None]).to(x.dtype)
                    out[row:row + count] = mean @ self.weight.t()
                    cache.state.index_copy_(0, slot, torch.cat((sums[-1], counts[-1:]))[None])
                    row += count
                return out

    if "sink_attention" not in part_registry.MIXERS:
        from turboserve_amd.parts.base import PagedKV

        @part_registry.register_mixer("sink_attention")
        class SinkAttention(Mixer):
            """One-head attention whose cached values are wider than its keys, plus the running
            mean of its inputs: a layer that keeps pages AND fixed-size state, and that asks the
            step for a field of its own (the bucket of five positions a token lies in, looked up
            in a learned table and added to the query).  Plain torch operations on the pages, no
            kernel of the engine: everything is indexed on the device, so it records."""

            def __init__(self, prefix, runtime, *, hidden_size, key_dim, value_dim, buckets):
                super().__init__(prefix, runtime)
                self.hidden, self.key_dim, self.value_dim, self.buckets = hidden_size, key_dim, value_dim, buckets
                self.w = {}

            def cache_need(self):
                return (PagedKV(1, self.key_dim, None, self.value_dim), FixedState((self.hidden + 1,), torch.float32))

            def step_fields(self):
                return (POSITION_BUCKET,)

            def tensor_specs(self):
                h, dk, dv = self.hidden, self.key_dim, self.value_dim
                shapes = {"q.weight": (dk, h), "k.weight": (dk, h), "v.weight": (dv, h), "o.weight": (h, dv),
                          "sink.weight": (h, h), "bucket_table": (self.buckets, dk)}
                return {self.name(key): TensorSpec(shape) for key, shape in shapes.items()}

            def load(self, tensors):
                self.w = {key: tensors[self.name(key)].float() for key in
                          ("q.weight", "k.weight", "v.weight", "o.weight", "sink.weight", "bucket_table")}

            def forward(self, x, ctx, cache):
                pages, state = cache
                assert tuple(pages.v.shape[1:]) == (1, self.value_dim, pages.block_size) and pages.k.shape[-1] == self.key_dim
                xf = x.float()
                bucket = ctx.extras["position_bucket"].long().clamp(max=self.buckets - 1)
                q = xf @ self.w["q.weight"].t() + self.w["bucket_table"].index_select(0, bucket)
                k, v = xf @ self.w["k.weight"].t(), xf @ self.w["v.weight"].t()
                num_pages, size = pages.k.shape[0], pages.block_size
                # write: slot -> row of the pages seen as [pages x size, width] (a padded row's slot is -1 and matches nothing)
                slots = ctx.slot_mapping[pages.group].long()
                hit = (slots[:, None] == torch.arange(num_pages * size, device=x.device)[None, :]).float()  # [T, slots]
                written = hit.sum(dim=0) > 0
                flat_k = pages.k.view(num_pages * size, self.key_dim)
                flat_k.copy_(torch.where(written[:, None], (hit.t() @ k).to(flat_k.dtype), flat_k))
                flat_v = pages.v.permute(0, 1, 3, 2).reshape(num_pages * size, self.value_dim)
                flat_v = torch.where(written[:, None], (hit.t() @ v).to(flat_v.dtype), flat_v)
                pages.v.copy_(flat_v.view(num_pages, 1, size, self.value_dim).permute(0, 1, 3, 2))
                # read: every token over the keys 0 .. its position of its request, through the block table
                table = ctx.block_tables[pages.group].index_select(0, ctx.token_seq.long()).long()  # [T, width]
                places = torch.arange(table.shape[1] * size, device=x.device)
                where = table.clamp(min=0)[:, places // size] * size + (places % size)[None, :]  # [T, L]
                keys = flat_k.float()[where]
                values = flat_v.float()[where]
                scores = (q[:, None, :] * keys).sum(dim=-1) * self.key_dim ** -0.5
                scores = scores.masked_fill(places[None, :] > ctx.positions[:, None], float("-inf"))
                attended = (torch.softmax(scores, dim=-1)[:, :, None] * values).sum(dim=1) @ self.w["o.weight"].t()
                # the running mean, per request, continued from the request's state slot
                rows_of = ctx.token_seq.long()
                slot_of = ctx.state_slots.long().index_select(0, rows_of)
                before = state.state.index_select(0, slot_of)  # [T, H + 1]
                same = (rows_of[:, None] == rows_of[None, :]) & (ctx.positions[None, :] <= ctx.positions[:, None])
                sums = before[:, : self.hidden] + same.float() @ xf
                counts = before[:, self.hidden] + same.float().sum(dim=1)
                mean = sums / counts[:, None]
                last = ctx.query_start_loc[1:].long() - 1  # each request's last row of this step
                state.state.index_copy_(0, ctx.state_slots.long(), torch.cat((sums, counts[:, None]), dim=1).index_select(0, last))
                return (attended + mean @ self.w["sink.weight"].t()).to(x.dtype)

    if "top1_experts" not in part_registry.FEED_FORWARDS:

        @part_registry.register_feed_forward("top1_experts")
        class Top1Experts(FeedForward):
            """A feed-forward with routing: 32-bit router logits pick one SwiGLU expert per token."""

            def __init__(self, prefix, runtime, *, hidden_size, intermediate_size, num_experts):
                super().__init__(prefix, runtime)
                self.hidden, self.inter, self.experts = hidden_size, intermediate_size, num_experts
                self.router = None
                self.weights = []

            def tensor_specs(self):
                specs = {self.name("router.weight"): TensorSpec((self.experts, self.hidden), kind="float_keep32")}
                for e in range(self.experts):
                    specs[self.name(f"experts.{e}.gate_proj.weight")] = TensorSpec((self.inter, self.hidden))
                    specs[self.name(f"experts.{e}.up_proj.weight")] = TensorSpec((self.inter, self.hidden))
                    specs[self.name(f"experts.{e}.down_proj.weight")] = TensorSpec((self.hidden, self.inter))
                return specs

            def load(self, tensors):
                self.router = tensors[self.name("router.weight")].float()
                self.weights = [tuple(tensors[self.name(f"experts.{e}.{n}_proj.weight")] for n in ("gate", "up", "down"))
                                for e in range(self.experts)]

            def forward(self, x, ctx):
                # Every expert on every row, the chosen one kept: nothing is read back to the
                # host, so the step stays recordable into a HIP graph (a toy may be wasteful).
                choice = (x.float() @ self.router.t()).argmax(dim=-1)
                out = torch.zeros_like(x)
                for e, (gate, up, down) in enumerate(self.weights):
                    act = torch.nn.functional.silu(x @ gate.t()) * (x @ up.t())
                    out = torch.where((choice == e)[:, None], act @ down.t(), out)
                return out

    if "learned_positions" not in part_registry.POSITION_ENCODINGS:

        @part_registry.register_position_encoding("learned_positions")
        class LearnedPositions(PositionEncoding):
            """Another position encoding: a learned vector per position, added to every head's
            query and key before the keys are stored (no rotation)."""

            def __init__(self, prefix, runtime, *, head_dim, max_positions):
                super().__init__(prefix, runtime)
                self.head_dim, self.max_positions = head_dim, max_positions
                self.table = None

            def tensor_specs(self):
                return {self.name("position_table"): TensorSpec((self.max_positions, self.head_dim))}

            def load(self, tensors):
                self.table = tensors[self.name("position_table")]

            def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, ctx, cache):
                ops = self.runtime.ops
                qkv = ops.dense(qkv, self.runtime.dtype).clone()
                offsets = self.table.index_select(0, ctx.positions.long())
                rotated = qkv[:, : (num_heads + num_kv_heads) * head_dim].view(qkv.shape[0], -1, head_dim)
                rotated += offsets[:, None, :]
                slots = ctx.slot_mapping[cache.group] if cache.writable else None
                return ops.rope_store(qkv, cache.k, cache.v, None, None, ctx.positions, slots, num_heads, num_kv_heads,
                                      head_dim, cache.block_size, ctx.max_context_len - 1, self.runtime.dtype)

    if "distance_bias" not in part_registry.POSITION_ENCODINGS:

        @part_registry.register_position_encoding("distance_bias")
        class DistanceBias(PositionEncoding):
            """A position encoding that leaves queries and keys as they are and acts inside the
            scores: head h's score of a key ``d`` positions back is lowered by ``slopes[h] * d``."""

            def __init__(self, prefix, runtime, *, slopes):
                super().__init__(prefix, runtime)
                self.slopes = torch.tensor(list(slopes), dtype=torch.float32, device=runtime.device)

            def score_slopes(self, num_heads):
                assert self.slopes.numel() == num_heads
                return self.slopes

            def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, ctx, cache):
                ops = self.runtime.ops
                slots = ctx.slot_mapping[cache.group] if cache.writable else None
                return ops.rope_store(ops.dense(qkv, self.runtime.dtype), cache.k, cache.v, None, None, ctx.positions, slots,
                                      num_heads, num_kv_heads, head_dim, cache.block_size, ctx.max_context_len - 1,
                                      self.runtime.dtype)

    if "scaled_table" not in part_registry.EMBEDDINGS:

        @part_registry.register_embedding("scaled_table")
        class ScaledTable(Embedding):
            """Another embedding: the table's row times a constant."""

            def __init__(self, prefix, runtime, *, vocab_size, hidden_size, multiplier):
                super().__init__(prefix, runtime)
                self.shape, self.multiplier, self.weight = (vocab_size, hidden_size), float(multiplier), None

            def tensor_specs(self):
                return {self.name("weight"): TensorSpec(self.shape)}

            def load(self, tensors):
                self.weight = tensors[self.name("weight")]

            def forward(self, token_ids, ctx):
                return self.runtime.ops.embed(self.weight, token_ids) * self.multiplier

    if "biased_head" not in part_registry.HEADS:

        @part_registry.register_head("biased_head")
        class BiasedHead(Head):
            """Another head: norm, a matrix of its own, a scale on the scores and a bias per token id."""

            def __init__(self, prefix, runtime, *, vocab_size, hidden_size, norm, scale):
                super().__init__(prefix, runtime)
                self.vocab, self.hidden, self.scale = vocab_size, hidden_size, float(scale)
                self.norm = part_registry.build_part("norm", norm, "model.norm", runtime)
                self.weight = self.bias = None

            def tensor_specs(self):
                return {**self.norm.tensor_specs(), self.name("weight"): TensorSpec((self.vocab, self.hidden)),
                        self.name("bias"): TensorSpec((self.vocab,))}

            def load(self, tensors):
                self.norm.load(tensors)
                self.weight, self.bias = tensors[self.name("weight")], tensors[self.name("bias")].float()

            def forward(self, stream, rows):
                hidden = self.norm.forward_residual(stream, rows)
                return self.runtime.ops.linear_float32_out(hidden, self.weight) * self.scale + self.bias

    if "ToyForCausalLM" not in arch_registry.ARCHITECTURES:

        def parse(data, name_or_path=""):
            return dict(data)

        def plan(cfg):
            hidden = cfg["hidden_size"]
            norm = PartSpec("rmsnorm", {"size": hidden, "eps": cfg["eps"]})
            ff = PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": cfg["intermediate_size"]})
            attention = PartSpec("gqa_attention", {
                "hidden_size": hidden, "num_heads": cfg["heads"], "num_kv_heads": cfg["kv_heads"], "head_dim": cfg["head_dim"],
                "scale": cfg["head_dim"] ** -0.5, "qkv_bias": True, "out_bias": False, "window": None,
                "position": PartSpec("rope", {"head_dim": cfg["head_dim"], "theta": 1e4, "scaling_factor": 1.0, "max_positions": 256})})
            learned = PartSpec("gqa_attention", dict(attention.params, position=PartSpec(
                "learned_positions", {"head_dim": cfg["head_dim"], "max_positions": 128})))
            biased = PartSpec("gqa_attention", dict(attention.params, position=PartSpec(
                "distance_bias", {"slopes": cfg["slopes"]})))
            toy = PartSpec("running_mean", {"hidden_size": hidden})
            routed = PartSpec("top1_experts", {"hidden_size": hidden, "intermediate_size": cfg["intermediate_size"],
                                               "num_experts": cfg["experts"]})
            sink = PartSpec("sink_attention", {"hidden_size": hidden, "key_dim": cfg["sink_key_dim"],
                                               "value_dim": cfg["sink_value_dim"], "buckets": cfg["sink_buckets"]})
            mixers = {"attention": attention, "attention_learned": learned, "attention_biased": biased, "state": toy,
                      "sink": sink}
            layers = []
            for index, kind in enumerate(cfg["mixers"]):  # mixer and feed-forward are chosen layer by layer
                block = PartSpec("prenorm", {"mixer": mixers[kind],
                                             "feed_forward": routed if cfg["feed_forwards"][index] == "routed" else ff,
                                             "mixer_norm": norm, "ff_norm": norm})
                layers.append(LayerSpec(f"model.layers.{index}", block))
            schedule = tuple(LayerCall(layer, cache_of) for layer, cache_of in cfg["schedule"])
            embedding = PartSpec("scaled_table", {"vocab_size": cfg["vocab_size"], "hidden_size": hidden,
                                                  "multiplier": cfg["embedding_multiplier"]})
            head = PartSpec("biased_head", {"vocab_size": cfg["vocab_size"], "hidden_size": hidden, "norm": norm,
                                            "scale": cfg["logit_scale"]})
            return ModelPlan(vocab_size=cfg["vocab_size"], hidden_size=hidden, layers=tuple(layers), schedule=schedule,
                             embedding=embedding, head=head)

        arch_registry.register_architecture("ToyForCausalLM", parse, plan)


def toy_plain_logits(cfg, tensors, tokens):
    """The toy model by the plain functions: whole sequence, no cache."""
    values = {"heads": cfg["heads"], "kv_heads": cfg["kv_heads"], "head_dim": cfg["head_dim"], "theta": 1e4,
              "rope_factor": 1.0, "eps": cfg["eps"]}
    h = tensors["model.embed_tokens.weight"][torch.tensor(tokens)] * cfg["embedding_multiplier"]
    pos = torch.arange(len(tokens))
    distance = (pos[None, :] - pos[:, None]).float()  # [query, key]: key position less query position
    kv_of_call = {}
    for call, (layer, cache_of) in enumerate(cfg["schedule"]):
        p = f"model.layers.{layer}"
        x = plain.rms_norm(h, tensors[f"{p}.input_layernorm.weight"], cfg["eps"])
        if cfg["mixers"][layer].startswith("attention"):
            heads, kvh, dim = cfg["heads"], cfg["kv_heads"], cfg["head_dim"]
            if cfg["mixers"][layer] == "attention":
                angles = plain.rope_angles(pos, dim, 1e4)
                encode = lambda t: plain.apply_rope(t, angles)
            elif cfg["mixers"][layer] == "attention_biased":
                encode = lambda t: t
            else:
                table = tensors[f"{p}.self_attn.position_table"]
                encode = lambda t: t + table[pos][:, None, :]
            q = (x @ tensors[f"{p}.self_attn.q_proj.weight"].T + tensors[f"{p}.self_attn.q_proj.bias"]).view(-1, heads, dim)
            q = encode(q)
            if cache_of is None:
                k = (x @ tensors[f"{p}.self_attn.k_proj.weight"].T + tensors[f"{p}.self_attn.k_proj.bias"]).view(-1, kvh, dim)
                v = (x @ tensors[f"{p}.self_attn.v_proj.weight"].T + tensors[f"{p}.self_attn.v_proj.bias"]).view(-1, kvh, dim)
                kv_of_call[call] = (encode(k), v)
            k, v = kv_of_call[call if cache_of is None else cache_of]
            if cfg["mixers"][layer] == "attention_biased":
                # scores + slope * (key - query), written out: the plain attention has no such term
                mask = plain.attention_mask(pos, len(tokens), None)
                mixed = torch.empty_like(q)
                for head in range(heads):
                    scores = (q[:, head] @ k[:, head // (heads // kvh)].T) * dim ** -0.5 + cfg["slopes"][head] * distance
                    probs = torch.softmax(scores.masked_fill(~mask, float("-inf")), dim=-1)
                    mixed[:, head] = probs @ v[:, head // (heads // kvh)]
            else:
                mixed = plain.attention(q, k, v, plain.attention_mask(pos, len(tokens), None), dim ** -0.5)
            mixed = mixed.reshape(len(tokens), -1) @ tensors[f"{p}.self_attn.o_proj.weight"].T
        elif cfg["mixers"][layer] == "sink":
            a = f"{p}.self_attn"
            q = x @ tensors[f"{a}.q.weight"].T + tensors[f"{a}.bucket_table"][pos // 5]
            k, v = x @ tensors[f"{a}.k.weight"].T, x @ tensors[f"{a}.v.weight"].T
            mask = plain.attention_mask(pos, len(tokens), None)
            scores = (q @ k.T) * cfg["sink_key_dim"] ** -0.5  # written out: the plain attention has one width for keys and values
            mixed = torch.softmax(scores.masked_fill(~mask, float("-inf")), dim=-1) @ v
            mean = torch.cumsum(x, dim=0) / torch.arange(1, len(tokens) + 1)[:, None]
            mixed = mixed @ tensors[f"{a}.o.weight"].T + mean @ tensors[f"{a}.sink.weight"].T
        else:
            mean = torch.cumsum(x, dim=0) / torch.arange(1, len(tokens) + 1)[:, None]
            mixed = mean @ tensors[f"{p}.self_attn.mix.weight"].T
        h = h + mixed
        x = plain.rms_norm(h, tensors[f"{p}.post_attention_layernorm.weight"], cfg["eps"])
        if cfg["feed_forwards"][layer] == "routed":
            choice = (x @ tensors[f"{p}.mlp.router.weight"].T).argmax(dim=-1)
            h = h + torch.stack([
                plain.swiglu_mlp(x[t:t + 1], *(tensors[f"{p}.mlp.experts.{int(choice[t])}.{n}_proj.weight"]
                                               for n in ("gate", "up", "down")))[0]
                for t in range(len(tokens))])
        else:
            h = h + plain.swiglu_mlp(x, *(tensors[f"{p}.mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
    h = plain.rms_norm(h, tensors["model.norm.weight"], cfg["eps"])
    return (h @ tensors["lm_head.weight"].T) * cfg["logit_scale"] + tensors["lm_head.bias"]


TOY_CONFIG = {
    "architectures": ["ToyForCausalLM"], "hidden_size": 40, "intermediate_size": 56, "vocab_size": 97, "heads": 5,
    "kv_heads": 1, "head_dim": 16, "eps": 1e-5, "experts": 3,
    "embedding_multiplier": 1.5, "logit_scale": 0.5, "slopes": [0.5, 0.25, 0.125, 0.0625, 0.03125],
    "sink_key_dim": 8, "sink_value_dim": 24, "sink_buckets": 64,
    "mixers": ["attention", "state", "attention", "attention_learned", "attention_biased", "sink"],
    "feed_forwards": ["swiglu", "routed", "swiglu", "routed", "swiglu", "swiglu"],
    # layer 0, the stateful layer (with a routed feed-forward), layer 0 AGAIN (weights reused, a
    # cache of its own), layer 2 reading the cache of the first call instead of keeping one, then
    # a layer whose attention takes learned positions instead of rotation, then one whose position
    # encoding is a bias on the scores, then a layer that keeps pages (values three times as wide
    # as its keys) and state, and reads a step field of its own.
    "schedule": [[0, None], [1, None], [0, None], [2, 0], [3, None], [4, None], [5, None]],
}


@pytest.fixture(scope="module")
def toy_folder(tmp_path_factory):
    from turboserve_amd.weights.random_init import write_random_model

    register_toy_architecture()
    return write_random_model(TOY_CONFIG, tmp_path_factory.mktemp("toy"), seed=5, dtype=torch.float32)


def test_toy_model_is_data(toy_folder):
    from turboserve_amd.cache.layout import CacheLayout
    from turboserve_amd.weights.random_init import describe_model

    _, model = describe_model(TOY_CONFIG)
    layout = CacheLayout.from_model(model)
    assert [u and u[0] for u in layout.entry_units[:6]] == ["pages", "state", "pages", "reads", "pages", "pages"]
    assert layout.entry_units[6] == (("pages", 1, 0), ("state", 1)), "the last layer keeps pages and state"
    assert len(layout.groups) == 2 and layout.groups[0].entries == (0, 2, 4, 5) and layout.groups[1].entries == (6,)
    assert (layout.groups[1].head_dim, layout.groups[1].value_width) == (8, 24)
    assert [entry for entry, _ in layout.state_entries] == [1, 6]
    assert [one.name for one in model.step_fields()] == ["position_bucket"]
    assert "model.layers.5.self_attn.bucket_table" in model.tensor_specs()
    names = list(model.tensor_specs())
    assert "model.layers.1.self_attn.mix.weight" in names and "model.layers.2.self_attn.q_proj.weight" in names
    assert "model.layers.1.mlp.experts.2.down_proj.weight" in names and "model.layers.1.mlp.router.weight" in names
    assert "model.layers.3.self_attn.position_table" in names and "model.layers.0.mlp.gate_proj.weight" in names
    assert "lm_head.bias" in names and "model.norm.weight" in names and names[0] == "model.embed_tokens.weight"


@pytest.mark.parametrize("cut", ["whole", "prefix_then_single", "portions", "mixed"])
def test_toy_architecture_steps_like_its_plain_form(toy_folder, cut):
    """Registered, built, loaded and stepped through the ordinary replay path under every
    cutting: the state slot carries the running mean across steps, padded graph rows and
    requests that end and free their slot for the next one."""
    from test_gpu_replay import CUTS, run_trace

    register_toy_architecture()
    raw, tensors = tiny.read_model_dir(toy_folder)
    requests = {f"t{i}": tiny.random_tokens(97, n, 300 + i) for i, n in enumerate([9, 41, 23, 60, 34])}
    steps = CUTS[cut](requests)
    got = th.collect(steps, run_trace(toy_folder, "float32", 8, steps), requests)
    for rid, toks in requests.items():
        want = toy_plain_logits(raw, tensors, toks)
        assert float((got[rid] - want).abs().max()) <= 1e-4, f"{cut} {rid}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_generates_through_the_engine_and_the_command_line(toy_folder, tmp_path, dtype, capsys):
    """The toy architecture (its configuration is a plain mapping with names of its own)
    through ``LLMEngine`` with the cache sized from the device's memory, and through the command
    line's ``generate`` and ``kv-size``: nothing in the engine, the sizing or the command line
    reads an architecture's configuration fields."""
    import json
    import re

    from turboserve_amd import cli
    from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
    from turboserve_amd.engine.llm_engine import LLMEngine
    from turboserve_amd.sampling.params import SamplingParams
    from turboserve_amd.weights.random_init import write_random_model

    register_toy_architecture()
    folder = toy_folder
    if dtype == "bfloat16":
        # Without the routed feed-forward: a router's near-tie may fall to another expert in
        # bfloat16, which is a different function, not a rounding error.
        dense = {**TOY_CONFIG, "feed_forwards": ["swiglu"] * 6}
        folder = write_random_model(dense, tmp_path / "toy_bf16", seed=5, dtype=torch.bfloat16, std=0.1)
    raw, tensors = tiny.read_model_dir(folder)
    prompts = [tiny.random_tokens(97, n, 40 + n) for n in (3, 12, 29)]
    new = 6

    def check_tokens(prompt, got):
        tokens = list(prompt)
        assert len(got) == new
        for token in got:
            logits = toy_plain_logits(raw, tensors, tokens)[-1]
            slack = 0.0 if dtype == "float32" else 3e-2 * float(logits.abs().max())
            assert float(logits.max() - logits[token]) <= slack, f"{dtype}: token {token} is not the plain argmax"
            tokens.append(token)

    config = EngineConfig(model=str(folder), dtype=dtype, max_model_len=64, scheduler=SchedulerConfig(
        max_num_seqs=4, max_num_batched_tokens=16, block_size=8))
    with LLMEngine(config) as engine:
        assert engine.sizing is not None and engine.sizing.reason == "max_model_len cap"
        assert engine.sizing.num_blocks == [32, 32] and engine.sizing.activation_bytes > 0
        outputs = engine.generate(prompts, SamplingParams(max_tokens=new, temperature=0.0, ignore_eos=True))
        for prompt, output in zip(prompts, outputs):
            check_tokens(prompt, output.new_token_ids)
        engine.scheduler.check_invariants()
    capsys.readouterr()
    args = ["engine", "generate", "--model", str(folder), "--dtype", dtype, "--max-tokens", str(new), "--ignore-eos",
            "--num-blocks", "32", "--block-size", "8"]
    assert cli.main(args + [a for p in prompts for a in ("--prompt-ids", ",".join(map(str, p)))]) == 0
    shown = [json.loads(m) for m in re.findall(r"^output \d+: (\[.*\])$", capsys.readouterr().out, flags=re.M)]
    assert len(shown) == len(prompts)
    for prompt, got in zip(prompts, shown):
        check_tokens(prompt, got)
    assert cli.main(["engine", "kv-size", "--model", str(folder), "--dtype", dtype, "--max-model-len", "64", "--block-size", "8"]) == 0
    sizing = capsys.readouterr().out
    sizing = json.loads(sizing[sizing.index("{"):])
    assert sizing["reason"] == "max_model_len cap" and sizing["num_blocks"] == [8 * 64, 8 * 64] and sizing["activation_bytes"] > 0


def test_a_part_can_keep_the_model_out_of_graphs(toy_folder):
    """A part that reads device data back on the host says `capturable = False`; the runner
    then records no HIP graph and steps the model eagerly, with the same logits."""
    from test_gpu_replay import run_trace
    from turboserve_amd.engine.replay import TraceReplayer
    from turboserve_amd.parts import registry as part_registry

    register_toy_architecture()
    routed = part_registry.FEED_FORWARDS["top1_experts"]
    raw, tensors = tiny.read_model_dir(toy_folder)
    requests = {"a": tiny.random_tokens(97, 20, 1), "b": tiny.random_tokens(97, 33, 2)}
    steps = th.prefix_then_single(requests)
    assert TraceReplayer(toy_folder, dtype="float32", max_tokens=128, page_size=8).runner.graphs is not None
    recorded = th.collect(steps, run_trace(toy_folder, "float32", 8, steps), requests)
    routed.capturable = False
    try:
        assert TraceReplayer(toy_folder, dtype="float32", max_tokens=128, page_size=8).runner.graphs is None
        eager = th.collect(steps, run_trace(toy_folder, "float32", 8, steps), requests)
    finally:
        routed.capturable = True
    for rid in requests:
        assert torch.equal(recorded[rid], eager[rid])


# -- long decoding, first tokens ----------------------------------------------------------------------


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(tmp_path, dtype):
    """A request that starts from a single token and is decoded token by token for 300 steps
    (through a window of 40 keys and pages of 32 that are given back on the way)."""
    from test_gpu_replay import check, run_trace

    config, seed, page = tiny.TINY["C"]
    folder = tiny.make_model_dir(tmp_path, config, seed, torch.float32 if dtype == "float32" else torch.bfloat16)
    tokens = tiny.random_tokens(config["vocab_size"], 301, 77)
    steps = [{"step": i, "entries": [{"id": "long", "tokens": [t], "want": [0]}], "end": ["long"] if i == 300 else []}
             for i, t in enumerate(tokens)]
    outputs = run_trace(folder, dtype, page, steps, max_tokens=320)
    got = th.collect(steps, outputs, {"long": tokens})
    check(got, {"long": tiny.plain_logits(folder, tokens)}, dtype, "long decoding")
