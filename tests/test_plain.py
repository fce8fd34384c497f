"""The plain implementation pinned by what fixes it beside the reference's text: vectors the
reference's own tests hold, special cases that reduce to a library routine, and invariants,
each chosen so that a plausible mistake (a wrong sign or pairing, a norm in the wrong place, a
dropped bias) fails it."""

from __future__ import annotations

import math

import pytest
import torch
import torch.nn.functional as F

import tiny
from plain import qwen2_plain as plain


# -- RMSNorm ----------------------------------------------------------------------------------------


def test_rms_norm_is_the_library_routine_in_32_bit():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 96, generator=g) * 3
    w = 1 + 0.2 * torch.randn(96, generator=g)
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (96,), w, 1e-5), rtol=1e-6, atol=1e-6)
    ref64 = x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-5) * w.double()
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-5).double(), ref64, rtol=1e-6, atol=1e-6)


def test_rms_norm_unit_rms_and_scale_invariance():
    x = torch.randn(4, 64, generator=torch.Generator().manual_seed(1))
    y = plain.rms_norm(x, torch.ones(64), 0.0)
    torch.testing.assert_close((y ** 2).mean(-1), torch.ones(4), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(plain.rms_norm(7.0 * x, torch.ones(64), 1e-12), y, rtol=1e-5, atol=1e-5)
    # eps sits inside the square root, added to the mean square (not to the rms, not to the sum).
    tiny_x = torch.full((1, 4), 1e-3)
    expect = 1e-3 / math.sqrt(1e-6 + 1e-2)
    torch.testing.assert_close(plain.rms_norm(tiny_x, torch.ones(4), 1e-2), torch.full((1, 4), expect))


def test_rms_norm_rounds_to_the_input_type_before_the_gain():
    """src/turboserve/engine/model/layers.py:208: ``weight * x32.to(input_dtype)``."""
    g = torch.Generator().manual_seed(2)
    x = torch.randn(32, 128, generator=g).bfloat16()
    w = (1 + 0.3 * torch.randn(128, generator=g)).bfloat16()
    normed = (x.float() * torch.rsqrt((x.float() ** 2).mean(-1, keepdim=True) + 1e-6)).bfloat16()
    assert torch.equal(plain.rms_norm(x, w, 1e-6), w * normed)
    assert plain.rms_norm(x, w, 1e-6).dtype == torch.bfloat16


# -- rotary -----------------------------------------------------------------------------------------


def test_rope_frequencies_and_identity_at_position_zero():
    angles = plain.rope_angles(torch.tensor([0, 1, 10]), 8, 10000.0)
    assert angles.shape == (3, 4) and angles.dtype == torch.float32
    assert torch.equal(angles[0], torch.zeros(4))
    expected = torch.tensor([10000.0 ** (-2 * i / 8) for i in range(4)])
    torch.testing.assert_close(angles[1], expected, rtol=1e-6, atol=0)  # inv_freq[0] = 1, theta^(-2i/D)
    torch.testing.assert_close(angles[2], 10 * expected, rtol=1e-6, atol=0)
    x = torch.randn(3, 2, 8, generator=torch.Generator().manual_seed(3))
    torch.testing.assert_close(plain.apply_rope(x, angles)[0], x[0])


def test_rope_pairs_the_halves_and_turns_counterclockwise():
    """Pairs are (i, i + D/2) (src/turboserve/engine/model/layers.py:214-222); an interleaved
    pairing or a flipped sign fails here."""
    dim = 8
    x = torch.zeros(1, 1, dim)
    x[0, 0, 1] = 1.0  # first element of pair (1, 5)
    angles = plain.rope_angles(torch.tensor([3]), dim, 100.0)
    out = plain.apply_rope(x, angles)[0, 0]
    a = float(angles[0, 1])
    expect = torch.zeros(dim)
    expect[1], expect[5] = math.cos(a), math.sin(a)
    torch.testing.assert_close(out, expect, rtol=1e-6, atol=1e-7)
    # The reference's expression itself: x * cos + rotate_half(x) * sin with cat(freqs, freqs).
    y = torch.randn(4, 3, dim, generator=torch.Generator().manual_seed(4))
    pos = torch.tensor([0, 5, 6, 40])
    ang = plain.rope_angles(pos, dim, 100.0)
    emb = torch.cat((ang, ang), dim=-1)
    rotated = torch.cat((-y[..., dim // 2:], y[..., : dim // 2]), dim=-1)
    want = y * emb.cos().unsqueeze(1) + rotated * emb.sin().unsqueeze(1)
    torch.testing.assert_close(plain.apply_rope(y, ang), want, rtol=1e-6, atol=1e-6)


def test_rope_keeps_norms_and_depends_on_distance_only():
    g = torch.Generator().manual_seed(5)
    q = torch.randn(1, 1, 32, generator=g)
    k = torch.randn(1, 1, 32, generator=g)

    def score(m: int, n: int) -> float:
        qa = plain.apply_rope(q, plain.rope_angles(torch.tensor([m]), 32, 1e4))
        ka = plain.apply_rope(k, plain.rope_angles(torch.tensor([n]), 32, 1e4))
        return float((qa * ka).sum())

    assert score(7, 3) == pytest.approx(score(104, 100), abs=1e-4)
    assert score(7, 3) != pytest.approx(score(3, 7), abs=1e-3)  # not symmetric: the sign matters
    rotated = plain.apply_rope(q, plain.rope_angles(torch.tensor([77]), 32, 1e4))
    assert float(rotated.norm()) == pytest.approx(float(q.norm()), rel=1e-5)


def test_rope_linear_scaling_divides_positions():
    a = plain.rope_angles(torch.tensor([8, 20]), 16, 1e4, 4.0)
    b = plain.rope_angles(torch.tensor([2, 5]), 16, 1e4, 1.0)
    torch.testing.assert_close(a, b)


# -- attention --------------------------------------------------------------------------------------


def test_mask_vector_of_the_reference():
    """tests/unit/test_paged_attention.py:221-237 in the reference: 3 queries after 2 cached
    tokens; a single decode query sees everything."""
    expected = torch.tensor([[True, True, True, False, False], [True, True, True, True, False],
                             [True, True, True, True, True]])
    assert torch.equal(plain.attention_mask(torch.tensor([2, 3, 4]), 5, None), expected)
    assert bool(plain.attention_mask(torch.tensor([5]), 6, None).all())


def test_attention_is_scaled_dot_product_attention():
    g = torch.Generator().manual_seed(6)
    heads, kv_heads, dim, ctx = 6, 2, 8, 11
    q = torch.randn(ctx, heads, dim, generator=g)
    k = torch.randn(ctx, kv_heads, dim, generator=g)
    v = torch.randn(ctx, kv_heads, dim, generator=g)
    scale = dim ** -0.5
    assert scale == pytest.approx(8 ** -0.5)  # tests/unit/test_model_config.py:104
    kk = k.repeat_interleave(heads // kv_heads, dim=1)  # attention.py:197-199
    vv = v.repeat_interleave(heads // kv_heads, dim=1)

    def sdpa(qs, **kw):
        return F.scaled_dot_product_attention(qs.transpose(0, 1)[None], kk.transpose(0, 1)[None],
                                              vv.transpose(0, 1)[None], scale=scale, **kw)[0].transpose(0, 1)

    causal = plain.attention(q, k, v, plain.attention_mask(torch.arange(ctx), ctx, None), scale)
    torch.testing.assert_close(causal, sdpa(q, is_causal=True), rtol=1e-5, atol=1e-6)
    last = plain.attention(q[-1:], k, v, plain.attention_mask(torch.tensor([ctx - 1]), ctx, None), scale)
    torch.testing.assert_close(last, sdpa(q[-1:]), rtol=1e-5, atol=1e-6)
    chunk_mask = plain.attention_mask(torch.arange(ctx - 3, ctx), ctx, None)
    chunk = plain.attention(q[-3:], k, v, chunk_mask, scale)
    torch.testing.assert_close(chunk, sdpa(q[-3:], attn_mask=chunk_mask[None, None]), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(chunk, causal[-3:], rtol=1e-5, atol=1e-6)


def test_attention_single_key_returns_its_value():
    """tests/unit/test_paged_attention.py:196-218."""
    g = torch.Generator().manual_seed(7)
    q = torch.randn(1, 4, 8, generator=g)
    k = torch.randn(1, 2, 8, generator=g)
    v = torch.randn(1, 2, 8, generator=g)
    out = plain.attention(q, k, v, plain.attention_mask(torch.tensor([0]), 1, None), 8 ** -0.5)
    torch.testing.assert_close(out, v.repeat_interleave(2, dim=1))


def test_window_rule():
    """A window at least as long as the context changes nothing; a window of one leaves each
    token its own value; window W keeps exactly W keys ending at the query."""
    g = torch.Generator().manual_seed(8)
    ctx = 9
    q = torch.randn(ctx, 2, 8, generator=g)
    k = torch.randn(ctx, 2, 8, generator=g)
    v = torch.randn(ctx, 2, 8, generator=g)
    pos = torch.arange(ctx)
    full = plain.attention(q, k, v, plain.attention_mask(pos, ctx, None), 1.0)
    torch.testing.assert_close(plain.attention(q, k, v, plain.attention_mask(pos, ctx, ctx), 1.0), full)
    torch.testing.assert_close(plain.attention(q, k, v, plain.attention_mask(pos, ctx, 1), 1.0), v)
    mask = plain.attention_mask(pos, ctx, 3)
    assert mask.sum(-1).tolist() == [1, 2, 3, 3, 3, 3, 3, 3, 3]
    assert mask[8].tolist() == [False] * 6 + [True] * 3


# -- feed-forward, block, model ---------------------------------------------------------------------


def test_swiglu():
    g = torch.Generator().manual_seed(9)
    x = torch.randn(3, 16, generator=g)
    wg, wu, wd = (torch.randn(24, 16, generator=g), torch.randn(24, 16, generator=g), torch.randn(16, 24, generator=g))
    want = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    torch.testing.assert_close(plain.swiglu_mlp(x, wg, wu, wd), want, rtol=1e-5, atol=1e-5)
    assert float(plain.swiglu_mlp(x, wg, torch.zeros_like(wu), wd).abs().max()) == 0.0
    assert float(plain.swiglu_mlp(torch.zeros(1, 16), wg, wu, wd).abs().max()) == 0.0  # silu(0) = 0


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    config, seed, _ = tiny.TINY["B"]
    folder = tiny.make_model_dir(tmp_path_factory.mktemp("plainB"), config, seed, torch.float32)
    return tiny.read_model_dir(folder)


def test_zero_projections_make_every_layer_the_identity(model_b):
    """Pre-norm residual order: with all projections zero, logits = head(norm(embedding))."""
    config, tensors = model_b
    zeroed = {name: (torch.zeros_like(t) if "_proj." in name else t) for name, t in tensors.items()}
    tokens = [3, 1, 4, 1, 5]
    hidden = plain.rms_norm(tensors["model.embed_tokens.weight"][tokens], tensors["model.norm.weight"], 1e-5)
    want = hidden @ tensors["lm_head.weight"].T
    torch.testing.assert_close(plain.forward_logits(config, zeroed, tokens), want, rtol=1e-5, atol=1e-6)


def test_qkv_bias_is_used(model_b):
    """Zero weights leave the bias: dropping a q/k/v bias changes the logits."""
    config, tensors = model_b
    changed = dict(tensors)
    changed["model.layers.0.self_attn.v_proj.bias"] = tensors["model.layers.0.self_attn.v_proj.bias"] + 0.5
    a = plain.forward_logits(config, tensors, [1, 2, 3])
    b = plain.forward_logits(config, changed, [1, 2, 3])
    assert float((a - b).abs().max()) > 1e-3


def test_shifting_all_positions_changes_nothing(model_b):
    """Only distances count (rotary encoding, causal and window masks)."""
    config, tensors = model_b
    tokens = tiny.random_tokens(config["vocab_size"], 30, 1)
    a = plain.forward_logits(config, tensors, tokens)
    b = plain.forward_logits(config, tensors, tokens, positions=range(50, 80))
    torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-4)


def test_prefix_logits_do_not_depend_on_what_follows(model_b):
    config, tensors = model_b
    tokens = tiny.random_tokens(config["vocab_size"], 25, 2)
    torch.testing.assert_close(plain.forward_logits(config, tensors, tokens)[:10],
                               plain.forward_logits(config, tensors, tokens[:10]), rtol=1e-5, atol=1e-5)


def test_window_layers_of_config_b(model_b):
    """Layer 0 keeps every key, layers 1 and 2 see 16: up to 16 tokens the window does not
    show, beyond it does."""
    config, tensors = model_b
    values = plain.cfg_values(config)
    assert [plain.layer_window(values, layer) for layer in range(3)] == [None, 16, 16]
    no_window = dict(config, use_sliding_window=False)
    short = tiny.random_tokens(config["vocab_size"], 16, 3)
    long = tiny.random_tokens(config["vocab_size"], 40, 4)
    torch.testing.assert_close(plain.forward_logits(config, tensors, short), plain.forward_logits(no_window, tensors, short))
    diff = (plain.forward_logits(config, tensors, long) - plain.forward_logits(no_window, tensors, long)).abs().max(dim=-1).values
    assert float(diff[:16].max()) == 0.0 and float(diff[16:].min()) > 0.0


def test_tied_head_uses_the_embedding(tmp_path):
    config, seed, _ = tiny.TINY["A"]
    raw, tensors = tiny.read_model_dir(tiny.make_model_dir(tmp_path, config, seed, torch.float32))
    assert "lm_head.weight" not in tensors
    hidden = plain.forward_hidden(raw, tensors, [5, 6, 7])
    torch.testing.assert_close(plain.logits_from_hidden(raw, tensors, hidden), hidden @ tensors["model.embed_tokens.weight"].T)
    assert plain.logits_from_hidden(raw, tensors, hidden).dtype == torch.float32


def test_kv_bytes_of_the_7b_shape():
    """57,344 bytes per token = 2 * 28 * 4 * 128 * 2 (docs/results.md:299 in the reference)."""
    shape = {"num_hidden_layers": 28, "hidden_size": 3584, "num_attention_heads": 28, "num_key_value_heads": 4,
             "intermediate_size": 18944, "vocab_size": 152064}
    assert plain.expected_kv_bytes_per_token(shape, 2) == 57344
    assert 65319 * 16 * 57344 == 59_930_443_776


# -- sampling ---------------------------------------------------------------------------------------


def test_philox_known_answers():
    """Known-answer vectors of Philox-4x32-10 (the Random123 distribution's kat_vectors)."""
    assert plain.philox4x32_10((0, 0, 0, 0), (0, 0)) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert plain.philox4x32_10((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2) == [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]
    assert plain.philox4x32_10((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0)) == [
        0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]
    u = [plain.philox_uniform(7, i) for i in range(2000)]
    assert all(0.0 <= x < 1.0 for x in u) and abs(sum(u) / len(u) - 0.5) < 0.03


def test_sampling_stage_vectors_of_the_reference():
    """tests/unit/test_sampler.py:55-104 in the reference."""
    logits = torch.tensor([0.0, 1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0])
    support = lambda t: {i for i, v in enumerate(t.tolist()) if v != float("-inf")}
    assert support(plain.top_k_filter(logits, 2)) == {6, 7}
    assert support(plain.top_k_filter(logits, 0)) == set(range(8))
    assert support(plain.top_k_filter(logits, 100)) == set(range(8))
    probs = torch.log(torch.tensor([0.5, 0.25, 0.15, 0.10]))
    assert support(plain.top_p_filter(probs, 0.4)) == {0}
    assert support(plain.top_p_filter(probs, 0.55)) == {0, 1}
    assert support(plain.top_p_filter(probs, 0.8)) == {0, 1, 2}
    assert support(plain.top_p_filter(probs, 0.95)) == {0, 1, 2, 3}
    assert support(plain.top_p_filter(probs, 1.0)) == {0, 1, 2, 3}
    out = plain.repetition_penalty(torch.tensor([2.0, -2.0, 0.5, 0.0]), [0, 1, 0, 0], 2.0)
    assert out.tolist() == [1.0, -4.0, 0.5, 0.0]  # divided, multiplied, once per token however often it was seen


def test_greedy_ignores_truncation_and_low_temperature_approaches_it():
    logits = torch.randn(16, generator=torch.Generator().manual_seed(3))
    token, _ = plain.sample_token(logits, temperature=0.0, top_k=3, top_p=0.5)
    assert token == int(logits.argmax())
    cold, _ = plain.sample_token(logits, temperature=1e-4, seed=5, draw_index=9)
    assert cold == int(logits.argmax())
    assert plain.log_softmax_at(logits, token) == pytest.approx(float(torch.log_softmax(logits, -1)[token]), abs=1e-6)


def test_draw_is_the_inverse_cdf():
    logits = torch.log(torch.tensor([0.1, 0.2, 0.3, 0.4]))
    for seed in range(50):
        token, cdf = plain.sample_token(logits, temperature=1.0, seed=seed, draw_index=seed * 3)
        u = plain.philox_uniform(seed, seed * 3)
        bounds = [0.0, 0.1, 0.3, 0.6, 1.0]
        assert bounds[token] <= u + 1e-9 and u < bounds[token + 1] + 1e-9
        assert float(cdf[-1]) == pytest.approx(1.0)
