"""Plain, slow Qwen2 forward pass: whole sequences, no cache, no paging, one function per part.

This file is the oracle of the test suite. It shares no code with ``turboserve_amd``: it reads
a raw ``config.json`` mapping and a ``{tensor name: tensor}`` mapping (Hugging Face names) and
computes with ordinary torch tensor arithmetic on the CPU.  Every function cites the lines of
the reference (paths under its ``src/turboserve/`` and ``tests/``) whose formula it restates.

Conventions: ``T`` tokens of ONE sequence at positions ``0..T-1`` unless ``positions`` says
otherwise; ``H`` hidden size; ``Hq``/``Hkv`` query/KV heads; ``D`` head size.
"""

from __future__ import annotations

from collections.abc import Mapping, Sequence

import torch

Tensors = Mapping[str, torch.Tensor]


# ---------------------------------------------------------------------------------------------
# configuration values, with the reference's defaults
# ---------------------------------------------------------------------------------------------


def cfg_values(cfg: Mapping) -> dict:
    """The numbers the formulas need, with the defaults of the reference.

    src/turboserve/engine/model/model_config.py:276-308 (heads, kv heads default = heads,
    head_dim default hidden/heads, eps default 1e-6, tie default false) and :109-123
    (rope_theta default 10000, ``linear`` scaling factor).  The sliding-window keys are not
    read by the reference (it rejects them, model_config.py:270-274); the rule used here is:
    layer ``l`` is windowed iff ``use_sliding_window and l >= max_window_layers``.
    """
    heads = int(cfg["num_attention_heads"])
    hidden = int(cfg["hidden_size"])
    rope = cfg.get("rope_parameters")
    if not isinstance(rope, Mapping):
        rope = {}
        if "rope_theta" in cfg:
            rope["rope_theta"] = cfg["rope_theta"]
        if isinstance(cfg.get("rope_scaling"), Mapping):
            rope.update(cfg["rope_scaling"])
    rope_type = str(rope.get("rope_type") or rope.get("type") or "default")
    return {
        "hidden": hidden,
        "layers": int(cfg["num_hidden_layers"]),
        "heads": heads,
        "kv_heads": int(cfg.get("num_key_value_heads", heads)),
        "head_dim": int(cfg.get("head_dim") or hidden // heads),
        "intermediate": int(cfg["intermediate_size"]),
        "vocab": int(cfg["vocab_size"]),
        "eps": float(cfg.get("rms_norm_eps", 1e-6)),
        "theta": float(rope.get("rope_theta", 10000.0)),
        "rope_factor": float(rope.get("factor", 1.0)) if rope_type == "linear" else 1.0,
        "tied": bool(cfg.get("tie_word_embeddings", False)),
        "use_window": bool(cfg.get("use_sliding_window", False)) and bool(cfg.get("sliding_window")),
        "window": int(cfg.get("sliding_window") or 0),
        "max_window_layers": int(cfg.get("max_window_layers", 0) or 0),
    }


def layer_window(values: Mapping, layer: int) -> int | None:
    """Window of ``layer`` (number of keys a query sees, itself included) or ``None``."""
    if values["use_window"] and layer >= values["max_window_layers"]:
        return values["window"]
    return None


# ---------------------------------------------------------------------------------------------
# parts
# ---------------------------------------------------------------------------------------------


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``weight * (x32 * rsqrt(mean(x32^2) + eps)).to(x.dtype)``.

    src/turboserve/engine/model/layers.py:202-208: variance and normalisation in fp32, cast
    back to the input dtype, THEN the gain.
    """
    x32 = x.to(torch.float32)
    variance = (x32 * x32).mean(dim=-1, keepdim=True)
    normed = x32 * torch.rsqrt(variance + eps)
    return weight * normed.to(x.dtype)


def rope_angles(positions: torch.Tensor, head_dim: int, theta: float, factor: float = 1.0) -> torch.Tensor:
    """``[T, D/2]`` fp32 angles ``(pos / factor) * theta^(-2i/D)``.

    src/turboserve/engine/model/layers.py:258-262 (inv_freq) and :281-284 (positions divided
    by the linear scaling factor, outer product).
    """
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    pos = positions.to(torch.float32)
    if factor != 1.0:
        pos = pos / factor
    return torch.outer(pos, inv_freq)


def apply_rope(x: torch.Tensor, angles: torch.Tensor) -> torch.Tensor:
    """Rotate ``x [T, heads, D]`` by ``angles [T, D/2]``; pairs are ``(i, i + D/2)``.

    src/turboserve/engine/model/layers.py:214-222 (``rotate_half``: ``[x1, x2] -> [-x2, x1]``)
    and :298-302 (``x*cos + rotate_half(x)*sin`` with ``cos = cat(freqs, freqs).cos()``).
    Written out per half: ``out1 = x1*cos - x2*sin``; ``out2 = x2*cos + x1*sin``.
    """
    half = x.shape[-1] // 2
    cos = angles.cos().to(x.dtype).unsqueeze(1)
    sin = angles.sin().to(x.dtype).unsqueeze(1)
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)


def attention_mask(query_positions: torch.Tensor, num_keys: int, window: int | None) -> torch.Tensor:
    """``[T, num_keys]`` bool, ``True`` = attend: key ``i <= p_q`` and, windowed, ``p_q - i < W``.

    src/turboserve/engine/model/attention.py:139-148: query ``j`` of ``q_len`` sits at absolute
    position ``ctx - q_len + j`` and sees keys up to and including itself.  The window bound is
    this build's rule (the reference has none).
    """
    keys = torch.arange(num_keys).unsqueeze(0)
    pq = query_positions.to(torch.long).unsqueeze(1)
    mask = keys <= pq
    if window is not None:
        mask = mask & ((pq - keys) < window)
    return mask


def attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    mask: torch.Tensor,
    scale: float,
) -> torch.Tensor:
    """Grouped-query attention by explicit formulas.

    ``q [Tq, Hq, D]``, ``k, v [Tk, Hkv, D]``, ``mask [Tq, Tk]`` -> ``[Tq, Hq, D]``.
    src/turboserve/engine/model/attention.py:196-209: KV head ``j`` serves query heads
    ``j*G .. j*G+G-1`` (``repeat_interleave(G, dim=1)``), scores ``q k^T * scale``, masked
    positions excluded from the softmax, output ``P v``.
    """
    heads, kv_heads = q.shape[1], k.shape[1]
    group = heads // kv_heads
    out = torch.empty_like(q)
    for h in range(heads):
        kh = h // group
        scores = (q[:, h, :].to(torch.float32) @ k[:, kh, :].to(torch.float32).T) * scale
        scores = scores.masked_fill(~mask, float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        out[:, h, :] = (probs @ v[:, kh, :].to(torch.float32)).to(q.dtype)
    return out


def swiglu_mlp(x: torch.Tensor, gate_w: torch.Tensor, up_w: torch.Tensor, down_w: torch.Tensor) -> torch.Tensor:
    """``down(silu(gate(x)) * up(x))`` with ``silu(z) = z * sigmoid(z)``.

    src/turboserve/engine/model/layers.py:61-67 (activation table) and :437-440.
    """
    gate = x @ gate_w.T
    up = x @ up_w.T
    act = gate * torch.sigmoid(gate)
    return (act * up) @ down_w.T


def attention_block(
    x: torch.Tensor,
    tensors: Tensors,
    prefix: str,
    values: Mapping,
    positions: torch.Tensor,
    window: int | None,
) -> torch.Tensor:
    """q/k/v projections with bias, head split, RoPE on q and k, attention, o projection.

    src/turboserve/engine/model/layers.py:376-391; biases on q/k/v and none on o are fixed
    for Qwen2 (model_config.py:285-288); scale is ``head_dim ** -0.5`` (model_config.py:224-227).
    """
    heads, kv_heads, dim = values["heads"], values["kv_heads"], values["head_dim"]
    T = x.shape[0]
    q = x @ tensors[f"{prefix}.q_proj.weight"].T + tensors[f"{prefix}.q_proj.bias"]
    k = x @ tensors[f"{prefix}.k_proj.weight"].T + tensors[f"{prefix}.k_proj.bias"]
    v = x @ tensors[f"{prefix}.v_proj.weight"].T + tensors[f"{prefix}.v_proj.bias"]
    q = q.view(T, heads, dim)
    k = k.view(T, kv_heads, dim)
    v = v.view(T, kv_heads, dim)
    angles = rope_angles(positions, dim, values["theta"], values["rope_factor"])
    q = apply_rope(q, angles)
    k = apply_rope(k, angles)
    # Whole sequence: the keys are this call's own tokens, key i sits at positions[i]; the
    # mask is written on absolute positions so that a shift of all positions changes nothing.
    rel = positions - positions[0]
    mask = attention_mask(rel, T, window)
    out = attention(q, k, v, mask, float(dim) ** -0.5)
    return out.reshape(T, heads * dim) @ tensors[f"{prefix}.o_proj.weight"].T


def decoder_layer(
    h: torch.Tensor, tensors: Tensors, layer: int, values: Mapping, positions: torch.Tensor
) -> torch.Tensor:
    """Pre-norm block: ``h += attn(norm1(h))``; ``h += mlp(norm2(h))``.

    src/turboserve/engine/model/layers.py:479-487.
    """
    p = f"model.layers.{layer}"
    x = rms_norm(h, tensors[f"{p}.input_layernorm.weight"], values["eps"])
    a = attention_block(x, tensors, f"{p}.self_attn", values, positions, layer_window(values, layer))
    h = h + a
    x = rms_norm(h, tensors[f"{p}.post_attention_layernorm.weight"], values["eps"])
    d = swiglu_mlp(
        x,
        tensors[f"{p}.mlp.gate_proj.weight"],
        tensors[f"{p}.mlp.up_proj.weight"],
        tensors[f"{p}.mlp.down_proj.weight"],
    )
    return h + d


def forward_hidden(
    cfg: Mapping, tensors: Tensors, token_ids: Sequence[int], positions: Sequence[int] | None = None
) -> torch.Tensor:
    """Embedding, every layer in order, final norm -> ``[T, H]``.

    src/turboserve/engine/model/model.py:105-108.
    """
    values = cfg_values(cfg)
    ids = torch.tensor(list(token_ids), dtype=torch.long)
    pos = torch.arange(len(ids)) if positions is None else torch.tensor(list(positions), dtype=torch.long)
    h = tensors["model.embed_tokens.weight"][ids]
    for layer in range(values["layers"]):
        h = decoder_layer(h, tensors, layer, values, pos)
    return rms_norm(h, tensors["model.norm.weight"], values["eps"])


def logits_from_hidden(cfg: Mapping, tensors: Tensors, hidden: torch.Tensor) -> torch.Tensor:
    """``(hidden @ lm_head^T).float()``; a tied model uses the embedding table.

    src/turboserve/engine/model/model.py:131-142 (tying) and :244.
    """
    values = cfg_values(cfg)
    head = tensors["model.embed_tokens.weight"] if values["tied"] else tensors["lm_head.weight"]
    return (hidden @ head.T).to(torch.float32)


def forward_logits(
    cfg: Mapping, tensors: Tensors, token_ids: Sequence[int], positions: Sequence[int] | None = None
) -> torch.Tensor:
    """``[T, V]`` fp32 logits of one whole sequence."""
    return logits_from_hidden(cfg, tensors, forward_hidden(cfg, tensors, token_ids, positions))


def as_float32(tensors: Tensors) -> dict[str, torch.Tensor]:
    """The same tensors widened to fp32 (values unchanged), for comparing a bf16 engine."""
    return {name: t.to(torch.float32) if t.is_floating_point() else t for name, t in tensors.items()}


# ---------------------------------------------------------------------------------------------
# generation and sampling
# ---------------------------------------------------------------------------------------------


def greedy_generate(cfg: Mapping, tensors: Tensors, prompt: Sequence[int], num_new: int) -> list[int]:
    """Argmax decoding by recomputing the whole sequence for every token."""
    tokens = list(prompt)
    for _ in range(num_new):
        logits = forward_logits(cfg, tensors, tokens)
        tokens.append(int(torch.argmax(logits[-1]).item()))
    return tokens[len(prompt):]


_PHILOX_M0 = 0xD2511F53
_PHILOX_M1 = 0xCD9E8D57
_PHILOX_W0 = 0x9E3779B9
_PHILOX_W1 = 0xBB67AE85
_MASK32 = 0xFFFFFFFF


def philox4x32_10(counter: Sequence[int], key: Sequence[int]) -> list[int]:
    """The Philox-4x32-10 block function (Salmon et al., "Parallel random numbers: as easy as
    1, 2, 3", 2011): four 32-bit words out for a four-word counter and a two-word key."""
    c = [int(v) & _MASK32 for v in counter]
    k0, k1 = int(key[0]) & _MASK32, int(key[1]) & _MASK32
    for _ in range(10):
        p0 = _PHILOX_M0 * c[0]
        p1 = _PHILOX_M1 * c[2]
        c = [
            ((p1 >> 32) ^ c[1] ^ k0) & _MASK32,
            p1 & _MASK32,
            ((p0 >> 32) ^ c[3] ^ k1) & _MASK32,
            p0 & _MASK32,
        ]
        k0 = (k0 + _PHILOX_W0) & _MASK32
        k1 = (k1 + _PHILOX_W1) & _MASK32
    return c


def philox_uniform(seed: int, index: int) -> float:
    """Uniform in ``[0, 1)`` for a request's ``index``-th draw.

    Counter ``(index, 0, 0, 0)``, key ``(seed & 2^32-1, seed >> 32)``; the result is the top
    24 bits of the first output word times ``2^-24``.  This is the engine's own rule (the
    reference draws with ``torch.multinomial``, core/sampler.py:285-296, whose stream a kernel
    cannot reproduce).
    """
    words = philox4x32_10((index & _MASK32, 0, 0, 0), (seed & _MASK32, (seed >> 32) & _MASK32))
    return (words[0] >> 8) * (1.0 / 16777216.0)


def repetition_penalty(logits: torch.Tensor, history: Sequence[int], penalty: float) -> torch.Tensor:
    """Seen tokens: a negative logit is multiplied by the penalty, any other divided by it.

    src/turboserve/engine/core/sampler.py:83-122.
    """
    out = logits.clone()
    if penalty == 1.0:
        return out
    for tok in set(history):
        out[tok] = out[tok] * penalty if out[tok] < 0 else out[tok] / penalty
    return out


def top_k_filter(logits: torch.Tensor, k: int) -> torch.Tensor:
    """Mask ``logits < k-th largest`` (ties at the threshold stay); ``k <= 0`` = off.

    src/turboserve/engine/core/sampler.py:138-148.
    """
    vocab = logits.shape[-1]
    if k <= 0 or k >= vocab:
        return logits
    threshold = torch.sort(logits, descending=True).values[k - 1]
    return logits.masked_fill(logits < threshold, float("-inf"))


def top_p_filter(logits: torch.Tensor, p: float) -> torch.Tensor:
    """Keep a token while the probability mass of the tokens strictly above it is ``<= p``.

    src/turboserve/engine/core/sampler.py:151-168 (``cumulative_before > p`` is removed).
    Equal logits form one group here (kept or dropped together); the reference's order among
    equal values is whatever its sort gives.
    """
    if p >= 1.0:
        return logits
    probs = torch.softmax(logits.to(torch.float64), dim=-1)
    keep = torch.zeros_like(logits, dtype=torch.bool)
    for i in range(logits.shape[-1]):
        mass_above = probs[logits > logits[i]].sum()
        keep[i] = bool(mass_above <= p)
    return logits.masked_fill(~keep, float("-inf"))


def sample_token(
    logits: torch.Tensor,
    *,
    temperature: float,
    seed: int = 0,
    draw_index: int = 0,
    top_k: int = 0,
    top_p: float = 1.0,
    penalty: float = 1.0,
    history: Sequence[int] = (),
) -> tuple[int, torch.Tensor]:
    """One row of sampling; returns ``(token, cdf)`` with ``cdf`` in fp64 (empty if greedy).

    Order of stages as src/turboserve/engine/core/sampler.py:216-238: penalty, temperature,
    top-k, top-p, then argmax for ``temperature == 0`` (greedy ignores the truncation,
    tests/unit/test_sampler.py:110-118) or a draw.  The draw is this engine's rule: the first
    token whose cumulative probability (vocabulary order) exceeds ``u = philox_uniform(seed,
    draw_index)``.
    """
    work = repetition_penalty(logits.to(torch.float32), history, penalty)
    if temperature <= 0.0:
        return int(torch.argmax(work).item()), torch.empty(0, dtype=torch.float64)
    work = work / temperature
    work = top_k_filter(work, top_k)
    work = top_p_filter(work, top_p)
    probs = torch.softmax(work.to(torch.float64), dim=-1)
    cdf = torch.cumsum(probs, dim=-1)
    u = philox_uniform(seed, draw_index)
    token = int(torch.searchsorted(cdf, torch.tensor(u, dtype=torch.float64), right=True).item())
    token = min(token, logits.shape[-1] - 1)
    while probs[token] == 0.0 and token > 0:  # u beyond the last positive mass through rounding
        token -= 1
    return token, cdf


def log_softmax_at(logits: torch.Tensor, token: int) -> float:
    """``log_softmax(logits)[token]`` (logprobs are taken before temperature, sampler.py:222-238)."""
    return float(torch.log_softmax(logits.to(torch.float64), dim=-1)[token].item())


def expected_kv_bytes_per_token(cfg: Mapping, itemsize: int) -> int:
    """``2 * L * Hkv * D * itemsize`` (model_config.py:234-242)."""
    values = cfg_values(cfg)
    return 2 * values["layers"] * values["kv_heads"] * values["head_dim"] * itemsize
