"""Grouped-query attention over the paged cache (src/turboserve/engine/model/layers.py:311-391,
src/turboserve/engine/model/attention.py:213-295)."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.kernels.ops import attention_geometry_error
from turboserve_amd.parts.base import CacheNeed, Mixer, PagedKV, PagedKVView, PartSpec, Runtime, TensorSpec
from turboserve_amd.parts.registry import build_part, register_mixer


@register_mixer("gqa_attention")
class GroupedQueryAttention(Mixer):
    """q/k/v projections (optionally biased), position encoding, cache write, attention of every
    token over its request's keys up to itself (optionally only the last ``window``), output
    projection.

    The three projections are held as one ``[(Hq + 2 Hkv) D, H]`` matrix (the checkpoint keeps
    them apart; ``load`` concatenates), so a step does one product for them.  Scale is a
    parameter (``head_dim ** -0.5`` for Qwen2, model_config.py:224-227)."""

    def __init__(
        self,
        prefix: str,
        runtime: Runtime,
        *,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        scale: float,
        qkv_bias: bool,
        out_bias: bool,
        window: int | None,
        position: PartSpec,
    ) -> None:
        super().__init__(prefix, runtime)
        # Refused here, when the model is put together, not at the first step after the weights
        # have been read: a geometry that no attention kernel takes.
        refusal = attention_geometry_error(int(num_heads), int(num_kv_heads), int(head_dim))
        if refusal is not None:
            raise ValueError(f"{prefix or 'attention'}: {refusal}")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.scale = float(scale)
        self.qkv_bias = bool(qkv_bias)
        self.out_bias = bool(out_bias)
        self.window = None if window is None else int(window)
        self.position = build_part("position_encoding", position, prefix, runtime)
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        self.qkv_weight: torch.Tensor | None = None
        self.qkv_bias_tensor: torch.Tensor | None = None
        self.o_weight: torch.Tensor | None = None
        self.o_bias_tensor: torch.Tensor | None = None

    def cache_need(self) -> CacheNeed:
        return PagedKV(self.num_kv_heads, self.head_dim, self.window)

    def is_capturable(self) -> bool:
        return self.capturable and self.position.is_capturable()

    def step_fields(self) -> tuple:
        return self.position.step_fields()

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        """The fused projection, the attention output and the output projection (32-bit: it is
        added to the residual stream) of a step."""
        return tokens * ((self.q_size + 2 * self.kv_size + self.q_size) * itemsize + self.hidden_size * 4)

    def tensor_specs(self) -> dict[str, TensorSpec]:
        specs = {
            self.name("q_proj.weight"): TensorSpec((self.q_size, self.hidden_size)),
            self.name("k_proj.weight"): TensorSpec((self.kv_size, self.hidden_size)),
            self.name("v_proj.weight"): TensorSpec((self.kv_size, self.hidden_size)),
            self.name("o_proj.weight"): TensorSpec((self.hidden_size, self.q_size)),
        }
        if self.qkv_bias:
            specs[self.name("q_proj.bias")] = TensorSpec((self.q_size,))
            specs[self.name("k_proj.bias")] = TensorSpec((self.kv_size,))
            specs[self.name("v_proj.bias")] = TensorSpec((self.kv_size,))
        if self.out_bias:
            specs[self.name("o_proj.bias")] = TensorSpec((self.hidden_size,))
        specs.update(self.position.tensor_specs())
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.qkv_weight = torch.cat(
            [tensors[self.name(f"{p}_proj.weight")] for p in ("q", "k", "v")], dim=0
        ).contiguous()
        if self.qkv_bias:
            self.qkv_bias_tensor = torch.cat(
                [tensors[self.name(f"{p}_proj.bias")] for p in ("q", "k", "v")], dim=0
            ).contiguous()
        self.o_weight = tensors[self.name("o_proj.weight")].contiguous()
        if self.out_bias:
            self.o_bias_tensor = tensors[self.name("o_proj.bias")].contiguous()
        self.position.load(tensors)

    def forward(self, x: torch.Tensor, ctx, cache: PagedKVView) -> torch.Tensor:
        ops = self.runtime.ops
        qkv = ops.linear(x, self.qkv_weight, self.qkv_bias_tensor)
        q, q_stride = self.position.encode_and_store(
            qkv, self.num_heads, self.num_kv_heads, self.head_dim, ctx, cache
        )
        attended = self.attend(q, q_stride, ctx, cache)
        return ops.linear(attended, self.o_weight, self.o_bias_tensor, for_residual=True)

    def attend(self, qkv: torch.Tensor, q_stride: int, ctx, cache: PagedKVView) -> torch.Tensor:
        """``[T, Hq D]`` attention output for the step's encoded queries: the first ``Hq D``
        elements of every ``q_stride``-long row of ``qkv``.

        bfloat16 runs use the matrix-core kernels where the geometry allows: one launch for the
        multi-token requests at the front of the batch, one for the single-token requests
        behind them; every 32-bit run, any other geometry and any position encoding that biases
        the scores goes through the generic kernel."""
        ops = self.runtime.ops
        table = ctx.block_tables[cache.group]
        slopes = self.position.score_slopes(self.num_heads)
        fast = slopes is None and ops.mfma_attention_supported(qkv.dtype, self.head_dim, cache.block_size)
        if fast:
            out = ops.rows_buffer(ctx.num_tokens, self.q_size, qkv.dtype, qkv.device)
            if ctx.num_prefill_seqs > 0:
                # The launch's list of row blocks is the same for every layer with this geometry.
                rows = ops.prefill_block_rows(self.head_dim, self.num_heads, self.num_kv_heads)
                geometry = dict(heads=self.num_heads, kv_heads=self.num_kv_heads, head_dim=self.head_dim,
                                block_size=cache.block_size, window=self.window)
                blocks = ctx.derive(("attention_prefill_blocks", rows, *geometry.values()), lambda step: ops.prefill_blocks(
                    step.query_lens[:step.num_prefill_seqs], step.context_lens_host[:step.num_prefill_seqs], rows, **geometry))
                ops.attention_prefill(
                    out, qkv, q_stride, cache.k, cache.v, table, ctx.query_start_loc, ctx.context_lens,
                    blocks, self.num_heads, self.scale, self.window, ctx.max_prefill_context_len, rows,
                )
            if ctx.num_decode_seqs > 0:
                ops.attention_decode(
                    out, qkv, q_stride, cache.k, cache.v, table, ctx.query_start_loc, ctx.context_lens,
                    ctx.num_prefill_seqs, ctx.num_decode_seqs, self.num_heads, self.scale, self.window,
                    min(ctx.max_decode_context_len, table.shape[1] * cache.block_size),
                    ctx.max_decode_context_dev,
                )
            return out
        return ops.paged_attention_generic(
            qkv, q_stride, cache.k, cache.v, table, ctx.token_seq, ctx.positions,
            self.num_heads, self.scale, self.window, slopes,
        )
