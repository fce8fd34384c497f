"""Typed view of a Qwen2 ``config.json``.

Every size and constant the model uses comes from here; nothing in the parts or kernels
carries a number of its own.  Field names, defaults and rejections follow the reference's
``ModelConfig`` (src/turboserve/engine/model/model_config.py:152-314) with one difference:
sliding-window attention, which the reference rejects (:270-274), is described by three more
fields and is supported.
"""

from __future__ import annotations

import json
from collections.abc import Mapping
from dataclasses import asdict, dataclass
from pathlib import Path
from typing import Any

import torch


class UnsupportedModelError(ValueError):
    """``config.json`` describes something this engine does not compute.

    Counterpart of the reference's error of the same name (model_config.py:70-76): refuse at
    load time instead of producing slightly wrong logits.
    """


#: Storage dtypes a checkpoint may declare (model_config.py:58-67).  Only bfloat16 and
#: float32 can be *run*; the others are recognised so the error can say so.
CHECKPOINT_DTYPES: dict[str, torch.dtype] = {
    "float16": torch.float16,
    "fp16": torch.float16,
    "half": torch.float16,
    "bfloat16": torch.bfloat16,
    "bf16": torch.bfloat16,
    "float32": torch.float32,
    "fp32": torch.float32,
    "float": torch.float32,
}

ROPE_TYPES = ("default", "linear")


def require_int(data: Mapping[str, Any], key: str, *, default: int | None = None) -> int:
    """A positive int field; absent, non-int and non-positive each get their own message
    (model_config.py:79-87)."""
    value = data.get(key, default)
    if value is None:
        raise UnsupportedModelError(f"config.json is missing the required field {key!r}")
    if isinstance(value, bool) or not isinstance(value, int):
        raise UnsupportedModelError(f"config.json field {key!r} must be an int, got {value!r}")
    if value < 1:
        raise UnsupportedModelError(f"config.json field {key!r} must be positive, got {value}")
    return value


def rope_settings(data: Mapping[str, Any]) -> tuple[float, float]:
    """``(theta, position divisor)`` from the flat (``rope_theta``/``rope_scaling``) or the
    nested (``rope_parameters``) spelling (model_config.py:90-123)."""
    block = data.get("rope_parameters")
    if not isinstance(block, Mapping):
        merged: dict[str, Any] = {}
        if "rope_theta" in data:
            merged["rope_theta"] = data["rope_theta"]
        if isinstance(data.get("rope_scaling"), Mapping):
            merged.update(data["rope_scaling"])
        block = merged
    theta = float(block.get("rope_theta", 10000.0))
    if theta <= 0:
        raise UnsupportedModelError(f"rope_theta must be positive, got {theta}")
    kind = str(block.get("rope_type") or block.get("type") or "default")
    if kind not in ROPE_TYPES:
        raise UnsupportedModelError(
            f"rope_type {kind!r} is not implemented; supported: {list(ROPE_TYPES)}"
        )
    factor = float(block.get("factor", 1.0)) if kind == "linear" else 1.0
    if factor <= 0:
        raise UnsupportedModelError(f"rope scaling factor must be positive, got {factor}")
    return theta, factor


def checkpoint_dtype(data: Mapping[str, Any]) -> torch.dtype | None:
    """``dtype`` (newer) or ``torch_dtype`` (older) of the checkpoint (model_config.py:126-137)."""
    raw = data.get("dtype", data.get("torch_dtype"))
    if raw is None:
        return None
    if isinstance(raw, torch.dtype):
        return raw
    name = str(raw).removeprefix("torch.")
    if name not in CHECKPOINT_DTYPES:
        raise UnsupportedModelError(f"unknown checkpoint dtype {raw!r}")
    return CHECKPOINT_DTYPES[name]


def eos_ids(data: Mapping[str, Any]) -> tuple[int, ...]:
    """``eos_token_id`` as a tuple, whether the file holds one id or a list (model_config.py:140-149)."""
    raw = data.get("eos_token_id")
    if raw is None:
        return ()
    if isinstance(raw, bool):
        raise UnsupportedModelError(f"unsupported eos_token_id {raw!r}")
    if isinstance(raw, int):
        return (raw,)
    if isinstance(raw, (list, tuple)):
        return tuple(int(t) for t in raw)
    raise UnsupportedModelError(f"unsupported eos_token_id {raw!r}")


@dataclass(frozen=True)
class Qwen2Config:
    """Architecture numbers of one ``Qwen2ForCausalLM`` checkpoint (frozen: the model, the
    cache sizing and the runner all share it)."""

    architecture: str
    model_type: str
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    hidden_act: str
    rms_norm_eps: float
    rope_theta: float
    rope_scaling_factor: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    qkv_bias: bool
    o_proj_bias: bool
    mlp_bias: bool
    use_sliding_window: bool = False
    sliding_window: int | None = None
    max_window_layers: int = 0
    torch_dtype: torch.dtype | None = None
    eos_token_ids: tuple[int, ...] = ()
    bos_token_id: int | None = None
    pad_token_id: int | None = None
    name_or_path: str = ""

    ARCHITECTURE = "Qwen2ForCausalLM"

    def __post_init__(self) -> None:
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise UnsupportedModelError(
                f"num_attention_heads={self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads={self.num_key_value_heads}; GQA requires it"
            )
        if self.hidden_act not in ("silu", "swish"):
            raise UnsupportedModelError(
                f"hidden_act {self.hidden_act!r} is not implemented; supported: ['silu', 'swish']"
            )
        if self.head_dim % 2 != 0:
            raise UnsupportedModelError(f"head_dim must be even for rotary embeddings, got {self.head_dim}")
        if self.mlp_bias:
            raise UnsupportedModelError("mlp_bias=true is not implemented for Qwen2")
        if self.use_sliding_window and (self.sliding_window is None or self.sliding_window < 1):
            raise UnsupportedModelError(
                f"use_sliding_window needs a positive sliding_window, got {self.sliding_window!r}"
            )

    # -- derived ----------------------------------------------------------------------------

    @property
    def num_kv_groups(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    @property
    def q_proj_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_proj_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def attn_scale(self) -> float:
        return float(self.head_dim) ** -0.5

    @property
    def is_gqa(self) -> bool:
        return self.num_kv_groups > 1

    def layer_window(self, layer: int) -> int | None:
        """Keys a query of ``layer`` sees, itself included, or ``None`` for all of them.

        Rule of this engine: with ``use_sliding_window`` the layers ``>= max_window_layers``
        are windowed and the ones below keep the whole context.
        """
        if self.use_sliding_window and layer >= self.max_window_layers:
            return self.sliding_window
        return None

    def kv_bytes_per_token(self, dtype: torch.dtype) -> int:
        """``2 * layers * kv_heads * head_dim * itemsize`` (model_config.py:234-242)."""
        return 2 * self.num_hidden_layers * self.num_key_value_heads * self.head_dim * dtype.itemsize

    def to_dict(self) -> dict[str, Any]:
        data = asdict(self)
        dtype = data.pop("torch_dtype")
        data["torch_dtype"] = None if dtype is None else str(dtype).removeprefix("torch.")
        data["eos_token_ids"] = list(self.eos_token_ids)
        return data

    def to_hf_dict(self) -> dict[str, Any]:
        """A ``config.json`` mapping that parses back to this configuration."""
        data: dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": self.model_type,
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "hidden_act": self.hidden_act,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "use_sliding_window": self.use_sliding_window,
            "sliding_window": self.sliding_window,
            "max_window_layers": self.max_window_layers,
        }
        if self.rope_scaling_factor != 1.0:
            data["rope_scaling"] = {"rope_type": "linear", "factor": self.rope_scaling_factor}
        if self.torch_dtype is not None:
            data["torch_dtype"] = str(self.torch_dtype).removeprefix("torch.")
        if self.eos_token_ids:
            data["eos_token_id"] = list(self.eos_token_ids)
        if self.bos_token_id is not None:
            data["bos_token_id"] = self.bos_token_id
        if self.pad_token_id is not None:
            data["pad_token_id"] = self.pad_token_id
        return data

    # -- construction -----------------------------------------------------------------------

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], *, name_or_path: str = "") -> "Qwen2Config":
        """Parse a ``config.json`` mapping (model_config.py:254-314)."""
        architectures = data.get("architectures") or []
        architecture = str(architectures[0]) if architectures else ""
        if architecture != cls.ARCHITECTURE:
            raise UnsupportedModelError(
                f"architecture {architecture or '<missing>'!r} is not a {cls.ARCHITECTURE}"
            )
        hidden_size = require_int(data, "hidden_size")
        heads = require_int(data, "num_attention_heads")
        kv_heads = require_int(data, "num_key_value_heads", default=heads)
        raw_head_dim = data.get("head_dim")
        head_dim = int(raw_head_dim) if raw_head_dim else hidden_size // heads
        if head_dim < 1:
            raise UnsupportedModelError(f"head_dim resolved to {head_dim}")
        theta, factor = rope_settings(data)
        use_window = bool(data.get("use_sliding_window", False)) and bool(data.get("sliding_window"))
        window = data.get("sliding_window")
        if window is not None and (isinstance(window, bool) or not isinstance(window, int)):
            raise UnsupportedModelError(f"config.json field 'sliding_window' must be an int, got {window!r}")
        max_window_layers = data.get("max_window_layers", 0) or 0
        if isinstance(max_window_layers, bool) or not isinstance(max_window_layers, int) or max_window_layers < 0:
            raise UnsupportedModelError(
                f"config.json field 'max_window_layers' must be a non-negative int, got {max_window_layers!r}"
            )
        return cls(
            architecture=architecture,
            model_type=str(data.get("model_type") or "qwen2"),
            hidden_size=hidden_size,
            num_hidden_layers=require_int(data, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=require_int(data, "intermediate_size"),
            vocab_size=require_int(data, "vocab_size"),
            hidden_act=str(data.get("hidden_act", "silu")),
            rms_norm_eps=float(data.get("rms_norm_eps", 1e-6)),
            rope_theta=theta,
            rope_scaling_factor=factor,
            max_position_embeddings=require_int(data, "max_position_embeddings", default=2048),
            tie_word_embeddings=bool(data.get("tie_word_embeddings", False)),
            # Qwen2's q/k/v bias is part of the architecture; o_proj never has one
            # (model_config.py:285-288).
            qkv_bias=True,
            o_proj_bias=False,
            mlp_bias=bool(data.get("mlp_bias", False)),
            use_sliding_window=use_window,
            sliding_window=int(window) if window else None,
            max_window_layers=int(max_window_layers),
            torch_dtype=checkpoint_dtype(data),
            eos_token_ids=eos_ids(data),
            bos_token_id=data.get("bos_token_id"),
            pad_token_id=data.get("pad_token_id"),
            name_or_path=name_or_path,
        )

    @classmethod
    def from_hf(cls, model_dir: str | Path) -> "Qwen2Config":
        """The configuration of a model folder (model_config.py:316-339); local folders only."""
        return cls.from_dict(read_config_json(model_dir), name_or_path=str(model_dir))


def read_config_json(model_dir: str | Path) -> dict[str, Any]:
    """The parsed ``config.json`` of a model folder (model_config.py:334-339)."""
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise UnsupportedModelError(f"no config.json under {model_dir}")
    data = json.loads(path.read_text(encoding="utf-8"))
    if not isinstance(data, dict):
        raise UnsupportedModelError(f"{path} does not contain a JSON object")
    return data
