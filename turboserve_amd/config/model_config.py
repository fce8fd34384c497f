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


# ---------------------------------------------------------------------------------------------
# The schema: which key of config.json fills which field, what kind of value it must be and
# what stands in when the file has none.  ``from_dict`` and ``to_hf_dict`` both walk it.
# ---------------------------------------------------------------------------------------------

REQUIRED = object()  # a key without a default


@dataclass(frozen=True)
class Key:
    """One plain key of ``config.json``.

    ``kind``: ``"count"`` (an int of at least ``least``; a bool or a string is refused),
    ``"flag"``, ``"real"``, ``"text"`` or ``"id"`` (an optional token id, kept as found).
    ``default`` may name another key's field (a ``str`` starting with ``=``): the value read
    for that field stands in."""

    field: str
    kind: str
    default: Any = REQUIRED
    least: int = 1

    def read(self, data: Mapping[str, Any], so_far: Mapping[str, Any]) -> Any:
        raw = data.get(self.field)
        if raw is None or (self.kind == "count" and self.least == 0 and not raw):
            if self.default is REQUIRED:
                raise UnsupportedModelError(f"config.json is missing the required field {self.field!r}")
            if isinstance(self.default, str) and self.default.startswith("="):
                return so_far[self.default[1:]]
            return self.default
        if self.kind == "count":
            if isinstance(raw, bool) or not isinstance(raw, int):
                raise UnsupportedModelError(f"config.json field {self.field!r} must be an int, got {raw!r}")
            if raw < self.least:
                bound = "positive" if self.least == 1 else "a non-negative int"
                raise UnsupportedModelError(f"config.json field {self.field!r} must be {bound}, got {raw}")
            return raw
        return {"flag": bool, "real": float, "text": str, "id": lambda v: v}[self.kind](raw)


#: Read in this order (a default may point back at an earlier field).  Defaults and the
#: messages of ``Key.read`` are the reference's (model_config.py:79-87, 278, 300-313).
PLAIN_KEYS: tuple[Key, ...] = (
    Key("model_type", "text", "qwen2"),
    Key("hidden_size", "count"),
    Key("num_hidden_layers", "count"),
    Key("num_attention_heads", "count"),
    Key("num_key_value_heads", "count", "=num_attention_heads"),
    Key("intermediate_size", "count"),
    Key("vocab_size", "count"),
    Key("hidden_act", "text", "silu"),
    Key("rms_norm_eps", "real", 1e-6),
    Key("max_position_embeddings", "count", 2048),
    Key("tie_word_embeddings", "flag", False),
    Key("mlp_bias", "flag", False),
    Key("max_window_layers", "count", 0, least=0),
    Key("bos_token_id", "id", None),
    Key("pad_token_id", "id", None),
)

#: Names a checkpoint may give its storage type (model_config.py:58-67).  Only bfloat16 and
#: float32 can be *run*; the others are recognised so the error can say so.
CHECKPOINT_DTYPES: dict[str, torch.dtype] = {
    **dict.fromkeys(("float16", "fp16", "half"), torch.float16),
    **dict.fromkeys(("bfloat16", "bf16"), torch.bfloat16),
    **dict.fromkeys(("float32", "fp32", "float"), torch.float32),
}

ROPE_TYPES = ("default", "linear")


# Keys that need more than one lookup each get a function: config.json -> {field: value}.


def _head_dim(data: Mapping[str, Any], so_far: Mapping[str, Any]) -> dict[str, Any]:
    """``head_dim`` if the file has one, else ``hidden_size // heads`` (model_config.py:279-282)."""
    given = data.get("head_dim")
    head_dim = int(given) if given else so_far["hidden_size"] // so_far["num_attention_heads"]
    if head_dim < 1:
        raise UnsupportedModelError(f"head_dim resolved to {head_dim}")
    return {"head_dim": head_dim}


def _rope(data: Mapping[str, Any], so_far: Mapping[str, Any]) -> dict[str, Any]:
    """Base and position divisor, from the nested spelling (``rope_parameters``) or the flat
    one (``rope_theta`` beside ``rope_scaling``) (model_config.py:90-123)."""
    nested = data.get("rope_parameters")
    if isinstance(nested, Mapping):
        settings = dict(nested)
    else:
        scaling = data.get("rope_scaling")
        settings = dict(scaling) if isinstance(scaling, Mapping) else {}
        if "rope_theta" in data:
            settings["rope_theta"] = data["rope_theta"]
    theta = float(settings.get("rope_theta", 10000.0))
    kind = str(settings.get("rope_type") or settings.get("type") or "default")
    factor = float(settings.get("factor", 1.0)) if kind == "linear" else 1.0
    for ok, message in (
        (theta > 0, f"rope_theta must be positive, got {theta}"),
        (kind in ROPE_TYPES, f"rope_type {kind!r} is not implemented; supported: {list(ROPE_TYPES)}"),
        (factor > 0, f"rope scaling factor must be positive, got {factor}"),
    ):
        if not ok:
            raise UnsupportedModelError(message)
    return {"rope_theta": theta, "rope_scaling_factor": factor}


def _window(data: Mapping[str, Any], so_far: Mapping[str, Any]) -> dict[str, Any]:
    """Sliding-window attention is on when the file says so *and* names a window."""
    window = data.get("sliding_window")
    if window is not None and (isinstance(window, bool) or not isinstance(window, int)):
        raise UnsupportedModelError(f"config.json field 'sliding_window' must be an int, got {window!r}")
    return {"use_sliding_window": bool(data.get("use_sliding_window", False)) and bool(window),
            "sliding_window": window or None}


def _storage_dtype(data: Mapping[str, Any], so_far: Mapping[str, Any]) -> dict[str, Any]:
    """``dtype`` (newer files) or ``torch_dtype`` (older) (model_config.py:126-137)."""
    named = data.get("dtype", data.get("torch_dtype"))
    if named is None or isinstance(named, torch.dtype):
        return {"torch_dtype": named}
    found = CHECKPOINT_DTYPES.get(str(named).removeprefix("torch."))
    if found is None:
        raise UnsupportedModelError(f"unknown checkpoint dtype {named!r}")
    return {"torch_dtype": found}


def _end_tokens(data: Mapping[str, Any], so_far: Mapping[str, Any]) -> dict[str, Any]:
    """``eos_token_id`` holds one id or a list of them (model_config.py:140-149)."""
    named = data.get("eos_token_id")
    if named is None:
        return {"eos_token_ids": ()}
    if isinstance(named, int) and not isinstance(named, bool):
        return {"eos_token_ids": (named,)}
    if isinstance(named, (list, tuple)):
        return {"eos_token_ids": tuple(int(t) for t in named)}
    raise UnsupportedModelError(f"unsupported eos_token_id {named!r}")


COMPOSITE_KEYS = (_head_dim, _rope, _window, _storage_dtype, _end_tokens)


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
        data: dict[str, Any] = {"architectures": [self.architecture]}
        for key in PLAIN_KEYS:
            value = getattr(self, key.field)
            if value is not None and key.field != "mlp_bias":
                data[key.field] = value
        data.update(head_dim=self.head_dim, rope_theta=self.rope_theta, use_sliding_window=self.use_sliding_window,
                    sliding_window=self.sliding_window)
        if self.rope_scaling_factor != 1.0:
            data["rope_scaling"] = {"rope_type": "linear", "factor": self.rope_scaling_factor}
        if self.torch_dtype is not None:
            data["torch_dtype"] = str(self.torch_dtype).removeprefix("torch.")
        if self.eos_token_ids:
            data["eos_token_id"] = list(self.eos_token_ids)
        return data

    # -- construction -----------------------------------------------------------------------

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], *, name_or_path: str = "") -> "Qwen2Config":
        """Parse a ``config.json`` mapping by the schema above (the reference's counterpart:
        model_config.py:254-314)."""
        named = data.get("architectures") or [""]
        if str(named[0]) != cls.ARCHITECTURE:
            raise UnsupportedModelError(f"architecture {str(named[0]) or '<missing>'!r} is not a {cls.ARCHITECTURE}")
        values: dict[str, Any] = {}
        for key in PLAIN_KEYS:
            values[key.field] = key.read(data, values)
        for composite in COMPOSITE_KEYS:
            values.update(composite(data, values))
        # Qwen2's q/k/v bias is part of the architecture, whatever ``attention_bias`` says; the
        # output projection never has one (model_config.py:285-288).
        return cls(architecture=cls.ARCHITECTURE, qkv_bias=True, o_proj_bias=False, name_or_path=name_or_path, **values)

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
