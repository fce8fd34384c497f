"""One registry from an architecture's name (``config.json``'s ``architectures[0]``) to its
configuration class and its plan builder.

The reference keeps only a dict of names (src/turboserve/engine/model/model_config.py:41-44)
and serves them with one class; here the name selects both how ``config.json`` is read and how
the model is put together, which is all another architecture has to supply.
"""

from __future__ import annotations

from collections.abc import Callable, Mapping
from dataclasses import dataclass
from typing import Any

from turboserve_amd.config.model_config import UnsupportedModelError


@dataclass(frozen=True)
class Architecture:
    name: str
    parse_config: Callable[..., Any]  # (mapping, name_or_path=...) -> typed config
    build_plan: Callable[[Any], Any]  # typed config -> ModelPlan


ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, parse_config: Callable[..., Any], build_plan: Callable[[Any], Any]) -> None:
    if name in ARCHITECTURES:
        raise ValueError(f"architecture {name!r} is already registered")
    ARCHITECTURES[name] = Architecture(name, parse_config, build_plan)


def architecture_of(data: Mapping[str, Any]) -> Architecture:
    """The registered architecture a ``config.json`` mapping names."""
    _ensure_builtin()
    names = data.get("architectures") or []
    name = str(names[0]) if names else ""
    if name not in ARCHITECTURES:
        raise UnsupportedModelError(
            f"architecture {name or '<missing>'!r} is not implemented; supported: {sorted(ARCHITECTURES)}"
        )
    return ARCHITECTURES[name]


def parse_model_config(data: Mapping[str, Any], *, name_or_path: str = "") -> Any:
    return architecture_of(data).parse_config(data, name_or_path=name_or_path)


def _ensure_builtin() -> None:
    if "Qwen2ForCausalLM" not in ARCHITECTURES:
        from turboserve_amd.config.model_config import Qwen2Config
        from turboserve_amd.models.qwen2 import qwen2_plan

        register_architecture("Qwen2ForCausalLM", Qwen2Config.from_dict, qwen2_plan)
