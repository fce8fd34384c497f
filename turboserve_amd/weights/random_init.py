"""Random weights from a configuration and a seed.

``write_random_model`` writes a model folder (``config.json`` + ``model.safetensors``) that the
ordinary loader then reads, so tests exercise the real path; ``random_tensors_on_device`` fills
a model in place for measurements where a folder of tens of gigabytes would be waste.

Draw rule (this engine's; the reference zeroes biases, src/turboserve/engine/model/model.py:248-268):
one CPU ``torch.Generator`` seeded with ``seed``; the model's tensors in model order
(embedding, each layer's tensors in the order its parts declare them, final norm, head); a
tensor whose spec says ``"ones"``/``"zeros"`` is filled so and draws nothing; every other
tensor, biases included, is drawn N(0, std) in 32-bit and then rounded to the folder's dtype.
A tied head is the embedding and draws nothing.
"""

from __future__ import annotations

import json
from collections.abc import Iterator, Mapping
from pathlib import Path
from typing import Any

import torch

from turboserve_amd.config.registry import architecture_of
from turboserve_amd.parts.base import Runtime, TensorSpec


def describe_model(config_data: Mapping[str, Any]):
    """``(typed config, model without weights)`` for a ``config.json`` mapping.  No GPU is
    needed: parts are only asked what tensors they expect."""
    import turboserve_amd.parts  # noqa: F401  (registers the built-in part kinds)
    from turboserve_amd.models.decoder import DecoderModel

    arch = architecture_of(config_data)
    config = arch.parse_config(config_data)
    runtime = Runtime(device=torch.device("cpu"), dtype=torch.float32, ops=None)
    return config, DecoderModel(arch.build_plan(config), runtime)


def draw_tensors(
    specs: Mapping[str, TensorSpec], seed: int, *, std: float = 0.02, dtype: torch.dtype = torch.float32
) -> Iterator[tuple[str, torch.Tensor]]:
    generator = torch.Generator(device="cpu")
    generator.manual_seed(int(seed))
    for name, spec in specs.items():
        if spec.kind == "int":
            raise ValueError(f"{name}: integer tables have no random initialisation")
        if spec.init == "ones":
            yield name, torch.ones(spec.shape, dtype=dtype)
        elif spec.init == "zeros":
            yield name, torch.zeros(spec.shape, dtype=dtype)
        else:
            values = torch.empty(spec.shape, dtype=torch.float32)
            values.normal_(0.0, std, generator=generator)
            yield name, values.to(dtype)


def write_random_model(
    config_data: Mapping[str, Any],
    folder: str | Path,
    *,
    seed: int,
    dtype: torch.dtype = torch.float32,
    std: float = 0.02,
) -> Path:
    """Write ``config.json`` and ``model.safetensors`` for ``config_data`` under ``folder``."""
    from safetensors.torch import save_file

    out = Path(folder)
    out.mkdir(parents=True, exist_ok=True)
    _, model = describe_model(config_data)
    tensors = dict(draw_tensors(model.tensor_specs(), seed, std=std, dtype=dtype))
    data = dict(config_data)
    data["torch_dtype"] = str(dtype).removeprefix("torch.")
    (out / "config.json").write_text(json.dumps(data, indent=2), encoding="utf-8")
    save_file(tensors, str(out / "model.safetensors"), metadata={"format": "pt"})
    return out


def random_tensors_on_device(model, seed: int, *, std: float = 0.02) -> None:
    """Fill ``model`` with N(0, std) weights drawn on its device (norm gains 1).  The values
    differ from the folder mode's; the distributions are the same.  A tensor is drawn when a part
    asks for it, from a generator seeded with ``seed`` and the tensor's place among the model's
    tensors: the values do not depend on the order of asking, and the model never holds a
    second copy of what its parts have fused."""
    from turboserve_amd.weights.loader import TensorSupply

    runtime = model.runtime
    specs = model.tensor_specs()
    places = {name: place for place, name in enumerate(specs)}

    def make(name: str) -> torch.Tensor:
        spec = specs[name]
        if spec.init == "ones":
            return torch.ones(spec.shape, dtype=runtime.dtype, device=runtime.device)
        if spec.init == "zeros":
            return torch.zeros(spec.shape, dtype=runtime.dtype, device=runtime.device)
        generator = torch.Generator(device=runtime.device)
        generator.manual_seed(int(seed) * 1_000_003 + places[name])
        values = torch.empty(spec.shape, dtype=runtime.dtype, device=runtime.device)
        values.normal_(0.0, std, generator=generator)
        return values

    model.load(TensorSupply(specs, make))
