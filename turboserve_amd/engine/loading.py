"""From a model folder to a model on the GPU, and from a model to its cache."""

from __future__ import annotations

from pathlib import Path
from typing import Any

import torch

import turboserve_amd.parts  # noqa: F401  (registers the built-in part kinds)
from turboserve_amd.cache.layout import CacheLayout
from turboserve_amd.cache.storage import CacheStorage
from turboserve_amd.config.model_config import read_config_json
from turboserve_amd.config.registry import architecture_of
from turboserve_amd.kernels.ops import Ops
from turboserve_amd.models.decoder import DecoderModel
from turboserve_amd.parts.base import Runtime
from turboserve_amd.weights.loader import LoadReport, load_model_weights, resolve_model_dir

RUN_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def resolve_run_dtype(name: str | torch.dtype) -> torch.dtype:
    """``bfloat16`` (the serving precision) or ``float32`` (everything in true 32-bit).  The
    reference also offers float16 and an ``auto`` that never picks bfloat16
    (src/turboserve/engine/core/types.py:80-94, 560-574); on this hardware bfloat16 is the
    default and float16 is not built."""
    if isinstance(name, torch.dtype):
        if name in RUN_DTYPES.values():
            return name
        raise ValueError(f"unsupported dtype {name}; expected one of {sorted(RUN_DTYPES)}")
    if name in ("auto", "bf16"):
        return torch.bfloat16
    if name in ("fp32", "float"):
        return torch.float32
    try:
        return RUN_DTYPES[name]
    except KeyError:
        raise ValueError(f"unsupported dtype {name!r}; expected one of {sorted(RUN_DTYPES)}") from None


def make_runtime(dtype: torch.dtype, device: str | torch.device = "cuda:0") -> Runtime:
    device = torch.device(device)
    return Runtime(device=device, dtype=dtype, ops=Ops(device))


def build_model(config_data: dict[str, Any], runtime: Runtime, *, name_or_path: str = ""):
    """``(typed config, model without weights)``; the class is chosen by ``architectures[0]``."""
    arch = architecture_of(config_data)
    config = arch.parse_config(config_data, name_or_path=name_or_path)
    return config, DecoderModel(arch.build_plan(config), runtime)


def load_model(model_dir: str | Path, *, dtype: str | torch.dtype = "bfloat16", device: str | torch.device = "cuda:0"):
    """``(typed config, model with weights, load report)`` from a folder with ``config.json``
    and safetensors (src/turboserve/engine/model/model.py:270-306)."""
    folder = resolve_model_dir(model_dir)
    data = read_config_json(folder)
    runtime = make_runtime(resolve_run_dtype(dtype), device)
    config, model = build_model(data, runtime, name_or_path=str(model_dir))
    report: LoadReport = load_model_weights(model, folder)
    return config, model, report


def build_storage(model: DecoderModel, num_pages: int | list[int], page_size: int, num_state_slots: int) -> CacheStorage:
    layout = CacheLayout.from_model(model)
    counts = [num_pages] * len(layout.groups) if isinstance(num_pages, int) else list(num_pages)
    return CacheStorage(layout, counts, page_size, num_state_slots, model.runtime.dtype, model.runtime.device)
