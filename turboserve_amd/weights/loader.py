"""Weights from safetensors, by tensor name.

What the model expects is the union of its parts' ``tensor_specs``; the loader reads each
named tensor's shape and type from the shards' headers and hands ``model.load`` a supply
that reads a tensor, converts it (floats to the run's dtype, integer tables to int32, a 32-bit
tensor whose spec says so stays 32-bit) and moves it to the device when a part asks for it.
Everything that does not fit — missing tensors, unexpected tensors, wrong shapes — is
collected and raised as ONE error, before any tensor's bytes are read.

Discovery and naming rules follow src/turboserve/engine/model/weights.py:105-276; the
difference is that a shape mismatch does not stop at the first one (:253-257) but is listed
with the rest.
"""

from __future__ import annotations

import json
import math
import weakref
from collections.abc import Callable, Iterable, Iterator, Mapping
from dataclasses import dataclass, field
from pathlib import Path

import torch

from turboserve_amd.parts.base import TensorSpec

SAFETENSORS_FILE = "model.safetensors"
SAFETENSORS_INDEX = "model.safetensors.index.json"

#: Tensors some exports carry that are derived, not learned (weights.py:49-54).
SKIPPED_SUFFIXES = (".rotary_emb.inv_freq", ".attn.bias", ".attn.masked_bias", ".masked_bias")

#: Prefixes some exporters put before the decoder's names (weights.py:57-61, 193-195).
PREFIX_REWRITES = (
    ("transformer.", "model."),
    ("language_model.model.", "model."),
    ("language_model.lm_head.", "lm_head."),
    ("model.decoder.", "model."),
)


class WeightLoadError(RuntimeError):
    """The checkpoint cannot be read or does not match the model."""


@dataclass
class LoadReport:
    """What a load did (weights.py:70-102)."""

    loaded: list[str] = field(default_factory=list)
    missing: list[str] = field(default_factory=list)
    unexpected: list[str] = field(default_factory=list)
    wrong_shape: list[str] = field(default_factory=list)
    wrong_type: list[str] = field(default_factory=list)
    ignored: list[str] = field(default_factory=list)
    num_bytes: int = 0

    @property
    def ok(self) -> bool:
        return not (self.missing or self.unexpected or self.wrong_shape or self.wrong_type)

    def summary(self) -> str:
        return (
            f"{len(self.loaded)} tensors ({self.num_bytes / 2**20:.1f} MiB) loaded, "
            f"{len(self.missing)} missing, {len(self.unexpected)} unexpected, "
            f"{len(self.wrong_shape)} with a wrong shape, {len(self.ignored)} ignored"
        )

    def error_message(self) -> str:
        lines = ["checkpoint does not match the model:"]
        for title, items in (
            ("missing", self.missing),
            ("unexpected", self.unexpected),
            ("wrong shape", self.wrong_shape),
            ("wrong type", self.wrong_type),
        ):
            if items:
                lines.append(f"  {title} ({len(items)}): " + "; ".join(items))
        return "\n".join(lines)


def resolve_model_dir(path: str | Path) -> Path:
    """A local model folder (weights.py:105-134; there is no download here)."""
    candidate = Path(path).expanduser()
    if candidate.is_dir():
        return candidate
    if candidate.exists():
        raise WeightLoadError(f"{candidate} is a file; expected a checkpoint directory")
    raise WeightLoadError(f"model folder {candidate} does not exist (models are read from local folders only)")


def safetensors_files(model_dir: Path) -> list[Path]:
    """The checkpoint's shards: those the index names (sorted, all must exist), else
    ``model.safetensors``, else every ``*.safetensors`` (weights.py:137-178)."""
    if not model_dir.is_dir():
        raise WeightLoadError(f"{model_dir} is not a directory")
    index_path = model_dir / SAFETENSORS_INDEX
    if index_path.is_file():
        weight_map = json.loads(index_path.read_text(encoding="utf-8")).get("weight_map")
        if not isinstance(weight_map, dict) or not weight_map:
            raise WeightLoadError(f"{index_path} has no usable weight_map")
        files = [model_dir / name for name in sorted({str(v) for v in weight_map.values()})]
        absent = [str(f) for f in files if not f.is_file()]
        if absent:
            raise WeightLoadError(f"shards listed in {index_path} are absent: {absent}")
        return files
    single = model_dir / SAFETENSORS_FILE
    if single.is_file():
        return [single]
    shards = sorted(model_dir.glob("*.safetensors"))
    if shards:
        return shards
    pickles = sorted(model_dir.glob("*.bin")) + sorted(model_dir.glob("*.pth")) + sorted(model_dir.glob("*.pt"))
    if pickles:
        raise WeightLoadError(
            f"{model_dir} holds only pickle checkpoints ({pickles[0].name}); only safetensors is read"
        )
    raise WeightLoadError(f"no safetensors checkpoint under {model_dir}")


def map_weight_name(name: str) -> str | None:
    """A checkpoint name as the model knows it, or ``None`` for a derived tensor that is
    skipped (weights.py:181-196)."""
    if name.endswith(SKIPPED_SUFFIXES):
        return None
    for old, new in PREFIX_REWRITES:
        if name.startswith(old):
            return new + name[len(old):]
    return name


@dataclass(frozen=True)
class StoredTensor:
    """A checkpoint tensor that has not been read yet: what the checks need, and how to read it."""

    shape: tuple[int, ...]
    dtype: torch.dtype
    read: Callable[[], torch.Tensor]

    @staticmethod
    def of(tensor: torch.Tensor) -> "StoredTensor":
        return StoredTensor(tuple(tensor.shape), tensor.dtype, lambda: tensor)


#: safetensors' names of the stored types this loader may meet.
STORED_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}  # fmt: skip


def iter_checkpoint_entries(files: list[Path]) -> Iterator[tuple[str, StoredTensor]]:
    """``(name, StoredTensor)`` for every tensor of the shards, from the shards' headers alone:
    no tensor's bytes are read before someone asks for it (``StoredTensor.read`` opens the shard
    for that one tensor, so a shard is never resident; discovery order as in
    weights.py:199-216)."""
    from safetensors import safe_open

    def reader(path: Path, name: str) -> Callable[[], torch.Tensor]:
        def read() -> torch.Tensor:
            try:
                with safe_open(str(path), framework="pt", device="cpu") as handle:
                    return handle.get_tensor(name)
            except Exception as exc:
                raise WeightLoadError(f"cannot read {name} from {path}: {exc}") from exc

        return read

    for path in files:
        try:
            with safe_open(str(path), framework="pt", device="cpu") as handle:
                for name in handle.keys():
                    piece = handle.get_slice(name)
                    stored = STORED_DTYPES.get(str(piece.get_dtype()))
                    if stored is None:
                        raise WeightLoadError(f"{path}: {name} is stored as {piece.get_dtype()}, which is not read")
                    yield name, StoredTensor(tuple(piece.get_shape()), stored, reader(path, name))
        except WeightLoadError:
            raise
        except Exception as exc:
            raise WeightLoadError(f"cannot read {path}: {exc}") from exc


def iter_checkpoint_tensors(files: list[Path]) -> Iterator[tuple[str, torch.Tensor]]:
    """``(name, CPU tensor)`` one at a time."""
    for name, entry in iter_checkpoint_entries(files):
        yield name, entry.read()


def kept_dtype(stored: torch.dtype, spec: TensorSpec, dtype: torch.dtype) -> torch.dtype | None:
    """The type the run keeps a tensor of ``spec`` in that the checkpoint stores as ``stored``
    (floats in the run's dtype, integer tables as int32, a 32-bit tensor whose spec says so
    stays 32-bit), or ``None`` if the stored type does not fit the spec."""
    if spec.kind == "int":
        return None if (stored.is_floating_point or stored == torch.bool) else torch.int32
    if not stored.is_floating_point:
        return None
    if spec.kind == "float_keep32" and stored == torch.float32:
        return torch.float32
    return dtype


def convert_tensor(tensor: torch.Tensor, spec: TensorSpec, dtype: torch.dtype) -> torch.Tensor | None:
    """The tensor as the run keeps it, or ``None`` if its stored type does not fit the spec."""
    kept = kept_dtype(tensor.dtype, spec, dtype)
    return None if kept is None else tensor.to(kept)


class TensorSupply(Mapping):
    """``name -> tensor`` as ``Part.load`` wants it, each tensor made (read, converted, moved to
    the device) when it is asked for and handed over, not kept.  A part that fuses what it is
    given into a layout of its own drops the originals as it goes, so a model never holds its
    weights twice; a checkpoint's bytes are never all in host memory either.  A tensor that is
    still alive when it is asked for again (the embedding table that a tied head shares) is
    handed out as the same object."""

    def __init__(self, names: Iterable[str], make: Callable[[str], torch.Tensor]) -> None:
        self._names = dict.fromkeys(names)
        self._make = make
        self._alive: weakref.WeakValueDictionary[str, torch.Tensor] = weakref.WeakValueDictionary()

    def __getitem__(self, name: str) -> torch.Tensor:
        tensor = self._alive.get(name)
        if tensor is None:
            if name not in self._names:
                raise KeyError(name)
            tensor = self._make(name)
            self._alive[name] = tensor
        return tensor

    def __iter__(self) -> Iterator[str]:
        return iter(self._names)

    def __len__(self) -> int:
        return len(self._names)


def load_tensors(
    specs: Mapping[str, TensorSpec],
    source: Iterator[tuple[str, torch.Tensor | StoredTensor]],
    *,
    dtype: torch.dtype,
    device: torch.device | str,
    ignorable: set[str] | frozenset[str] = frozenset(),
) -> tuple[TensorSupply, LoadReport]:
    """Match named tensors against ``specs``; returns what fitted (a ``TensorSupply``: nothing
    is read or moved before it is asked for) and the full report."""
    report = LoadReport()
    found: dict[str, tuple[StoredTensor, torch.dtype]] = {}
    for raw_name, given in source:
        entry = given if isinstance(given, StoredTensor) else StoredTensor.of(given)
        name = map_weight_name(raw_name)
        if name is None:
            report.ignored.append(raw_name)
            continue
        spec = specs.get(name)
        if spec is None:
            (report.ignored if name in ignorable else report.unexpected).append(raw_name)
            continue
        if name in found:
            report.unexpected.append(f"{raw_name} (given twice)")
            continue
        if tuple(entry.shape) != tuple(spec.shape):
            report.wrong_shape.append(f"{name}: model has {tuple(spec.shape)}, checkpoint has {tuple(entry.shape)}")
            continue
        kept = kept_dtype(entry.dtype, spec, dtype)
        if kept is None:
            report.wrong_type.append(f"{name}: expected {spec.kind}, checkpoint has {entry.dtype}")
            continue
        found[name] = (entry, kept)
        report.loaded.append(name)
        report.num_bytes += math.prod(entry.shape) * kept.itemsize
    bad = {entry.split(":", 1)[0] for entry in (*report.wrong_shape, *report.wrong_type)}
    report.missing = [name for name in specs if name not in found and name not in bad]

    def make(name: str) -> torch.Tensor:
        entry, kept = found[name]
        return entry.read().to(kept).to(device)

    return TensorSupply(found, make), report


def load_model_weights(model, model_dir: str | Path, *, strict: bool = True) -> LoadReport:
    """Fill ``model`` (anything with ``tensor_specs``, ``ignorable_names``, ``load`` and a
    ``runtime``) from the safetensors files of ``model_dir``."""
    folder = resolve_model_dir(model_dir)
    files = safetensors_files(folder)
    tensors, report = load_tensors(
        model.tensor_specs(),
        iter_checkpoint_entries(files),
        dtype=model.runtime.dtype,
        device=model.runtime.device,
        ignorable=model.ignorable_names(),
    )
    if not report.ok:
        if strict or report.missing or report.wrong_shape or report.wrong_type:
            raise WeightLoadError(report.error_message())
    model.load(tensors)
    return report
