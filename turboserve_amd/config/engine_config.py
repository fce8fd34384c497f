"""Options of the scheduler and of the engine (src/turboserve/engine/core/types.py:484-593).

Names and defaults are the reference's where it has them.  What it has and this engine does
not is either absent (speculative and LoRA blocks) or, where a caller of the reference is likely
to pass it, accepted in its "off" value only: ``enable_prefix_caching`` (the reference's default
is on; here it must be off) and ``policy`` (first come, first served).
"""

from __future__ import annotations

import os
from collections.abc import Mapping
from dataclasses import dataclass, field
from typing import Any


@dataclass
class SchedulerConfig:
    """Limits of one step (types.py:484-518)."""

    max_num_seqs: int = 64
    max_num_batched_tokens: int = 2048
    block_size: int = 16
    num_blocks: int | None = None
    enable_chunked_prefill: bool = True
    enable_prefix_caching: bool = False  # not built: every prompt is computed in full
    policy: str = "fcfs"  # the only order of admission

    def __post_init__(self) -> None:
        if self.enable_prefix_caching:
            raise ValueError("enable_prefix_caching=True: this engine has no prefix cache; pass False")
        if self.policy != "fcfs":
            raise ValueError(f"policy {self.policy!r} is not built; the only policy is 'fcfs'")
        for name in ("max_num_seqs", "max_num_batched_tokens", "block_size"):
            value = getattr(self, name)
            if isinstance(value, bool) or not isinstance(value, int) or value < 1:
                raise ValueError(f"{name} must be an int >= 1, got {value!r}")
        if self.num_blocks is not None and (not isinstance(self.num_blocks, int) or self.num_blocks < 1):
            raise ValueError(f"num_blocks must be an int >= 1 or None, got {self.num_blocks!r}")
        if self.block_size & (self.block_size - 1):
            raise ValueError(f"block_size must be a power of two, got {self.block_size}")
        if self.max_num_batched_tokens < self.block_size:
            raise ValueError(
                f"max_num_batched_tokens ({self.max_num_batched_tokens}) must be at least one block "
                f"({self.block_size})"
            )


@dataclass
class EngineConfig:
    """Everything needed to build an engine (types.py:521-593)."""

    model: str
    tokenizer: str | None = None
    dtype: str = "auto"  # auto | bfloat16 | float32
    device: str = "auto"  # auto | cuda | cuda:N
    gpu_memory_utilization: float = 0.9
    max_model_len: int | None = None
    seed: int | None = None
    scheduler: SchedulerConfig = field(default_factory=SchedulerConfig)
    #: In the reference's record (types.py:543-547) for subsystems that are not built here:
    #: only ``None`` is accepted.
    speculative: dict | None = None
    lora: dict | None = None
    #: Step sizes (tokens) at which the BLAS library's kernels for this model's projections are
    #: timed at start-up and the fastest kept (bfloat16 only; a few seconds per size).  Empty:
    #: the library's own heuristic picks.  No counterpart in the reference.
    tune_gemm_tokens: tuple[int, ...] = ()
    #: Run the library products of every step at one of a few sizes (the next one up: multiples
    #: of 32 tokens to 256, of 64 to 512, of 128 to 1,024, of 256 beyond, and the token budget)
    #: and time the library's kernels at all of them at start-up, so that every step, not only
    #: one of a listed size, runs on timed kernels (bfloat16 only; a minute or two the first
    #: time, read from ``gemm_tuning_file`` afterwards).  No counterpart in the reference.
    tune_gemm_step_sizes: bool = False
    #: Where the timed choices are kept between runs; None is a per-user cache file.
    gemm_tuning_file: str | None = None
    #: Launch a decode step before the host has read the tokens of the step before it (they
    #: are copied on the device), so that the GPU does not wait while the host schedules and
    #: builds outputs.  Results are the same tokens; a request that ends on a stop token costs
    #: one token's worth of work that is thrown away.  No counterpart in the reference.
    run_ahead: bool = True

    def __post_init__(self) -> None:
        if self.speculative is not None or self.lora is not None:
            raise ValueError("speculative decoding and LoRA are not built: leave `speculative` and `lora` at None")
        if self.dtype not in ("auto", "bfloat16", "float32"):
            raise ValueError(f"unsupported dtype {self.dtype!r}; expected auto, bfloat16 or float32")
        if self.device != "auto" and not self.device.startswith("cuda"):
            raise ValueError(f"unsupported device {self.device!r}: this engine runs on the GPU only")
        if not 0.0 < self.gpu_memory_utilization <= 1.0:
            raise ValueError(f"gpu_memory_utilization must be in (0, 1], got {self.gpu_memory_utilization!r}")
        if self.max_model_len is not None and self.max_model_len < 1:
            raise ValueError(f"max_model_len must be >= 1, got {self.max_model_len!r}")
        self.tune_gemm_tokens = tuple(self.tune_gemm_tokens)
        if any(isinstance(t, bool) or not isinstance(t, int) or t < 1 for t in self.tune_gemm_tokens):
            raise ValueError(f"tune_gemm_tokens must be ints >= 1, got {self.tune_gemm_tokens!r}")

    @classmethod
    def from_env(cls, environ: Mapping[str, str] | None = None, **overrides: Any) -> "EngineConfig":
        """An engine configuration from the process-wide ``TURBOSERVE_*`` variables the
        reference's settings read (src/turboserve/config.py:38-64, types.py:575-593): MODEL,
        DTYPE, DEVICE, GPU_MEMORY_UTILIZATION, MAX_NUM_SEQS, MAX_NUM_BATCHED_TOKENS, BLOCK_SIZE,
        NUM_BLOCKS, ENABLE_CHUNKED_PREFILL, and this engine's own RUN_AHEAD.  Unset variables keep this class's defaults;
        ``overrides`` win over the environment."""
        env = os.environ if environ is None else environ

        def get(name: str, convert):
            raw = env.get(f"TURBOSERVE_{name}")
            return None if raw is None or raw == "" else convert(raw)

        def truth(raw: str) -> bool:
            if raw.strip().lower() in ("1", "true", "yes", "on"):
                return True
            if raw.strip().lower() in ("0", "false", "no", "off"):
                return False
            raise ValueError(f"not a boolean: {raw!r}")

        scheduler = {k: v for k, v in {
            "max_num_seqs": get("MAX_NUM_SEQS", int),
            "max_num_batched_tokens": get("MAX_NUM_BATCHED_TOKENS", int),
            "block_size": get("BLOCK_SIZE", int),
            "num_blocks": get("NUM_BLOCKS", int),
            "enable_chunked_prefill": get("ENABLE_CHUNKED_PREFILL", truth),
        }.items() if v is not None}
        fields = {k: v for k, v in {
            "model": get("MODEL", str),
            "dtype": get("DTYPE", str),
            "device": get("DEVICE", str),
            "gpu_memory_utilization": get("GPU_MEMORY_UTILIZATION", float),
            "run_ahead": get("RUN_AHEAD", truth),
        }.items() if v is not None}
        fields["scheduler"] = SchedulerConfig(**scheduler)
        fields.update(overrides)
        if "model" not in fields:
            raise ValueError("no model: set TURBOSERVE_MODEL or pass model=")
        return cls(**fields)

    @property
    def block_size(self) -> int:
        return self.scheduler.block_size

    @property
    def num_blocks(self) -> int | None:
        return self.scheduler.num_blocks

    def resolved_device(self) -> str:
        return "cuda:0" if self.device in ("auto", "cuda") else self.device

    def resolved_dtype(self) -> str:
        """``auto`` is bfloat16: the matrix cores' native serving precision here (the
        reference's ``auto`` picks float16 on a GPU, types.py:566-574)."""
        return "bfloat16" if self.dtype == "auto" else self.dtype
