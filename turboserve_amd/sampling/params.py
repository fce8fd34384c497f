"""Per-request sampling options (src/turboserve/engine/core/types.py:97-143)."""

from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum


class FinishReason(str, Enum):
    """Why a request stopped (types.py:127-143).  ``str`` values so they serialise as is."""

    STOP = "stop"
    LENGTH = "length"
    ABORT = "abort"

    def __str__(self) -> str:
        return self.value


@dataclass
class SamplingParams:
    """Names, defaults and bounds as the reference's (types.py:110-119): ``temperature == 0``
    is greedy, ``top_k == 0`` is no top-k filter, ``top_p == 1`` no nucleus filter."""

    max_tokens: int = 128
    temperature: float = 1.0
    top_p: float = 1.0
    top_k: int = 0
    seed: int | None = None
    stop_token_ids: list[int] = field(default_factory=list)
    stop: list[str] = field(default_factory=list)
    repetition_penalty: float = 1.0
    ignore_eos: bool = False
    logprobs: bool = False

    def __post_init__(self) -> None:
        if isinstance(self.max_tokens, bool) or not isinstance(self.max_tokens, int) or self.max_tokens < 1:
            raise ValueError(f"max_tokens must be an int >= 1, got {self.max_tokens!r}")
        if not self.temperature >= 0.0:
            raise ValueError(f"temperature must be >= 0, got {self.temperature!r}")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError(f"top_p must be in (0, 1], got {self.top_p!r}")
        if isinstance(self.top_k, bool) or not isinstance(self.top_k, int) or self.top_k < 0:
            raise ValueError(f"top_k must be an int >= 0, got {self.top_k!r}")
        if not self.repetition_penalty > 0.0:
            raise ValueError(f"repetition_penalty must be > 0, got {self.repetition_penalty!r}")
        if self.seed is not None and (isinstance(self.seed, bool) or not isinstance(self.seed, int)):
            raise ValueError(f"seed must be an int, got {self.seed!r}")
        self.temperature = float(self.temperature)
        self.top_p = float(self.top_p)
        self.repetition_penalty = float(self.repetition_penalty)
        self.stop_token_ids = [int(t) for t in self.stop_token_ids]
        self.stop = [str(s) for s in self.stop]

    @property
    def is_greedy(self) -> bool:
        return self.temperature == 0.0

    @property
    def is_plain_greedy(self) -> bool:
        """Greedy with nothing that changes the argmax or asks for more than the token."""
        return self.is_greedy and self.repetition_penalty == 1.0 and not self.logprobs
