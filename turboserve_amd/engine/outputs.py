"""What the engine hands back for a request (src/turboserve/engine/core/types.py:596-634)."""

from __future__ import annotations

from dataclasses import dataclass, field

from turboserve_amd.engine.sequence import RequestTiming
from turboserve_amd.sampling.params import FinishReason


@dataclass
class RequestOutput:
    """One step's progress on one request: the new token ids and text (a delta, not the
    total), whether and why it finished, and running counts."""

    request_id: str
    new_token_ids: list[int] = field(default_factory=list)
    text_delta: str = ""
    finished: bool = False
    finish_reason: FinishReason | None = None
    timing: RequestTiming | None = None
    prompt_tokens: int = 0
    output_tokens: int = 0
    cached_prompt_tokens: int = 0  # always 0: there is no prefix cache (types.py:596-634 has the field)
    logprobs: list[float] = field(default_factory=list)
