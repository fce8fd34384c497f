"""Incremental detokenisation and stop strings (src/turboserve/engine/runtime/streaming.py:91-351).

A tokenizer is needed only for text: prompts and outputs as token ids work without one.
"""

from __future__ import annotations

from collections.abc import Iterable
from dataclasses import dataclass
from pathlib import Path
from typing import Any

REPLACEMENT_CHAR = "�"
WINDOW_TOKENS = 8


@dataclass
class DecodedDelta:
    text: str = ""
    stop: str | None = None

    @property
    def stopped(self) -> bool:
        return self.stop is not None


class TokenizerFile:
    """A ``tokenizer.json`` read with the ``tokenizers`` library (a file-format library, no
    model code).  ``encode`` adds no special tokens (src/turboserve/engine/runtime/engine.py:270-281)."""

    def __init__(self, path: str | Path) -> None:
        from tokenizers import Tokenizer

        self._tok = Tokenizer.from_file(str(path))
        #: The id of the end-of-sequence token that ``tokenizer_config.json`` beside the file
        #: names (``"eos_token"``: a string, or a mapping with ``"content"``), or ``None``.
        self.eos_token_id: int | None = None
        config = Path(path).with_name("tokenizer_config.json")
        if config.is_file():
            import json

            named = json.loads(config.read_text(encoding="utf-8")).get("eos_token")
            if isinstance(named, dict):
                named = named.get("content")
            if isinstance(named, str):
                self.eos_token_id = self._tok.token_to_id(named)

    def encode(self, text: str, add_special_tokens: bool = False) -> list[int]:
        return list(self._tok.encode(text, add_special_tokens=add_special_tokens).ids)

    def decode(self, token_ids: list[int], skip_special_tokens: bool = True) -> str:
        return self._tok.decode(list(token_ids), skip_special_tokens=skip_special_tokens)


def get_tokenizer(path: str | Path | None) -> TokenizerFile | None:
    """The tokenizer of a model folder, or ``None`` if it has no ``tokenizer.json``."""
    if path is None:
        return None
    candidate = Path(path)
    if candidate.is_dir():
        candidate = candidate / "tokenizer.json"
    return TokenizerFile(candidate) if candidate.is_file() else None


class IncrementalDetokenizer:
    """Windowed re-decoding: text is the difference between decoding ``tokens[prefix:]`` and
    ``tokens[prefix:read]``; a window that ends inside a character (U+FFFD) emits nothing yet
    (streaming.py:91-190)."""

    def __init__(self, tokenizer: Any, *, skip_special_tokens: bool = True) -> None:
        self._tokenizer = tokenizer
        self._skip = skip_special_tokens
        self._tokens: list[int] = []
        self._prefix = 0
        self._read = 0
        self.text = ""

    def _decode(self, ids: list[int]) -> str:
        return self._tokenizer.decode(list(ids), skip_special_tokens=self._skip)

    def append(self, token_ids: Iterable[int]) -> str:
        new = list(token_ids)
        if not new:
            return ""
        self._tokens.extend(new)
        before = self._decode(self._tokens[self._prefix:self._read])
        window = self._decode(self._tokens[self._prefix:])
        if window.endswith(REPLACEMENT_CHAR):
            return ""
        if window.startswith(before):
            delta = window[len(before):]
        else:
            full = self._decode(self._tokens)
            delta = full[len(self.text):] if full.startswith(self.text) else full
        self._prefix = self._read
        self._read = len(self._tokens)
        if len(self._tokens) - self._prefix > WINDOW_TOKENS:
            self._prefix = len(self._tokens) - WINDOW_TOKENS
        self.text += delta
        return delta

    def flush(self) -> str:
        if self._read >= len(self._tokens):
            return ""
        before = self._decode(self._tokens[self._prefix:self._read])
        window = self._decode(self._tokens[self._prefix:])
        delta = window[len(before):] if window.startswith(before) else ""
        self._prefix = self._read
        self._read = len(self._tokens)
        self.text += delta
        return delta


class StopStringMatcher:
    """Holds back the shortest suffix that could still grow into a stop string and cuts the
    text before a completed one (streaming.py:193-262)."""

    def __init__(self, stop: Iterable[str] = ()) -> None:
        self._stop = tuple(s for s in stop if s)
        self._max_len = max((len(s) for s in self._stop), default=0)
        self._buffer = ""

    @property
    def is_active(self) -> bool:
        return bool(self._stop)

    def feed(self, text: str) -> DecodedDelta:
        if not self._stop:
            return DecodedDelta(text=text)
        self._buffer += text
        hits = [(self._buffer.find(s), s) for s in self._stop if s in self._buffer]
        if hits:
            index, matched = min(hits)
            emit, self._buffer = self._buffer[:index], ""
            return DecodedDelta(text=emit, stop=matched)
        keep = 0
        for length in range(min(len(self._buffer), self._max_len - 1), 0, -1):
            if any(s.startswith(self._buffer[-length:]) for s in self._stop):
                keep = length
                break
        emit = self._buffer[:len(self._buffer) - keep]
        self._buffer = self._buffer[len(self._buffer) - keep:]
        return DecodedDelta(text=emit)

    def flush(self) -> str:
        pending, self._buffer = self._buffer, ""
        return pending


class StreamingDecoder:
    """Per-request text state: detokeniser plus stop-string matcher (streaming.py:265-327).
    Without a tokenizer it emits no text and never stops on a string."""

    def __init__(self, tokenizer: Any | None, stop: Iterable[str] = ()) -> None:
        self.detokenizer = IncrementalDetokenizer(tokenizer) if tokenizer is not None else None
        self.matcher = StopStringMatcher(stop if tokenizer is not None else ())
        self.text = ""

    def feed(self, token_ids: Iterable[int]) -> DecodedDelta:
        if self.detokenizer is None:
            return DecodedDelta()
        delta = self.matcher.feed(self.detokenizer.append(token_ids))
        self.text += delta.text
        return delta

    def finish(self) -> str:
        if self.detokenizer is None:
            return ""
        tail = self.detokenizer.flush()
        pending = self.matcher.flush() + tail if self.matcher.is_active else tail
        self.text += pending
        return pending
