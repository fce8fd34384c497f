"""Text out of token ids, piece by piece, and stop strings.

The behaviour is the reference's (src/turboserve/engine/runtime/streaming.py:91-351): text is
passed on as soon as it is certain, a character whose bytes have not all arrived is held back,
text that could still grow into a stop string is held back, a completed stop string ends the
request and is cut from its text, and whatever is held when the request ends otherwise is
passed on.  The design is this engine's: one object per request (:class:`TextStream`) that
re-decodes only a short tail of the tokens and finds stop strings with one automaton over all
of them, a character at a time, so that the result does not depend on how the text arrived in
pieces.

A tokenizer is needed only for text: prompts and outputs as token ids work without one.
"""

from __future__ import annotations

from collections.abc import Iterable
from dataclasses import dataclass
from pathlib import Path
from typing import Any

#: What a decoder puts where bytes do not (yet) make a character.
UNDECIDED = "\ufffd"


@dataclass
class TextDelta:
    """What a push of tokens released: ``text`` to pass on, and the stop string that ended the
    request, if one did."""

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


class StopAutomaton:
    """All stop strings as one trie with fall-back links (Aho-Corasick): fed a character at a
    time, its state is the longest end of the text so far that begins a stop string, which is
    exactly the text that has to be held back; a state that ends a stop string means the
    request stops.  Where several stop strings end at the same character, the longest counts
    (it begins earliest)."""

    def __init__(self, stops: Iterable[str]) -> None:
        self.stops = tuple(dict.fromkeys(s for s in stops if s))
        self._next: list[dict[str, int]] = [{}]
        self._depth = [0]
        self._ends: list[str | None] = [None]  # the longest stop string that ends in this state
        for stop in self.stops:
            node = 0
            for char in stop:
                if char not in self._next[node]:
                    self._next[node][char] = len(self._next)
                    self._next.append({})
                    self._depth.append(self._depth[node] + 1)
                    self._ends.append(None)
                node = self._next[node][char]
            self._ends[node] = stop
        # Fall-back links, breadth first: the longest proper end of a state's string that is itself
        # a beginning of a stop string; a state inherits a stop string that ends in its fall-back.
        self._back = [0] * len(self._next)
        queue = list(self._next[0].values())
        for node in queue:
            for char, child in self._next[node].items():
                back = self._back[node]
                while back and char not in self._next[back]:
                    back = self._back[back]
                self._back[child] = self._next[back].get(char, 0)
                if self._ends[child] is None:
                    self._ends[child] = self._ends[self._back[child]]
                queue.append(child)

    def step(self, state: int, char: str) -> int:
        while state and char not in self._next[state]:
            state = self._back[state]
        return self._next[state].get(char, 0)

    def held(self, state: int) -> int:
        """Characters at the end of the text that may still become a stop string."""
        return self._depth[state]

    def ended(self, state: int) -> str | None:
        return self._ends[state]


class TextStream:
    """One request's text.  ``push(token_ids)`` returns what those tokens release; ``close()``
    what is still held when the request ends for another reason than a stop string.

    Decoding: only a tail of the tokens is ever decoded again.  The tail is re-decoded whole at
    every push, because a tokenizer joins tokens by rules of its own (a space before a word, a
    character spread over several tokens); of its text, what was passed on before is skipped
    and the rest is new, except for the characters at the very end that are still undecided
    (the decoder's U+FFFD for bytes that do not make a character yet).  When the tail has grown
    past ``RESEAL_TOKENS`` and ends on a whole character, all but its last ``CONTEXT_TOKENS``
    tokens are sealed: they are never decoded again, and the kept ones (whose text has been
    passed on) stay as the context the next tokens are joined to.  Should a tail's text ever
    not continue what it spelled before (a decoder that rewrites earlier characters), text
    that is out stays out and the new text goes on from where the two part.

    Without a tokenizer nothing is decoded, no text is released and no stop string is found.
    """

    RESEAL_TOKENS = 24
    CONTEXT_TOKENS = 6

    def __init__(self, tokenizer: Any | None, stop: Iterable[str] = (), *, skip_special_tokens: bool = True) -> None:
        self._tokenizer = tokenizer
        self._skip = skip_special_tokens
        self._automaton = StopAutomaton(stop) if tokenizer is not None else StopAutomaton(())
        self._state = 0
        self._tail: list[int] = []   # the tokens decoded at every push
        self._spelled = ""           # the part of the tail's text that has gone to the stop automaton
        self._held = ""              # text gone to the automaton that it holds back
        self.stopped_by: str | None = None
        self.text = ""               # everything released so far

    # -- decoding ------------------------------------------------------------------------------

    def _spell(self) -> str:
        return self._tokenizer.decode(list(self._tail), skip_special_tokens=self._skip)

    def _certain(self, token_ids: Iterable[int]) -> str:
        """The text that the new tokens make certain."""
        self._tail.extend(token_ids)
        spelled = self._spell()
        decided = len(spelled.rstrip(UNDECIDED))
        if spelled.startswith(self._spelled):
            start = len(self._spelled)
        else:  # the decoder rewrote what it had spelled: go on from where the two texts part
            start = next((i for i, (a, b) in enumerate(zip(spelled, self._spelled)) if a != b), min(len(spelled), len(self._spelled)))
        fresh = spelled[start:decided] if decided > start else ""
        self._spelled = spelled[:max(decided, start)]
        if len(self._tail) > self.RESEAL_TOKENS and decided == len(spelled):
            self._tail = self._tail[-self.CONTEXT_TOKENS:]
            self._spelled = self._spell()
        return fresh

    # -- stop strings --------------------------------------------------------------------------

    def _screen(self, fresh: str) -> TextDelta:
        """Pass ``fresh`` through the stop automaton: what it lets go, and a stop if one ended."""
        if not self._automaton.stops:
            return TextDelta(fresh)
        pending = self._held + fresh
        for offset, char in enumerate(fresh):
            self._state = self._automaton.step(self._state, char)
            ended = self._automaton.ended(self._state)
            if ended is not None:
                upto = len(self._held) + offset + 1 - len(ended)
                self._held, self.stopped_by = "", ended
                return TextDelta(pending[:upto], ended)
        keep = self._automaton.held(self._state)
        self._held = pending[len(pending) - keep:] if keep else ""
        return TextDelta(pending[:len(pending) - keep])

    # -- the request's side --------------------------------------------------------------------

    def push(self, token_ids: Iterable[int]) -> TextDelta:
        if self._tokenizer is None or self.stopped_by is not None:
            return TextDelta()
        delta = self._screen(self._certain(token_ids))
        self.text += delta.text
        return delta

    def close(self) -> str:
        """The request ended (length, an end token, an abort): everything still held is text."""
        if self._tokenizer is None or self.stopped_by is not None:
            return ""
        spelled = self._spell() if self._tail else ""
        undecided = spelled[len(self._spelled):] if spelled.startswith(self._spelled) else ""
        rest, self._held, self._tail, self._spelled = self._held + undecided, "", [], ""
        self.text += rest
        return rest
