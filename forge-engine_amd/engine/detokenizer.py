"""Text out of generated token ids, a fragment at a time.

Behaviour follows the reference's incremental detokenizer
(src/forge_engine/engine.py:295-362): every push decodes the whole generated
sequence again; text that could still grow into a stop string, and trailing
U+FFFD (half of a multi-byte character), is held back; a complete stop string
ends the text just before it.
"""

from __future__ import annotations

REPLACEMENT = "�"


class IncrementalDetokenizer:
    def __init__(self, tokenizer, stop_strings=()) -> None:
        if any(not stop for stop in stop_strings):
            raise ValueError("stop strings must be non-empty")
        self._tokenizer = tokenizer
        self._stops = tuple(stop_strings)
        self._ids: list[int] = []
        self._text = ""
        self._sent = 0
        self._stopped = False

    @property
    def stopped(self) -> bool:
        return self._stopped

    @property
    def token_ids(self) -> tuple[int, ...]:
        return tuple(self._ids)

    def push(self, token_id: int) -> str:
        if self._stopped:
            raise RuntimeError("cannot push tokens after a stop string")
        self._ids.append(token_id)
        self._text = self._tokenizer.decode(self._ids, skip_special_tokens=True)
        return self._emit(final=False)

    def finish(self) -> str:
        return "" if self._stopped else self._emit(final=True)

    def _emit(self, final: bool) -> str:
        text = self._text
        hits = [at for at in (text.find(stop) for stop in self._stops) if at >= 0]
        if hits:
            end = min(hits)
            self._stopped = True
        elif final:
            end = len(text)
        else:
            held = len(text) - len(text.rstrip(REPLACEMENT))
            for stop in self._stops:
                for size in range(min(len(text), len(stop) - 1), held, -1):
                    if text.endswith(stop[:size]):
                        held = size
                        break
            end = len(text) - held
        if end < self._sent:
            raise ValueError("the tokenizer changed text that was already sent")
        fragment = text[self._sent:end]
        self._sent = end
        return fragment
