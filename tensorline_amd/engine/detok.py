"""Text of a growing token sequence, piece by piece, for streaming.

Tokens do not turn into text one by one.  A character may be spread over several tokens (the
bytes of one UTF-8 character), and what a token decodes to may depend on what stands before it
(a tokenizer drops the space of a word that starts a text).  Decoding the whole output again for
every token would fix both and cost time quadratic in its length.  Instead (the method of the
reference's streaming path, tensorline/detok.py:13-27) new tokens are decoded together with the
tokens of the piece emitted last, and the new piece is what that joint text has beyond the text
of the last piece alone; while the joint text ends in U+FFFD, the mark of an unfinished
character, nothing is emitted and the tokens are held for the next call.

The text of the last piece alone is kept, not decoded again on every call, so a call that emits
nothing costs one decode and a call that emits costs two.  Works with any tokenizer that has
``decode(ids, skip_special_tokens=...)``.
"""
from __future__ import annotations

UNFINISHED = "�"


class IncrementalDetokenizer:
    def __init__(self, tokenizer):
        self.tokenizer = tokenizer
        self._context: list[int] = []      # the tokens of the piece emitted last
        self._context_text = ""            # what they decode to on their own
        self._held: list[int] = []         # tokens since then, not emitted yet

    def _decode(self, ids: list[int]) -> str:
        return self.tokenizer.decode(ids, skip_special_tokens=True) if ids else ""

    def _emit(self, joint: str) -> str:
        piece = joint[len(self._context_text):]
        self._context, self._held = self._held, []
        self._context_text = self._decode(self._context)
        return piece

    def push(self, new_ids: list[int]) -> str:
        """Take more tokens; returns the text that is now certain, or "" while a character is unfinished."""
        self._held.extend(int(t) for t in new_ids)
        if not self._held:
            return ""
        joint = self._decode(self._context + self._held)
        if joint.endswith(UNFINISHED) or len(joint) <= len(self._context_text):
            return ""
        return self._emit(joint)

    def flush(self) -> str:
        """At the end of the output: whatever is still held, an unfinished character included."""
        if not self._held:
            return ""
        joint = self._decode(self._context + self._held)
        return self._emit(joint) if len(joint) > len(self._context_text) else ""
