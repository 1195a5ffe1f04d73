"""Incremental detokenisation for streaming: decode a small window of recent tokens instead of the
whole output, and hold back while the tail is an incomplete character (reference:
tensorline/detok.py:13-27).  Works with any tokenizer that has ``decode(ids, skip_special_tokens)``."""
from __future__ import annotations


class IncrementalDetokenizer:
    def __init__(self, tokenizer):
        self.tokenizer = tokenizer
        self.ids: list[int] = []
        self.window_start = 0      # start of the already emitted window kept for context
        self.emitted_upto = 0      # tokens before this index have been emitted

    def push(self, new_ids: list[int]) -> str:
        self.ids.extend(new_ids)
        old = self.tokenizer.decode(self.ids[self.window_start:self.emitted_upto], skip_special_tokens=True)
        new = self.tokenizer.decode(self.ids[self.window_start:], skip_special_tokens=True)
        if len(new) > len(old) and not new.endswith("�"):
            self.window_start, self.emitted_upto = self.emitted_upto, len(self.ids)
            return new[len(old):]
        return ""
