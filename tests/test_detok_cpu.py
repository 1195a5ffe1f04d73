"""Incremental detokenisation: pieces pushed token by token, or several at a time, join to the text
of decoding everything at once, on text whose characters span several tokens (analogue of the
reference's tests/test_streaming.py:20-29)."""
import pytest

from tensorline_amd.engine.detok import IncrementalDetokenizer

TEXTS = ["plain words, twice  spaced", "café naïve — ﬁne", "你好，世界！ mixed 日本語 text",
         "faces \U0001F600\U0001F44D\U0001F3FD and a flag \U0001F1E9\U0001F1EA", "x"]


class ByteTokenizer:
    """One token per UTF-8 byte: every character beyond ASCII is spread over several tokens."""

    def __init__(self):
        self.decodes = 0

    def encode(self, text):
        return list(text.encode("utf-8"))

    def decode(self, ids, skip_special_tokens=True):
        self.decodes += 1
        return bytes(ids).decode("utf-8", errors="replace")


class WordTokenizer:
    """A token is a word with the space before it; decoding drops the space that starts a text, as
    sentence-piece style tokenizers do: what a token gives depends on what stands before it."""

    def __init__(self):
        self.words: list[str] = []

    def encode(self, text):
        out = []
        for w in text.split(" "):
            if w not in self.words:
                self.words.append(w)
            out.append(self.words.index(w))
        return out

    def decode(self, ids, skip_special_tokens=True):
        return " ".join(self.words[i] for i in ids)


def trained_bpe():
    """A byte-level BPE of the tokenizers package, trained here on a few lines."""
    tokenizers = pytest.importorskip("tokenizers")
    from tokenizers import decoders, models, pre_tokenizers, trainers
    tok = tokenizers.Tokenizer(models.BPE())
    tok.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False)
    tok.decoder = decoders.ByteLevel()
    trainer = trainers.BpeTrainer(vocab_size=300, initial_alphabet=pre_tokenizers.ByteLevel.alphabet(), show_progress=False)
    tok.train_from_iterator(TEXTS * 3, trainer)

    class Wrapped:
        def encode(self, text):
            return tok.encode(text).ids

        def decode(self, ids, skip_special_tokens=True):
            return tok.decode(ids, skip_special_tokens=skip_special_tokens)
    return Wrapped()


@pytest.mark.parametrize("make", [ByteTokenizer, WordTokenizer, trained_bpe], ids=["bytes", "words", "bpe"])
@pytest.mark.parametrize("step", [1, 2, 3, 5])
def test_pieces_join_to_the_full_decode(make, step):
    tok = make()
    for text in TEXTS:
        ids = tok.encode(text)
        d = IncrementalDetokenizer(tok)
        pieces = [d.push(ids[i:i + step]) for i in range(0, len(ids), step)]
        assert "�" not in "".join(pieces)
        assert "".join(pieces) + d.flush() == tok.decode(ids) == text


def test_unfinished_characters_are_held_back_and_cost_one_decode():
    tok = ByteTokenizer()
    d = IncrementalDetokenizer(tok)
    ids = tok.encode("a\U0001F600b")
    assert d.push(ids[:1]) == "a"
    before = tok.decodes
    assert [d.push([t]) for t in ids[1:4]] == ["", "", ""]          # three of the emoji's four bytes
    assert tok.decodes - before == 3                                # the last piece's text is not decoded again
    assert d.push(ids[4:5]) == "\U0001F600" and d.push(ids[5:]) == "b"
    # a text that ends in the middle of a character: flush gives what a full decode gives
    d = IncrementalDetokenizer(tok)
    assert d.push(ids[:3]) == "" and d.flush() == tok.decode(ids[:3]) and d.flush() == ""
