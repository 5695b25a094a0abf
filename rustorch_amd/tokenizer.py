"""Tokenizer side of the CLI: the mirror of `TokenizerWrapper`
(example-cli/src/tokenizer/wrapper.rs:7-103), a thin layer over the Hugging Face `tokenizers` file format
(`tokenizer.json`), with the same special-token lookups."""
from __future__ import annotations

import os
from typing import Sequence

from .errors import InvalidParameters


class TokenizerWrapper:
    def __init__(self, tokenizer):
        self.tokenizer = tokenizer

    @classmethod
    def from_file(cls, path) -> "TokenizerWrapper":
        """wrapper.rs:14-29: a missing file and an unreadable one are two different errors."""
        from tokenizers import Tokenizer
        path = os.fspath(path)
        if not os.path.exists(path):
            raise InvalidParameters("Tokenizer file not found: %s" % path)
        try:
            return cls(Tokenizer.from_file(path))
        except Exception as e:                      # the library raises its own exception type
            raise InvalidParameters("Failed to load tokenizer: %s" % e) from e

    @classmethod
    def dummy(cls) -> "TokenizerWrapper":
        """wrapper.rs:32-42: an empty BPE model, for tests."""
        from tokenizers import Tokenizer
        from tokenizers.models import BPE
        return cls(Tokenizer(BPE()))

    def inner(self):
        return self.tokenizer

    def encode(self, text: str, add_special_tokens: bool = True) -> list[int]:
        return list(self.tokenizer.encode(text, add_special_tokens=add_special_tokens).ids)

    def decode(self, ids: Sequence[int], skip_special_tokens: bool = True) -> str:
        return self.tokenizer.decode([int(i) for i in ids], skip_special_tokens=skip_special_tokens)

    def vocab_size(self) -> int:
        return int(self.tokenizer.get_vocab_size(with_added_tokens=True))

    def _first(self, *names):
        for n in names:
            i = self.tokenizer.token_to_id(n)
            if i is not None:
                return int(i)
        return None

    def bos_token_id(self):
        return self._first("<s>", "[BOS]", "<|begin_of_text|>")

    def eos_token_id(self):
        return self._first("</s>", "[EOS]", "<|end_of_text|>")

    def pad_token_id(self):
        return self._first("<pad>", "[PAD]")

    def unk_token_id(self):
        return self._first("<unk>", "[UNK]")
