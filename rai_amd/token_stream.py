"""Incremental detokenisation for the text-generation loop.

Mirrors `TokenOutputStream` of the reference (rai-models/src/llm/mod.rs:6-69): the stream keeps every token id seen so
far and two cursors; `next_token` decodes the not-yet-emitted tail once without and once with the new token and hands
back the new text only when the decoded string grew and ends in an alphanumeric character, so a multi-token UTF-8
sequence or a word piece is held back until it is complete.

The tokenizer is any object with the Hugging Face `tokenizers.Tokenizer` calls used here:
`encode(text, add_special_tokens=True).ids` and `decode(ids, skip_special_tokens=True)`.

Lengths and the split point are byte offsets of the UTF-8 text, as in the reference (`String::len`,
`str::split_at`); a split inside a character raises, where the reference panics.
"""
from __future__ import annotations

import unicodedata
from typing import List, Optional, Sequence


def _is_alphanumeric(ch: str) -> bool:
    """`char::is_alphanumeric`: Unicode Alphabetic, or a number of category Nd, Nl or No.

    Alphabetic is the letter categories plus Nl plus Other_Alphabetic; the latter (combining vowel signs and the like,
    categories Mn/Mc/So) has no accessor in `unicodedata`, so of those only the combining marks are taken: a text that
    ends in one is emitted, as the reference does for the marks that carry the property.
    """
    cat = unicodedata.category(ch)
    return cat[0] == "L" or cat in ("Nd", "Nl", "No", "Mc") or (cat == "Mn" and unicodedata.combining(ch) == 0)


class TokenOutputStream:
    def __init__(self, tokenizer):
        self.tokenizer = tokenizer
        self._tokens: List[int] = []
        self.current_index = 0
        self.prev_index = 0

    def tokens(self) -> Sequence[int]:
        return self._tokens

    def is_empty(self) -> bool:
        return not self._tokens

    def __len__(self) -> int:
        return len(self._tokens)

    def prompt(self, prompt: str) -> None:
        """Tokenises `prompt` with special tokens and appends it (mod.rs:37-42)."""
        self._tokens.extend(int(t) for t in self.tokenizer.encode(prompt, add_special_tokens=True).ids)
        self.prev_index = self.current_index
        self.current_index = len(self._tokens)

    def _decode(self, ids: Sequence[int]) -> str:
        return self.tokenizer.decode(list(ids), skip_special_tokens=True)

    def next_token(self, token: int) -> Optional[str]:
        """Appends `token`; returns the newly completed text or None (mod.rs:50-67)."""
        prev_text = "" if not self._tokens else self._decode(self._tokens[self.prev_index:self.current_index])
        self._tokens.append(int(token))
        text = self._decode(self._tokens[self.prev_index:])
        prev_bytes, text_bytes = prev_text.encode("utf-8"), text.encode("utf-8")
        if len(text_bytes) > len(prev_bytes) and _is_alphanumeric(text[-1]):
            tail = text_bytes[len(prev_bytes):]
            try:
                new_text = tail.decode("utf-8")
                text_bytes[:len(prev_bytes)].decode("utf-8")
            except UnicodeDecodeError as e:
                raise ValueError("byte index %d is not a char boundary" % len(prev_bytes)) from e
            self.prev_index = self.current_index
            self.current_index = len(self._tokens)
            return new_text
        return None
