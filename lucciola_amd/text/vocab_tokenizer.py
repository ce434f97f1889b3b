"""Text to token ids and back, as the reference's ``QwenTokenizer`` does it
(include/tokenizer.h:9-19, src/tokenizer.cc): ``vocab.json`` alone (token string -> id), no
merges and no special-token parsing.  The engine itself knows token ids only; this is the
convenience around it that the reference's command line and ``AsyncEngine`` have.

Encoding (src/tokenizer.cc:87-132): every byte of the UTF-8 text becomes one character of
the byte-level alphabet of the vocabulary; from the front, the longest entry of the
vocabulary that the rest starts with is taken; a character that starts no entry is dropped.
Decoding (src/tokenizer.cc:159-204): the token's characters go back to bytes; a character
outside the alphabet stands for its own UTF-8 bytes.
"""
from __future__ import annotations

import codecs
import json
from dataclasses import dataclass
from typing import Dict, Iterable, List, Sequence


def byte_alphabet() -> List[str]:
    """The character that stands for each byte (src/tokenizer.cc:45-63): printable bytes
    ('!'..'~', 0xA1..0xAC, 0xAE..0xFF) stand for themselves, the others take the code points
    from 256 on in their order."""
    own = set(range(0x21, 0x7F)) | set(range(0xA1, 0xAD)) | set(range(0xAE, 0x100))
    table, fresh = [], 256
    for b in range(256):
        if b in own:
            table.append(chr(b))
        else:
            table.append(chr(fresh))
            fresh += 1
    return table


class VocabTokenizer:
    def __init__(self, vocab: Dict[str, int]):
        if not vocab:
            raise ValueError("the vocabulary is empty")
        self.token_to_id = {str(t): int(i) for t, i in vocab.items()}
        size = max(self.token_to_id.values()) + 1
        self.id_to_token: List[str] = [""] * size
        for token, i in self.token_to_id.items():
            if 0 <= i < size:
                self.id_to_token[i] = token
        self._longest = max(len(t) for t in self.token_to_id)
        self._to_char = byte_alphabet()
        self._to_byte = {c: b for b, c in enumerate(self._to_char)}

    @classmethod
    def from_file(cls, path: str) -> "VocabTokenizer":
        with open(path, "r", encoding="utf-8") as fh:
            return cls(json.load(fh))

    def __len__(self) -> int:
        return len(self.id_to_token)

    def encode(self, text: str) -> List[int]:
        mapped = "".join(self._to_char[b] for b in text.encode("utf-8"))
        ids, at, n = [], 0, len(mapped)
        while at < n:
            for length in range(min(self._longest, n - at), 0, -1):
                found = self.token_to_id.get(mapped[at:at + length])
                if found is not None:
                    ids.append(found)
                    at += length
                    break
            else:
                at += 1          # nothing in the vocabulary starts here
        return ids

    def token_bytes(self, token_id: int) -> bytes:
        """The bytes of one token; an id outside the vocabulary is empty (src/tokenizer.cc:160-162)."""
        if not 0 <= token_id < len(self.id_to_token):
            return b""
        out = bytearray()
        for ch in self.id_to_token[token_id]:
            b = self._to_byte.get(ch)
            if b is None:
                out += ch.encode("utf-8")
            else:
                out.append(b)
        return bytes(out)

    def decode(self, ids: Iterable[int]) -> str:
        return b"".join(self.token_bytes(i) for i in ids).decode("utf-8", errors="replace")

    def stream(self) -> "TextStream":
        return TextStream(self)


class TextStream:
    """Text of a request token by token: a character whose bytes are spread over several
    tokens comes out with the token that completes it."""

    def __init__(self, tokenizer: VocabTokenizer):
        self._tokenizer = tokenizer
        self._decoder = codecs.getincrementaldecoder("utf-8")(errors="replace")

    def feed(self, token_id: int, last: bool = False) -> str:
        return self._decoder.decode(self._tokenizer.token_bytes(token_id), final=last)


@dataclass(frozen=True)
class ChatFormat:
    """The prompt the reference builds around a user's line (src/async_engine.cc:82-106,
    examples/qwen_dynamic.cc:48-66): <start> "system\\n" system <end> <enter> <start>
    "user\\n" line <end> <enter> <start> "assistant\\n".  The three ids are not in vocab.json;
    the defaults are the reference's literals."""
    start_id: int = 151644
    end_id: int = 151645
    enter_id: int = 1699
    system: str = "You are a helpful assistant."

    def prompt(self, tokenizer: VocabTokenizer, user_text: str) -> List[int]:
        ids: List[int] = [self.start_id]
        ids += tokenizer.encode("system\n" + self.system)
        ids += [self.end_id, self.enter_id, self.start_id]
        ids += tokenizer.encode("user\n" + user_text)
        ids += [self.end_id, self.enter_id, self.start_id]
        ids += tokenizer.encode("assistant\n")
        return ids


def find_vocab(folder: str):
    """The tokenizer of a model folder, or None if it has no vocab.json."""
    import os
    path = os.path.join(folder, "vocab.json")
    return VocabTokenizer.from_file(path) if os.path.isfile(path) else None
