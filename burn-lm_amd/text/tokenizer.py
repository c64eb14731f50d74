"""Text <-> token ids for the server layer and the command line.

``ByteTokenizer``: a token is a byte value, as the reference's test tokenizer
(crates/burn-lm-llama/src/tokenizer/byte.rs:3-49: bos 0, eos 1, stop ids [2]); it needs a
vocabulary of at least 256.  Where the reference prints the id list on decode (byte.rs:34-36),
this one gives the bytes back as text.  A ``tokenizer.json`` in the model folder is used instead
when the ``tokenizers`` package can read it; which of its special tokens begin and end a text and
which stop a generation is the architecture's knowledge (``registry.Architecture.special_tokens``;
the reference's Llama-3 tokenizer: crates/burn-lm-llama/src/tokenizer/tiktoken.rs:12-15, 126-132),
used as far as the file defines them."""
from __future__ import annotations

import os
from typing import List


class ByteTokenizer:
    bos_id, eos_id = 0, 1

    def encode(self, text: str, bos: bool = False, eos: bool = False) -> List[int]:
        ids = list(text.encode("utf-8"))
        return ([self.bos_id] if bos else []) + ids + ([self.eos_id] if eos else [])

    def decode(self, tokens) -> str:
        return bytes(t for t in tokens if 0 <= t < 256).decode("utf-8", errors="replace")

    def stop_ids(self):
        return [2]


class FileTokenizer:
    def __init__(self, path, special_tokens=None):
        from tokenizers import Tokenizer
        self._tok = Tokenizer.from_file(path)
        sp = special_tokens or {}
        self._stops = tuple(sp.get("stops", ()))
        self.bos_id = self._tok.token_to_id(sp["bos"]) if sp.get("bos") else None
        self.eos_id = self._tok.token_to_id(sp["eos"]) if sp.get("eos") else None

    def encode(self, text, bos=False, eos=False):
        ids = self._tok.encode(text, add_special_tokens=False).ids
        if bos and self.bos_id is not None:
            ids = [self.bos_id] + ids
        if eos and self.eos_id is not None:
            ids = ids + [self.eos_id]
        return ids

    def decode(self, tokens):
        return self._tok.decode(list(tokens), skip_special_tokens=True)

    def stop_ids(self):
        ids = [self._tok.token_to_id(t) for t in self._stops]
        return [i for i in ids if i is not None]


def for_folder(folder: str, vocab_size: int, special_tokens=None):
    """special_tokens: the architecture's names of the tokens that begin, end and stop a text."""
    path = os.path.join(folder, "tokenizer.json")
    if os.path.exists(path):
        try:
            return FileTokenizer(path, special_tokens)
        except Exception as e:  # unreadable file: say so and fall back to bytes
            print(f"warning: {path} could not be read ({e}); using the byte tokenizer")
    if vocab_size < 256:
        raise ValueError(f"the byte tokenizer needs a vocabulary of at least 256, the model has {vocab_size}; "
                         f"pass token ids instead of text")
    return ByteTokenizer()


class StreamingDecoder:
    """Text of a growing list of tokens, piece by piece.  A token decoded on its own can lose what
    it shares with its neighbours (a leading space, the bytes of one character spread over two
    tokens), so a piece is what decoding the last emitted tokens *with* the new ones adds to decoding
    them alone: two tokens of overlap, as the reference does
    (crates/burn-lm-llama/src/generation/streaming.rs:10-57).  A piece that would end in half a
    character is held back until the character is whole."""
    OVERLAP = 2

    def __init__(self, tokenizer):
        self.tokenizer = tokenizer
        self.tokens = []
        self.emitted = 0

    def push(self, token):
        """-> the text this token completes ('' if it has to wait for the next one)."""
        self.tokens.append(token)
        start = max(0, self.emitted - self.OVERLAP)
        whole = self.tokenizer.decode(self.tokens[start:])
        before = self.tokenizer.decode(self.tokens[start:self.emitted])
        if whole.endswith("\ufffd") or not whole.startswith(before):
            return ""
        piece = whole[len(before):]
        if piece:
            self.emitted = len(self.tokens)
        return piece

    def flush(self):
        """What is still held back when the tokens end (half a character comes out as it decodes)."""
        start = max(0, self.emitted - self.OVERLAP)
        whole = self.tokenizer.decode(self.tokens[start:])
        before = self.tokenizer.decode(self.tokens[start:self.emitted])
        self.emitted = len(self.tokens)
        return whole[len(before):] if whole.startswith(before) else ""
