"""Text <-> token ids for the command line: greedy longest match over the vocabulary with
byte fallback, as the reference's tokenizer does (src/tokenizer.cpp:85-149 encode,
:166-197 decode, :65-83 the end-of-turn token by name).  The vocabulary comes from a
``tokenizer.json`` in the model folder (``model.vocab`` and ``added_tokens``).  Requests to the
library itself are token ids; this file only serves ``infer -i / -f``."""
from __future__ import annotations

import json
import os

EOT_NAMES = ("<|eot_id|>", "<|end|>", "<|im_end|>", "<|endoftext|>", "<|end_of_text|>")


class Tokenizer:
    def __init__(self, vocab: dict, bos_id: int | None = None, eos_id: int | None = None):
        self.id_of = {tok.replace("▁", " "): i for tok, i in vocab.items()}
        self.piece = {i: t for t, i in self.id_of.items()}
        self.bos_id, self.eos_id = bos_id, eos_id
        self.byte_start = vocab.get("<0x00>")
        self.eot_id = None
        for name in EOT_NAMES:                       # the last vocabulary entry with such a name
            if name in vocab and (self.eot_id is None or vocab[name] > self.eot_id):
                self.eot_id = vocab[name]
        self.trie = {}
        for tok, i in self.id_of.items():
            node = self.trie
            for b in tok.encode("utf-8"):
                node = node.setdefault(b, {})
            if tok:
                node[-1] = i

    @classmethod
    def from_folder(cls, folder: str, bos_id=None, eos_id=None):
        path = os.path.join(folder, "tokenizer.json")
        if not os.path.isfile(path):
            return None
        with open(path, encoding="utf-8") as f:
            raw = json.load(f)
        vocab = dict(raw.get("model", {}).get("vocab", {}))
        for t in raw.get("added_tokens", []):
            vocab[t["content"]] = t["id"]
        return cls(vocab, bos_id, eos_id)

    @classmethod
    def from_gguf(cls, metadata: dict, bos_id=None, eos_id=None):
        """The vocabulary a GGUF file carries (``tokenizer.ggml.tokens``, src/tokenizer.cpp:13-60)."""
        tokens = metadata.get("tokenizer.ggml.tokens")
        if tokens is None:
            return None
        if bos_id is None and "tokenizer.ggml.bos_token_id" in metadata:
            bos_id = int(metadata["tokenizer.ggml.bos_token_id"])
        if eos_id is None and "tokenizer.ggml.eos_token_id" in metadata:
            eos_id = int(metadata["tokenizer.ggml.eos_token_id"])
        return cls({str(t): i for i, t in enumerate(tokens)}, bos_id, eos_id)

    @classmethod
    def from_model(cls, path: str, bos_id=None, eos_id=None):
        """tokenizer.json of a model folder, else the vocabulary inside its GGUF file."""
        tok = cls.from_folder(path, bos_id, eos_id) if os.path.isdir(path) else None
        if tok is None:
            from .registry import find_gguf
            gguf = find_gguf(path)
            if gguf is not None:
                from .weights.gguf_io import GGUFFile
                tok = cls.from_gguf(GGUFFile(gguf).metadata, bos_id, eos_id)
        return tok

    def encode(self, text: str, add_bos: bool = True) -> list:
        data = text.encode("utf-8")
        out = [self.bos_id] if add_bos and self.bos_id is not None else []
        i = 0
        while i < len(data):
            node, best, best_len = self.trie, None, 0
            for j in range(i, len(data)):
                node = node.get(data[j])
                if node is None:
                    break
                if -1 in node:
                    best, best_len = node[-1], j - i + 1
            if best is not None:
                out.append(best)
                i += best_len
            elif self.byte_start is not None:
                out.append(self.byte_start + data[i])
                i += 1
            else:
                raise ValueError(f"Cannot encode byte 0x{data[i]:02x} and no byte fallback available")
        return out

    def decode_token(self, token: int, prev: int | None = None) -> bytes:
        if self.byte_start is not None and self.byte_start <= token < self.byte_start + 256:
            return bytes([token - self.byte_start])
        piece = self.piece.get(token, "")
        if prev is not None and prev == self.bos_id and piece.startswith(" "):
            piece = piece[1:]
        return piece.encode("utf-8")

    def decode(self, tokens) -> str:
        out, prev = b"", None
        for t in tokens:
            out += self.decode_token(t, prev)
            prev = t
        return out.decode("utf-8", errors="replace")
