"""GPT-2 byte-level BPE tokenizer, host side only.

Mirrors `gpu_host::tokenizer` (crates/core/gpu-host/src/tokenizer.rs:1-62): `Gpt2Tokenizer` with `encode`
(special tokens recognised in the text, as `encode_with_special_tokens` there, tokenizer.rs:47-49), `decode`
(tokenizer.rs:52-56), `vocab_size` (tokenizer.rs:59-61), `GPT2_VOCAB_SIZE`, `ENDOFTEXT_TOKEN_ID` and `TokenizerError`
with its two kinds (tokenizer.rs:15-21).  The reference wraps tiktoken-rs' built-in `r50k_base` table; no vocabulary
ships with this package, so the table is read from files the caller names:

* tiktoken's format, one `base64(token bytes) rank` pair per line (`r50k_base.tiktoken`), or
* GPT-2's original pair `encoder.json` / `vocab.json` (token text in the printable-byte alphabet -> id) and
  `vocab.bpe` / `merges.txt` (used only to check the table: every merge result must be a token).

The algorithm is the published one of r50k_base: the text is cut by GPT-2's pattern, each piece is taken as bytes, and
the adjacent pair of parts whose concatenation has the lowest rank is merged until no concatenation is a token.
"""
import base64
import json
import os

import regex

GPT2_VOCAB_SIZE = 50257
ENDOFTEXT_TOKEN_ID = 50256
ENDOFTEXT = "<|endoftext|>"

# the split pattern of GPT-2 / r50k_base
_PATTERN = r"""'s|'t|'re|'ve|'m|'ll|'d| ?\p{L}+| ?\p{N}+| ?[^\s\p{L}\p{N}]+|\s+(?!\S)|\s+"""


class TokenizerError(Exception):
    """kind: "init" (the table could not be set up) or "decode" (ids that are no tokens, bytes that are no UTF-8)."""

    def __init__(self, kind, message):
        super().__init__(f"tokenizer {kind} error: {message}")
        self.kind = kind


def bytes_to_unicode():
    """GPT-2's printable stand-in for every byte value: the byte order of the first 256 ranks."""
    keep = list(range(ord("!"), ord("~") + 1)) + list(range(0xA1, 0xAC + 1)) + list(range(0xAE, 0xFF + 1))
    chars = keep[:]
    extra = 0
    for b in range(256):
        if b not in keep:
            keep.append(b)
            chars.append(256 + extra)
            extra += 1
    return {b: chr(c) for b, c in zip(keep, chars)}


class Gpt2Tokenizer:
    def __init__(self, ranks, special_tokens=None):
        """ranks: {token bytes: id}; special_tokens: {text: id}, by default <|endoftext|> = the id after the last rank."""
        if not ranks:
            raise TokenizerError("init", "empty vocabulary")
        for b in range(256):
            if bytes([b]) not in ranks:
                raise TokenizerError("init", f"byte {b} is not a token: the vocabulary is not byte-level")
        self._ranks = dict(ranks)
        if len(set(self._ranks.values())) != len(self._ranks):
            raise TokenizerError("init", "two tokens share an id")
        if special_tokens is None:
            special_tokens = {ENDOFTEXT: max(self._ranks.values()) + 1}
        self._special = dict(special_tokens)
        self._by_id = {i: t for t, i in self._ranks.items()}
        for text, i in self._special.items():
            if i in self._by_id:
                raise TokenizerError("init", f"special token {text!r} takes the id of a token")
            self._by_id[i] = text.encode("utf-8")
        self._split = regex.compile(_PATTERN)
        self._special_split = regex.compile("|".join(regex.escape(t) for t in sorted(self._special, key=len, reverse=True))) \
            if self._special else None
        self._cache = {}

    # ---- construction ----
    @classmethod
    def new(cls, path=None):
        """The reference's `Gpt2Tokenizer::new()` (tokenizer.rs:39-43).  `path`, or the environment variable
        AGPU_GPT2_VOCAB: an r50k_base.tiktoken file, or a directory holding one, or holding GPT-2's
        encoder.json/vocab.json and vocab.bpe/merges.txt."""
        path = path or os.environ.get("AGPU_GPT2_VOCAB")
        if not path:
            raise TokenizerError("init", "no vocabulary: pass a path or set AGPU_GPT2_VOCAB (r50k_base.tiktoken, or a "
                                         "directory with encoder.json + vocab.bpe); none ships with this package")
        if os.path.isdir(path):
            for name in ("r50k_base.tiktoken", "gpt2.tiktoken"):
                if os.path.exists(os.path.join(path, name)):
                    return cls.from_tiktoken_file(os.path.join(path, name))
            for vocab, merges in (("encoder.json", "vocab.bpe"), ("vocab.json", "merges.txt")):
                if os.path.exists(os.path.join(path, vocab)):
                    m = os.path.join(path, merges)
                    return cls.from_gpt2_files(os.path.join(path, vocab), m if os.path.exists(m) else None)
            raise TokenizerError("init", f"no vocabulary files in {path}")
        if path.endswith(".json"):
            return cls.from_gpt2_files(path, None)
        return cls.from_tiktoken_file(path)

    @classmethod
    def from_tiktoken_file(cls, path):
        ranks = {}
        try:
            with open(path, "rb") as f:
                for line in f:
                    if not line.strip():
                        continue
                    token, rank = line.split()
                    ranks[base64.b64decode(token)] = int(rank)
        except (OSError, ValueError) as e:
            raise TokenizerError("init", f"{path}: {e}") from e
        return cls(ranks)

    @classmethod
    def from_gpt2_files(cls, vocab_json, merges_txt=None):
        back = {c: b for b, c in bytes_to_unicode().items()}
        try:
            with open(vocab_json, encoding="utf-8") as f:
                vocab = json.load(f)
            ranks, special = {}, {}
            for text, i in vocab.items():
                if text == ENDOFTEXT:
                    special[text] = int(i)
                else:
                    ranks[bytes(back[c] for c in text)] = int(i)
            if merges_txt:
                with open(merges_txt, encoding="utf-8") as f:
                    for line in f:
                        if line.startswith("#version") or not line.strip():
                            continue
                        a, b = line.split()
                        if bytes(back[c] for c in a + b) not in ranks:
                            raise ValueError(f"merge {a!r} {b!r} gives no token of the vocabulary")
        except (OSError, ValueError, KeyError) as e:
            raise TokenizerError("init", f"{vocab_json}: {e}") from e
        return cls(ranks, special or None)

    def save_tiktoken_file(self, path):
        with open(path, "wb") as f:
            for token, rank in sorted(self._ranks.items(), key=lambda kv: kv[1]):
                f.write(base64.b64encode(token) + b" " + str(rank).encode() + b"\n")

    # ---- the reference's three methods ----
    def vocab_size(self):
        return len(self._by_id)

    def encode(self, text):
        """Token ids of `text`; the special tokens' texts are recognised and give their ids (tokenizer.rs:47-49)."""
        out = []
        pos = 0
        if self._special_split is not None:
            for m in self._special_split.finditer(text):
                self._encode_ordinary(text[pos:m.start()], out)
                out.append(self._special[m.group()])
                pos = m.end()
        self._encode_ordinary(text[pos:], out)
        return out

    def decode(self, tokens):
        """The text of `tokens` (tokenizer.rs:52-56): an error for an id that is no token or bytes that are no UTF-8."""
        try:
            data = b"".join(self._by_id[int(t)] for t in tokens)
        except KeyError as e:
            raise TokenizerError("decode", f"no token with id {e.args[0]}") from e
        try:
            return data.decode("utf-8")
        except UnicodeDecodeError as e:
            raise TokenizerError("decode", str(e)) from e

    def decode_bytes(self, tokens):
        try:
            return b"".join(self._by_id[int(t)] for t in tokens)
        except KeyError as e:
            raise TokenizerError("decode", f"no token with id {e.args[0]}") from e

    # ---- byte pair merging ----
    def _encode_ordinary(self, text, out):
        for piece in self._split.findall(text):
            data = piece.encode("utf-8")
            ids = self._cache.get(data)
            if ids is None:
                ids = self._merge(data)
                if len(self._cache) < 65536:
                    self._cache[data] = ids
            out.extend(ids)

    def _merge(self, data):
        ranks = self._ranks
        whole = ranks.get(data)
        if whole is not None:
            return [whole]
        parts = [data[i:i + 1] for i in range(len(data))]
        while len(parts) > 1:
            best, at = None, -1
            for i in range(len(parts) - 1):
                r = ranks.get(parts[i] + parts[i + 1])
                if r is not None and (best is None or r < best):
                    best, at = r, i
            if best is None:
                break
            parts[at:at + 2] = [parts[at] + parts[at + 1]]
        return [ranks[p] for p in parts]
