"""TEST INFRASTRUCTURE ONLY: restatement of the reference's two tokenizers, statement by
statement, in plain Python.  Nothing under wgml_amd/ imports this file; only tests/ may.

    LlamaTokenizer   crates/wgml/src/models/llama2/tokenizer.rs:8-180
    Gpt2Tokenizer    crates/wgml/src/models/gpt2/tokenizer.rs:13-217

How it is pinned: the reference holds no tokenizer test, vocabulary or golden ids, and no
vocabulary file exists in this environment, so the restatement is checked against cases
traced by hand on small vocabularies (tests/test_tokenizer.py: every intermediate merge is
written out there), against the published GPT-2 byte-to-unicode table's known entries
(space -> U+0120, newline -> U+010A, 188 self-mapped bytes), and against the pre-tokenizer
splits the pattern must give by its definition.  Token ids of a real Llama or GPT-2
vocabulary: parity unpinned.

The pre-tokenizer pattern is used as the reference writes it, through the `regex` module
(`re` has no \\p{..} classes); its leftmost-first alternation is the regex crate's too.
"""
from __future__ import annotations

from typing import Dict, List, Sequence, Tuple

import regex

# White_Space, what Rust's char::is_whitespace / str::trim_start use
_WS = set([0x09, 0x0A, 0x0B, 0x0C, 0x0D, 0x20, 0x85, 0xA0, 0x1680, 0x2028, 0x2029, 0x202F, 0x205F,
           0x3000] + list(range(0x2000, 0x200B)))


def _trim_start(s: str) -> str:
    i = 0
    while i < len(s) and ord(s[i]) in _WS:
        i += 1
    return s[i:]


class LlamaTokenizer:
    def __init__(self, tokens: Sequence[str], scores: Sequence[float], bos: int, eos: int, unk: int):
        # from_gguf (tokenizer.rs:23-51)
        self.vocab = list(tokens)
        self.vocab_scores = [float(s) for s in scores]
        self.bos, self.eos, self.unk = bos, eos, unk
        self.vocab_index: Dict[str, int] = {}
        for n, t in enumerate(self.vocab):
            self.vocab_index[t] = n

    def encode(self, text: str, bos: bool, eos: bool) -> List[int]:
        # tokenizer.rs:73-166
        text = text.replace(" ", "▁")
        tokens: List[int] = []
        if bos:
            tokens.append(self.bos)
        for ch in text:
            if ch in self.vocab_index:
                tokens.append(self.vocab_index[ch])
            else:
                for byte in ch.encode("utf-8"):
                    tokens.append(byte + 3)
        i = 0
        while i < max(len(tokens) - 2, 0):
            tok = self.vocab[tokens[i]] + self.vocab[tokens[i + 1]] + self.vocab[tokens[i + 2]]
            if tok == "<s>":
                tokens[i] = self.bos
                del tokens[i + 2]
                del tokens[i + 1]
            i += 1
        i = 0
        while i < max(len(tokens) - 3, 0):
            tok = (self.vocab[tokens[i]] + self.vocab[tokens[i + 1]] + self.vocab[tokens[i + 2]] +
                   self.vocab[tokens[i + 3]])
            if tok == "</s>":
                tokens[i] = self.eos
                del tokens[i + 3]
                del tokens[i + 2]
                del tokens[i + 1]
            i += 1
        if not tokens:
            raise ValueError("tokens.len() - 1 underflows: the reference panics here")
        while True:
            best_score, best_id, best_idx = float("-inf"), 0, None
            for i in range(len(tokens) - 1):
                pair = self.vocab[tokens[i]] + self.vocab[tokens[i + 1]]
                idx = self.vocab_index.get(pair)
                if idx is not None and self.vocab_scores[idx] > best_score:
                    best_score, best_id, best_idx = self.vocab_scores[idx], idx, i
            if best_idx is None:
                break
            tokens[best_idx] = best_id
            del tokens[best_idx + 1]
        if eos:
            tokens.append(self.eos)
        return tokens

    def decode(self, prev_token: int, token: int) -> str:
        # tokenizer.rs:168-180
        piece = self.vocab[token]
        if prev_token == 1:
            piece = _trim_start(piece)
        if piece.startswith("<0x"):
            hex2 = piece[3:5]
            try:
                if len(hex2) == 2:
                    return chr(int(hex2, 16))  # byte_pieces[b] = b as u8 as char
            except ValueError:
                pass
        return piece.replace("▁", " ")


def bytes_to_unicode() -> Dict[int, str]:
    # tokenizer.rs:21-36
    bs = list(range(33, 127)) + list(range(161, 173)) + list(range(174, 256))
    cs = list(bs)
    n = 0
    for b in range(256):
        if b not in bs:
            bs.append(b)
            cs.append(256 + n)
            n += 1
    return {b: chr(c) for b, c in zip(bs, cs)}


class Gpt2Tokenizer:
    PAT = regex.compile(r"'s|'t|'re|'ve|'m|'ll|'d| ?\p{L}+| ?\p{N}+| ?[^\s\p{L}\p{N}]+|\s+")
    SPECIAL = regex.compile(r"<[^<>]*>")

    def __init__(self, tokens: Sequence[str], merges: Sequence[str], bos: int, eos: int):
        # from_gguf (tokenizer.rs:54-95)
        self.bos, self.eos = bos, eos
        self.merges: Dict[Tuple[str, str], int] = {}
        for i, line in enumerate(merges):
            parts = line.split()
            self.merges[(parts[0], parts[1])] = i
        self.byte_encoder = bytes_to_unicode()
        self.byte_decoder = {c: b for b, c in self.byte_encoder.items()}
        self.decoder = {i: t for i, t in enumerate(tokens)}
        self.encoder = {t: i for i, t in enumerate(tokens)}

    def bpe(self, token: str) -> str:
        # tokenizer.rs:168-216
        word = list(token)
        pairs = set(zip(word[:-1], word[1:]))
        if not pairs:
            return token
        while True:
            bigram = min(pairs, key=lambda p: self.merges.get(p, 2**64))
            first, second = bigram
            if bigram not in self.merges:
                break
            new_word: List[str] = []
            i = 0
            while i < len(word):
                try:
                    j = word.index(first, i) - i
                except ValueError:
                    new_word.extend(word[i:])
                    break
                new_word.extend(word[i:i + j])
                i += j
                if i < len(word) - 1 and word[i + 1] == second:
                    new_word.append(first + second)
                    i += 2
                else:
                    new_word.append(word[i])
                    i += 1
            word = new_word
            if len(word) == 1:
                break
            pairs = set(zip(word[:-1], word[1:]))
        return " ".join(word)

    def encode(self, text: str) -> List[int]:
        # tokenizer.rs:105-144
        out: List[int] = []

        def tokenize(substr: str) -> None:
            for m in self.PAT.finditer(substr):
                enc = "".join(self.byte_encoder[b] for b in m.group(0).encode("utf-8"))
                for piece in self.bpe(enc).split(" "):
                    if piece in self.encoder:
                        out.append(self.encoder[piece])

        cursor = 0
        for m in self.SPECIAL.finditer(text):
            if cursor != m.start():
                tokenize(text[cursor:m.start()])
            out.append(self.encoder[m.group(0)])  # KeyError where the reference panics
            cursor = m.end()
        if cursor < len(text):
            tokenize(text[cursor:])
        return out

    def decode(self, tokens: Sequence[int]) -> str:
        # tokenizer.rs:154-166
        text = "".join(self.decoder[t] for t in tokens if t in self.decoder)
        return "".join(chr(self.byte_decoder[c]) for c in text if c in self.byte_decoder)
