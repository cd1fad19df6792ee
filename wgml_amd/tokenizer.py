"""Tokenizers with the reference's names and methods: `LlamaTokenizer`
(models/llama2/tokenizer.rs:8-180) and `Gpt2Tokenizer` (models/gpt2/tokenizer.rs:38-217),
over the library's host implementation."""
from __future__ import annotations

import ctypes as C
from typing import Iterable, List, Sequence

import numpy as np

from . import _lib
from ._lib import call


def _pack(strings: Sequence[str]):
    """One block of UTF-8 bytes + n + 1 offsets."""
    raw = [s.encode("utf-8") for s in strings]
    offsets = np.zeros(len(raw) + 1, np.uint64)
    np.cumsum([len(r) for r in raw], out=offsets[1:])
    return b"".join(raw), offsets


class _Tokenizer:
    _h = None

    def __del__(self):
        try:
            if self._h:
                _lib.lib.wgml_tokenizer_destroy(self._h)
                self._h = None
        except Exception:
            pass

    def __len__(self) -> int:
        return call("wgml_tokenizer_vocab_size", self._h)

    def eos(self) -> int:
        return call("wgml_tokenizer_eos", self._h)

    def bos(self) -> int:
        return call("wgml_tokenizer_bos", self._h)

    def token_bytes(self, token: int) -> bytes:
        s, n = C.c_char_p(), C.c_uint64()
        call("wgml_tokenizer_token", self._h, int(token), C.byref(s), C.byref(n))
        return C.string_at(s, n.value)

    def bos_str(self) -> str:
        return self.token_bytes(self.bos()).decode("utf-8", "replace")

    def eos_str(self) -> str:
        return self.token_bytes(self.eos()).decode("utf-8", "replace")

    def _ids(self, name: str, *args) -> List[int]:
        n = C.c_uint64()
        call(name, *args, None, 0, C.byref(n))
        out = np.empty(n.value, np.uint32)
        if n.value:
            call(name, *args, out.ctypes.data_as(C.c_void_p), n.value, C.byref(n))
        return [int(t) for t in out]

    def _text(self, name: str, *args) -> bytes:
        n = C.c_uint64()
        call(name, *args, None, 0, C.byref(n))
        buf = C.create_string_buffer(max(1, n.value))
        if n.value:
            call(name, *args, buf, n.value, C.byref(n))
        return buf.raw[:n.value]


class LlamaTokenizer(_Tokenizer):
    def __init__(self, tokens: Sequence[str], scores: Iterable[float], bos: int, eos: int, unk: int):
        blob, offsets = _pack(tokens)
        sc = np.ascontiguousarray(np.asarray(scores, np.float32))
        if sc.size != len(tokens):
            raise ValueError(f"{sc.size} scores for {len(tokens)} tokens")
        h = C.c_void_p()
        call("wgml_llama_tokenizer_create", blob, offsets.ctypes.data_as(C.c_void_p), len(tokens),
             sc.ctypes.data_as(C.c_void_p), bos, eos, unk, C.byref(h))
        self._h = h

    @classmethod
    def from_gguf(cls, gguf) -> "LlamaTokenizer":
        md = gguf.metadata
        return cls(md["tokenizer.ggml.tokens"], md["tokenizer.ggml.scores"],
                   int(md["tokenizer.ggml.bos_token_id"]), int(md["tokenizer.ggml.eos_token_id"]),
                   int(md["tokenizer.ggml.unknown_token_id"]))

    def unk(self) -> int:
        return call("wgml_tokenizer_unk", self._h)

    def encode(self, text: str, bos: bool, eos: bool) -> List[int]:
        raw = text.encode("utf-8")
        return self._ids("wgml_llama_tokenizer_encode", self._h, raw, len(raw), int(bos), int(eos))

    def decode(self, prev_token: int, token: int) -> str:
        return self._text("wgml_llama_tokenizer_decode", self._h, int(prev_token),
                          int(token)).decode("utf-8", "replace")


def llama2_chat_prompt(messages: Sequence[dict], bos_token: str = "<s>", eos_token: str = "</s>") -> str:
    """The Llama-2 chat prompt for a list of {"role", "content"} messages, as the reference's
    default template for this model produces it (`LlamaTokenizer::CHAT_TEMPLATE`,
    models/llama2/tokenizer.rs:19 with llama-2-chat.jinja): an optional leading system message
    is wrapped in <<SYS>> markers and prepended to the first user message; user turns become
    `bos [INST] content [/INST]`, assistant turns ` content eos`; contents are stripped of
    surrounding whitespace; roles must alternate user / assistant.  (Only the text the template's
    branches emit is produced: the line breaks and indentation between its blocks, which depend
    on the template engine's whitespace settings, are not.  `wgml_amd.ChatTemplate` renders that
    template, or any other, whitespace included.)"""
    msgs = list(messages)
    system = ""
    if msgs and msgs[0]["role"] == "system":
        system = "<<SYS>>\n" + msgs[0]["content"].strip() + "\n<</SYS>>\n\n"
        msgs = msgs[1:]
    out = []
    for i, m in enumerate(msgs):
        if (m["role"] == "user") != (i % 2 == 0):
            raise ValueError("Conversation roles must alternate user/assistant/user/assistant/...")
        content = (system + m["content"] if i == 0 else m["content"]).strip()
        if m["role"] == "user":
            out.append(bos_token + "[INST] " + content + " [/INST]")
        elif m["role"] == "assistant":
            out.append(" " + content + " " + eos_token)
    return "".join(out)


class Gpt2Tokenizer(_Tokenizer):
    def __init__(self, tokens: Sequence[str], merges: Sequence[str], bos: int, eos: int):
        blob, offsets = _pack(tokens)
        mblob, moffsets = _pack(merges)
        h = C.c_void_p()
        call("wgml_gpt2_tokenizer_create", blob, offsets.ctypes.data_as(C.c_void_p), len(tokens),
             mblob, moffsets.ctypes.data_as(C.c_void_p), len(merges), bos, eos, C.byref(h))
        self._h = h

    @classmethod
    def from_gguf(cls, gguf) -> "Gpt2Tokenizer":
        md = gguf.metadata
        return cls(md["tokenizer.ggml.tokens"], md["tokenizer.ggml.merges"],
                   int(md["tokenizer.ggml.bos_token_id"]), int(md["tokenizer.ggml.eos_token_id"]))

    def encode(self, text: str) -> List[int]:
        raw = text.encode("utf-8")
        return self._ids("wgml_gpt2_tokenizer_encode", self._h, raw, len(raw))

    def decode(self, tokens: Sequence[int], raw_bytes: bool = False):
        """The reference's decode (every byte becomes the character of that value); with
        `raw_bytes` the decoded bytes themselves."""
        arr = np.ascontiguousarray(np.asarray(tokens, np.uint32))
        out = self._text("wgml_gpt2_tokenizer_decode", self._h, arr.ctypes.data_as(C.c_void_p),
                         arr.size, int(raw_bytes))
        return out if raw_bytes else out.decode("utf-8", "replace")
