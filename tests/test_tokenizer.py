"""Tokenizers: the library (wgml_amd.LlamaTokenizer / Gpt2Tokenizer over
wgml_amd/csrc/tokenizer.cpp) against (1) cases traced by hand on small vocabularies,
(2) the statement-by-statement restatement of the reference in oracle/tokenizers.py
(whose pre-tokenizer is the reference's pattern run by the `regex` module, an
implementation independent of the hand-written scanner in the library), on seeded random
texts, and (3) vocabularies read back from GGUF files.

The reference holds no tokenizer test or golden ids and no real vocabulary exists here:
ids on a real Llama / GPT-2 vocabulary are parity unpinned.
"""
import os
import random
import sys

import numpy as np
import pytest

import wgml_amd as W
from wgml_amd._lib import WgmlError

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "oracle"))
import tokenizers as orc  # noqa: E402

import gguf_writer as gw  # noqa: E402


# ------------------------------------------------------------------ Llama ---
def llama_vocab():
    """<unk>, <s>, </s>, the 256 byte tokens, then characters and pieces with scores."""
    tokens = ["<unk>", "<s>", "</s>"] + [f"<0x{b:02X}>" for b in range(256)]
    scores = [0.0] * len(tokens)
    for ch in "▁helowrd<>/sabcix":
        tokens.append(ch)
        scores.append(-100.0)
    for piece, sc in (("he", -1), ("ll", -2), ("hell", -3), ("hello", -4), ("▁w", -5), ("or", -6),
                      ("ld", -7), ("▁wor", -8), ("▁world", -9), ("ab", -20), ("bc", -20),
                      ("▁hello", -30), (" \tq", -50), ("\u00a0\u3000z", -50)):
        tokens.append(piece)
        scores.append(float(sc))
    return tokens, scores


@pytest.fixture(scope="module")
def llama():
    tokens, scores = llama_vocab()
    return W.LlamaTokenizer(tokens, scores, 1, 2, 0), orc.LlamaTokenizer(tokens, scores, 1, 2, 0), tokens


def test_llama_merge_order_traced_by_hand(llama):
    tok, _, tokens = llama
    ix = {t: i for i, t in enumerate(tokens)}
    # h e l l o ▁ w o r l d
    # -> he(-1) -> ll(-2) -> hell(-3) -> hello(-4) -> ▁w(-5) -> or(-6) -> ld(-7, beats ▁wor -8)
    # -> ▁wor(-8) -> ▁world(-9);  "hello" + "▁world" is no token, so the loop ends
    assert tok.encode("hello world", False, False) == [ix["hello"], ix["▁world"]]
    assert tok.encode("hello world", True, True) == [1, ix["hello"], ix["▁world"], 2]
    # a leading space: ▁ h e l l o -> ... -> ▁ hello -> ▁hello(-30)
    assert tok.encode(" hello", False, False) == [ix["▁hello"]]


def test_llama_equal_scores_leftmost_pair_wins(llama):
    tok, _, tokens = llama
    ix = {t: i for i, t in enumerate(tokens)}
    # "ab" and "bc" score the same: the comparison is strict, so "ab" (found first) merges
    assert tok.encode("abc", False, False) == [ix["ab"], ix["c"]]


def test_llama_byte_fallback_and_specials(llama):
    tok, _, tokens = llama
    ix = {t: i for i, t in enumerate(tokens)}
    # 'é' (C3 A9) is no token: its bytes + 3
    assert tok.encode("é", False, False) == [0xC3 + 3, 0xA9 + 3]
    # "<s>" / "</s>" spelled out with single-character tokens become the special ids
    assert tok.encode("<s>hi", False, False) == [1, ix["h"], ix["i"]]
    assert tok.encode("hi</s>", False, False) == [ix["h"], ix["i"], 2]
    assert tok.bos() == 1 and tok.eos() == 2 and tok.unk() == 0
    assert tok.bos_str() == "<s>" and tok.eos_str() == "</s>" and len(tok) == len(tokens)


def test_llama_decode(llama):
    tok, _, tokens = llama
    ix = {t: i for i, t in enumerate(tokens)}
    assert tok.decode(5, ix["▁world"]) == " world"
    assert tok.decode(1, ix["▁world"]) == " world"  # U+2581 is not white space: nothing trimmed
    assert tok.decode(5, 3 + 0x41) == "A"
    assert tok.decode(5, 3 + 0xE9) == "é"  # the character U+00E9, not the byte
    assert tok.decode(5, ix["<"]) == "<"
    # after <s> (id 1) leading white space goes, of any Unicode kind
    assert tok.decode(1, ix[" \tq"]) == "q" and tok.decode(5, ix[" \tq"]) == " \tq"
    assert tok.decode(1, ix["\u00a0\u3000z"]) == "z"


def test_llama_errors(llama):
    tok, _, _ = llama
    with pytest.raises(WgmlError):
        tok.encode("", False, False)  # the reference panics (tokens.len() - 1 underflows)
    assert tok.encode("", True, False) == [1]
    with pytest.raises(WgmlError):
        tok.decode(0, 10_000)
    small = W.LlamaTokenizer(["<unk>", "<s>", "</s>", "a"], [0, 0, 0, 0], 1, 2, 0)
    with pytest.raises(WgmlError):
        small.encode("b", False, False)  # byte fallback 0x62 + 3 is beyond the 4 tokens


ALPHABET = list("helowrdabcix <>/s") + ["é", "▁", "世", "\n", "\t", "1", "'", "!", "Ω", " ", "😀"]


def test_llama_matches_restatement_on_random_text(llama):
    tok, ref, _ = llama
    rng = random.Random(7)
    for case in range(300):
        text = "".join(rng.choice(ALPHABET) for _ in range(rng.randint(1, 40)))
        for bos, eos in ((False, False), (True, True)):
            assert tok.encode(text, bos, eos) == ref.encode(text, bos, eos), repr(text)
    for prev in (0, 1, 7):
        for t in range(len(tok)):
            assert tok.decode(prev, t) == ref.decode(prev, t), (prev, t)


# ------------------------------------------------------------------ GPT-2 ---
def gpt2_vocab():
    b2u = orc.bytes_to_unicode()
    tokens = [b2u[b] for b in range(256)]
    merges = ["h e", "l l", "he ll", "hell o", "Ġ w", "o r", "Ġw or", "l d", "Ġwor ld", "1 2",
              "Ġ 12", "! !", "' m", "Ġ Ġ", "a b", "ab c", "Ã ©", "Ġ h", "Ġh e"]
    for m in merges:
        a, b = m.split()
        if a + b not in tokens:
            tokens.append(a + b)
    tokens.append("<|endoftext|>")
    return tokens, merges


@pytest.fixture(scope="module")
def gpt2():
    tokens, merges = gpt2_vocab()
    eot = len(tokens) - 1
    return (W.Gpt2Tokenizer(tokens, merges, eot, eot), orc.Gpt2Tokenizer(tokens, merges, eot, eot),
            tokens)


def test_byte_alphabet_known_entries():
    b2u = orc.bytes_to_unicode()
    assert b2u[ord(" ")] == "Ġ" and b2u[ord("\n")] == "Ċ" and b2u[0] == "Ā"
    assert b2u[173] == "Ń" and b2u[ord("A")] == "A" and b2u[255] == "ÿ"
    assert sum(1 for b, c in b2u.items() if ord(c) == b) == 188 and len(set(b2u.values())) == 256


def test_gpt2_merges_traced_by_hand(gpt2):
    tok, _, tokens = gpt2
    ix = {t: i for i, t in enumerate(tokens)}
    # "hello": h e l l o -> he l l o (rank 0) -> he ll o (1) -> hell o (2) -> hello (3)
    # " world": Ġ w o r l d -> Ġw o r l d (4) -> Ġw or l d (5) -> Ġwor l d (6) -> Ġwor ld (7)
    #           -> Ġworld (8)
    assert tok.encode("hello world") == [ix["hello"], ix["Ġworld"]]
    # the pattern splits "I'm 12 ok!!  x" into I | 'm | ␣12 | ␣ok | !! | ␣␣ | x  (no look-ahead in
    # the reference's pattern: both spaces form one piece); merges never cross a split
    assert tok.encode("I'm 12 ok!!  x") == [ix["I"], ix["'m"], ix["Ġ12"], ix["Ġ"], ix["o"], ix["k"],
                                            ix["!!"], ix["ĠĠ"], ix["x"]]
    # a b c -> ab c (rank 14) -> abc (15)
    assert tok.encode("abc") == [ix["abc"]]
    # multi-byte characters go through their bytes: é = C3 A9 -> "Ã" "©" -> merged
    assert tok.encode("é") == [ix["Ã©"]]


def test_gpt2_special_tokens(gpt2):
    tok, _, tokens = gpt2
    ix = {t: i for i, t in enumerate(tokens)}
    eot = ix["<|endoftext|>"]
    assert tok.encode("hello<|endoftext|>hello") == [ix["hello"], eot, ix["hello"]]
    assert tok.encode("<|endoftext|>") == [eot]
    assert tok.encode("a<b") == [ix["a"], ix["<"], ix["b"]]  # no closing '>': ordinary text
    with pytest.raises(WgmlError):
        tok.encode("x<nope>y")  # the reference indexes its map with the match and panics
    assert tok.bos() == eot and tok.eos() == eot and tok.eos_str() == "<|endoftext|>"


def test_gpt2_decode(gpt2):
    tok, ref, tokens = gpt2
    ids = tok.encode("hello world é!")
    assert tok.decode(ids, raw_bytes=True) == "hello world é!".encode()
    # the reference maps every byte to the character of that value: é comes back as "Ã©"
    assert tok.decode(ids) == "hello world Ã©!" == ref.decode(ids)
    assert tok.decode([len(tokens) + 5]) == ""  # unknown ids are skipped


def test_gpt2_matches_restatement_on_random_text(gpt2):
    tok, ref, _ = gpt2
    rng = random.Random(11)
    # letters, numbers (Nd, Nl, No), white space of several kinds, punctuation, marks, symbols
    alphabet = list("helowrdabc12!!'mstvIx  \n\t.,-") + [
        "\u00e9", "\u03a9", "\u044f", "\u4e16", "\u754c", "\u0663", "\u096b", "\u2163", "\u00b2",
        "\u00bd", "\u00a0", "\u2003", "\u3000", "\u0301", "\U0001F600", "\u20ac", "'", "re", "ve",
        "ll", "'d", "_", "\u0085", "\u1680"]
    for case in range(400):
        text = "".join(rng.choice(alphabet) for _ in range(rng.randint(1, 30)))
        assert tok.encode(text) == ref.encode(text), repr(text)
        ids = ref.encode(text)
        assert tok.decode(ids) == ref.decode(ids), repr(text)
        assert tok.decode(ids, raw_bytes=True) == text.encode(), repr(text)


# ------------------------------------------------------------------- GGUF ---
def test_tokenizers_from_gguf(tmp_path, llama, gpt2):
    tokens, scores = llama_vocab()
    path = tmp_path / "llama_tok.gguf"
    gw.write_gguf(path, [
        ("tokenizer.ggml.tokens", gw.ARRAY, (gw.STRING, tokens)),
        ("tokenizer.ggml.scores", gw.ARRAY, (gw.F32, scores)),
        ("tokenizer.ggml.bos_token_id", gw.U32, 1),
        ("tokenizer.ggml.eos_token_id", gw.U32, 2),
        ("tokenizer.ggml.unknown_token_id", gw.U32, 0)], [])
    g = W.Gguf(path)
    tok = W.LlamaTokenizer.from_gguf(g)
    assert tok.encode("hello world", True, False) == llama[0].encode("hello world", True, False)
    assert len(tok) == len(tokens)

    gtokens, merges = gpt2_vocab()
    path = tmp_path / "gpt2_tok.gguf"
    gw.write_gguf(path, [
        ("tokenizer.ggml.tokens", gw.ARRAY, (gw.STRING, gtokens)),
        ("tokenizer.ggml.merges", gw.ARRAY, (gw.STRING, merges)),
        ("tokenizer.ggml.bos_token_id", gw.U32, len(gtokens) - 1),
        ("tokenizer.ggml.eos_token_id", gw.U32, len(gtokens) - 1)], [])
    g2 = W.Gguf(path)
    tok2 = W.Gpt2Tokenizer.from_gguf(g2)
    assert tok2.encode("hello world") == gpt2[0].encode("hello world")
    assert np.array_equal(tok2.encode("I'm 12"), gpt2[0].encode("I'm 12"))


def test_invalid_utf8_does_not_crash(llama, gpt2):
    # raw bytes through the C entry points (the Python classes only ever pass valid UTF-8):
    # malformed sequences are taken byte by byte as U+FFFD, nothing is read past the end
    rng = random.Random(3)
    ltok, gtok = llama[0], gpt2[0]
    for case in range(300):
        raw = bytes(rng.randrange(256) for _ in range(rng.randint(1, 24)))
        ids = ltok._ids("wgml_llama_tokenizer_encode", ltok._h, raw, len(raw), 1, 0)
        assert ids[0] == 1 and all(0 <= t < len(ltok) for t in ids)
        try:
            ids = gtok._ids("wgml_gpt2_tokenizer_encode", gtok._h, raw, len(raw))
            assert all(0 <= t < len(gtok) for t in ids)
        except WgmlError:
            pass  # a "<...>" run that is no token
    for bad in (b"\xe2\x96", b"\xf0\x9f\x98", b"\xc3", b"\xed\xa0\x80", b"\xf4\x90\x80\x80"):
        ids = ltok._ids("wgml_llama_tokenizer_encode", ltok._h, bad, len(bad), 0, 0)
        assert ids  # U+FFFD is no token of the vocabulary: its bytes EF BF BD + 3, per malformed byte
        assert all(t in (0xEF + 3, 0xBF + 3, 0xBD + 3) for t in ids)


def test_llama2_chat_prompt():
    from wgml_amd.tokenizer import llama2_chat_prompt

    one = llama2_chat_prompt([{"role": "user", "content": " Hello  "}])
    assert one == "<s>[INST] Hello [/INST]"
    full = llama2_chat_prompt([{"role": "system", "content": "Be brief.\n"},
                               {"role": "user", "content": "Hi"},
                               {"role": "assistant", "content": "Hello."},
                               {"role": "user", "content": "Bye"}])
    assert full == ("<s>[INST] <<SYS>>\nBe brief.\n<</SYS>>\n\nHi [/INST] Hello. </s>"
                    "<s>[INST] Bye [/INST]")
    with pytest.raises(ValueError):
        llama2_chat_prompt([{"role": "assistant", "content": "x"}])
    with pytest.raises(ValueError):
        llama2_chat_prompt([{"role": "user", "content": "a"}, {"role": "user", "content": "b"}])
    assert llama2_chat_prompt([]) == ""
