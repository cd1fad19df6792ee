"""GGUF reader: the reference's own fixture (assets/gguf/dummy.gguf, written by llama.cpp's
llama-gguf example and loaded by gguf.rs:715-722) with its known contents, an independent
struct-based parser as cross-check, malformed input, and a round trip of a tiny Llama model
through a file.  No GPU needed."""
import os
import struct

import numpy as np
import pytest

import gguf_writer as gw
import wgml_amd as W
from wgml_amd.models import HostMatrix, Llama2Config, synth_llama

HERE = os.path.dirname(os.path.abspath(__file__))
DUMMY = os.path.join(HERE, "golden", "dummy.gguf")

MICRO = Llama2Config(dim=256, hidden_dim=512, n_layers=2, n_q_heads=4, n_kv_heads=2,
                     vocab_size=320, seq_len=32, rope_base_freq=500000.0,
                     rms_norm_eps=float(np.float32(1e-5)))  # the file holds f32 values


def test_dummy_known_contents():
    g = W.Gguf(DUMMY)
    assert g.version == 3 and g.alignment == 32
    md = g.metadata
    assert len(md) == 15
    assert md["some.parameter.uint8"] == 0x12 and md["some.parameter.int8"] == -0x13
    assert md["some.parameter.uint16"] == 0x1234 and md["some.parameter.int16"] == -0x1235
    assert md["some.parameter.uint32"] == 0x12345678 and md["some.parameter.int32"] == -0x12345679
    assert md["some.parameter.uint64"] == 0x123456789abcdef0
    assert md["some.parameter.int64"] == -0x123456789abcdef1
    assert md["some.parameter.float32"] == float(np.float32(0.123456789))
    assert md["some.parameter.float64"] == 0.1234567890123456789
    assert md["some.parameter.bool"] is True
    assert md["some.parameter.string"] == "hello world"
    assert md["some.parameter.arr.i16"].tolist() == [1, 2, 3, 4]
    np.testing.assert_array_equal(md["some.parameter.arr.f32"], np.float32([3.145, 2.718, 1.414]))
    assert md["some.parameter.arr.str"] == ["hello", "world", "!"]
    assert sorted(g.tensors) == [f"tensor_{i}" for i in range(10)]
    for i in range(10):
        t = g.tensors[f"tensor_{i}"]
        assert t.qtype == W.F32
        n = int(np.prod(t.dimensions))
        v = t.as_f32()
        assert v.size == n and np.all(v == 100.0 + i)  # llama-gguf fills tensor i with 100 + i
        assert t.offset % 32 == 0
    assert g.tensors["tensor_0"].dimensions == (7, 8, 6, 4)
    assert g.tensors["tensor_9"].offset - g.tensors["tensor_0"].offset == 8928


def test_dummy_against_independent_parser():
    raw = open(DUMMY, "rb").read()
    version, md, tensors = gw.parse_gguf(raw)
    g = W.Gguf(raw)  # from bytes, like Gguf::from_bytes
    assert g.version == version and set(g.metadata) == set(md) and set(g.tensors) == set(tensors)
    for k, v in md.items():
        got = g.metadata[k]
        if isinstance(v, list) and not isinstance(v[0], str):
            assert got.tolist() == pytest.approx(v)
        elif isinstance(v, float):
            assert got == pytest.approx(v, rel=1e-7)
        else:
            assert got == v
    for name, (ttype, dims, off) in tensors.items():
        t = g.tensors[name]
        assert (t.qtype, list(t.dimensions), t.offset) == (ttype, dims, off)
        n = int(np.prod(dims))
        np.testing.assert_array_equal(t.as_f32(), np.frombuffer(raw, "<f4", n, off))


def test_malformed_input_is_refused(tmp_path):
    raw = bytearray(open(DUMMY, "rb").read())
    with pytest.raises(W.WgmlError, match="magic"):
        W.Gguf(b"GGUX" + bytes(raw[4:]))
    for cut in (3, 12, 40, 200, 1000, 1216 + 100):
        with pytest.raises(W.WgmlError):
            W.Gguf(bytes(raw[:cut]))
    bad = bytearray(raw)
    struct.pack_into("<Q", bad, 8, 1 << 40)  # absurd tensor count
    with pytest.raises(W.WgmlError):
        W.Gguf(bytes(bad))
    # counts that are smaller than the file but larger than its remaining bytes could hold
    # (13 bytes per metadata record, 24 per tensor record at the least)
    for off in (8, 16):
        bad = bytearray(raw)
        struct.pack_into("<Q", bad, off, len(raw) // 2)
        with pytest.raises(W.WgmlError, match="implausible"):
            W.Gguf(bytes(bad))
    # dimensions whose product wraps around 2^64 to a small number must not pass the
    # "lies inside the file" check
    g = W.Gguf(bytes(raw))
    name, t = next((n, t) for n, t in g.tensors.items() if len(t.dimensions) >= 2)
    g.close()
    at = bytes(raw).index(name.encode() + struct.pack("<I", len(t.dimensions)))
    dims_off = at + len(name) + 4
    bad = bytearray(raw)
    struct.pack_into("<QQ", bad, dims_off, 1 << 32, 1 << 32)
    with pytest.raises(W.WgmlError, match="implausible"):
        W.Gguf(bytes(bad))
    with pytest.raises(W.WgmlError, match="cannot open"):
        W.Gguf(str(tmp_path / "missing.gguf"))


def test_alignment_key_and_all_value_types(tmp_path):
    md = [("general.alignment", gw.U32, 64), ("a.u8", gw.U8, 7), ("a.i64", gw.I64, -5),
          ("a.f64", gw.F64, 2.5), ("a.bool", gw.BOOL, 0), ("a.str", gw.STRING, "héllo"),
          ("a.arr", gw.ARRAY, (gw.U32, [1, 2, 3])), ("a.empty", gw.ARRAY, (gw.STRING, []))]
    blocks = W.quantize(W.Q8_0, W.rng_normal(3, 64))
    tensors = [("x", W.Q8_0, [32, 2], blocks.tobytes()), ("y", W.F32, [3], np.float32([1, 2, 3]).tobytes())]
    p = tmp_path / "t.gguf"
    gw.write_gguf(p, md, tensors, alignment=64)
    g = W.Gguf(p)
    assert g.alignment == 64 and g.metadata["a.str"] == "héllo" and g.metadata["a.bool"] is False
    assert g.metadata["a.arr"].tolist() == [1, 2, 3] and g.metadata["a.empty"] == []
    assert g.tensors["x"].offset % 64 == 0 and g.tensors["y"].offset % 64 == 0
    np.testing.assert_array_equal(g.tensors["x"].data, blocks)
    np.testing.assert_array_equal(g.tensors["y"].as_f32(), [1, 2, 3])


@pytest.mark.parametrize("model_type,name", [(0, "llama"), (1, "qwen2")])
def test_llama_round_trip_through_a_file(tmp_path, model_type, name):
    w = synth_llama(MICRO, seed=11, scheme="q4_k_m")
    rng = np.random.default_rng(0)
    if model_type == 1:
        for l in w.layers:
            l["attn_q_bias"] = rng.standard_normal(MICRO.dim).astype(np.float32)
            l["attn_k_bias"] = rng.standard_normal(MICRO.kv_dim).astype(np.float32)
            l["attn_v_bias"] = rng.standard_normal(MICRO.kv_dim).astype(np.float32)
    p = tmp_path / "m.gguf"
    gw.llama_to_gguf(p, w, model_name=name)
    g = W.Gguf(p)
    cfg = W.llama2_config_from_gguf(g, model_type)
    assert cfg == MICRO
    w2 = W.llama2_weights_from_gguf(g, cfg)
    assert len(w2.layers) == MICRO.n_layers
    for a, b in zip(w.layers, w2.layers):
        assert set(a) == set(b)
        for k in a:
            if isinstance(a[k], HostMatrix):
                assert (a[k].qtype, a[k].nrows, a[k].ncols) == (b[k].qtype, b[k].nrows, b[k].ncols)
                np.testing.assert_array_equal(np.asarray(a[k].data).view(np.uint8).reshape(-1),
                                              np.asarray(b[k].data).view(np.uint8).reshape(-1))
            else:
                np.testing.assert_array_equal(a[k], b[k])
    np.testing.assert_array_equal(w.token_embd, w2.token_embd)
    np.testing.assert_array_equal(w.output_norm, w2.output_norm)
    assert w2.weight_bytes_per_token() == w.weight_bytes_per_token()


def test_defaults_and_tied_output(tmp_path):
    # no rope.freq_base / rms epsilon keys -> 10000 and 1e-6; no output.weight -> token_embd;
    # a quantized token_embd is expanded to f32 as the reference does at load
    w = synth_llama(MICRO, seed=12, scheme="q8_0")
    p = tmp_path / "m.gguf"
    raw = gw.llama_to_gguf(p, w, token_embd_type=W.Q8_0)
    version, md, tensors = gw.parse_gguf(raw)
    keep_md = [(k, gw.U32 if isinstance(v, int) else gw.STRING, v) for k, v in md.items()
               if not isinstance(v, (float, list))]
    keep_md.append(("tokenizer.ggml.tokens", gw.ARRAY, (gw.STRING, md["tokenizer.ggml.tokens"])))
    g0 = W.Gguf(p)
    tl = [(n, t.qtype, [d for d in t.dimensions[:2]] if t.dimensions[1] > 1 else [t.dimensions[0]],
           t.data.tobytes()) for n, t in g0.tensors.items() if n != "output.weight"]
    p2 = tmp_path / "tied.gguf"
    gw.write_gguf(p2, keep_md, tl)
    g = W.Gguf(p2)
    cfg = W.llama2_config_from_gguf(g)
    assert cfg.rope_base_freq == 10000.0 and cfg.rms_norm_eps == 1.0e-6
    w2 = W.llama2_weights_from_gguf(g, cfg)
    assert w2.output.qtype == W.Q8_0 and (w2.output.nrows, w2.output.ncols) == (MICRO.vocab_size, MICRO.dim)
    q = W.quantize(W.Q8_0, np.ascontiguousarray(w.token_embd, np.float32).reshape(-1))
    np.testing.assert_array_equal(np.asarray(w2.output.data).reshape(-1), q)
    import oracle as orc
    np.testing.assert_array_equal(w2.token_embd.reshape(-1), orc.dequantize(W.Q8_0, q, q.size // 34 * 32))


def test_gpt2_round_trip_through_a_file(tmp_path):
    # Gpt2Params::from_gguf / Gpt2Weights::from_gguf key and tensor names
    from wgml_amd.models import Gpt2Params, synth_gpt2

    p = Gpt2Params(n_vocab=320, n_seq=32, n_embd=64, n_head=4, n_layer=2, ff_len=256, attn_b=192)
    w = synth_gpt2(p, seed=21)
    rng = np.random.default_rng(1)
    for l in w.layers:
        l["ln_1_b"] = rng.standard_normal(p.n_embd).astype(np.float32)
        l["ln_2_g"] = rng.standard_normal(p.n_embd).astype(np.float32)
    w.ln_f_b = rng.standard_normal(p.n_embd).astype(np.float32)
    path = tmp_path / "gpt2.gguf"
    gw.gpt2_to_gguf(path, w)
    g = W.Gguf(path)
    p2 = W.gpt2_params_from_gguf(g)
    assert p2 == p
    w2 = W.gpt2_weights_from_gguf(g, p2)
    assert len(w2.layers) == p.n_layer
    for a, b in zip(w.layers, w2.layers):
        assert set(a) == set(b)
        for k in a:
            if isinstance(a[k], HostMatrix):
                assert (a[k].qtype, a[k].nrows, a[k].ncols) == (b[k].qtype, b[k].nrows, b[k].ncols)
                np.testing.assert_array_equal(np.asarray(a[k].data).view(np.uint8).reshape(-1),
                                              np.asarray(b[k].data).view(np.uint8).reshape(-1))
            else:
                np.testing.assert_array_equal(a[k], b[k])
    np.testing.assert_array_equal(w.wte, w2.wte)
    np.testing.assert_array_equal(w.wpe, w2.wpe)
    np.testing.assert_array_equal(w.ln_f_g, w2.ln_f_g)
    np.testing.assert_array_equal(w.ln_f_b, w2.ln_f_b)
    # lm_head is the token_embd tensor (tied): f32 here, one row per token
    assert (w2.lm_head.qtype, w2.lm_head.nrows, w2.lm_head.ncols) == (W.F32, p.n_vocab, p.n_embd)
    np.testing.assert_array_equal(np.asarray(w2.lm_head.data).view(np.float32).reshape(p.n_vocab, -1),
                                  w.wte)

    # quantized embeddings are expanded for the look-ups and kept quantized for lm_head
    path = tmp_path / "gpt2_q8.gguf"
    gw.gpt2_to_gguf(path, w, embd_type=W.Q8_0)
    g = W.Gguf(path)
    w3 = W.gpt2_weights_from_gguf(g, W.gpt2_params_from_gguf(g))
    q = W.quantize(W.Q8_0, np.ascontiguousarray(w.wte, np.float32).reshape(-1))
    np.testing.assert_array_equal(np.asarray(w3.lm_head.data).reshape(-1), q)
    np.testing.assert_array_equal(w3.wte.reshape(-1), W.dequantize_host(W.Q8_0, q, w.wte.size))
    with pytest.raises(KeyError):
        W.gpt2_params_from_gguf(W.Gguf(DUMMY))


def test_mutated_files_never_crash_the_reader():
    # seeded byte flips, length-field overwrites and truncations of the fixture: the reader
    # either parses the result or reports an error (the reference panics on several of these,
    # gguf.rs:248-294); it must not read outside the buffer
    raw = open(DUMMY, "rb").read()
    rng = np.random.default_rng(1234)
    header_len = 1216  # metadata + tensor infos of the fixture end here
    parsed = refused = 0
    for case in range(600):
        b = bytearray(raw)
        kind = case % 3
        if kind == 0:  # flip a few bytes in the header region
            for _ in range(int(rng.integers(1, 4))):
                b[int(rng.integers(0, header_len))] = int(rng.integers(0, 256))
        elif kind == 1:  # overwrite an aligned 8-byte field with a huge or odd value
            off = int(rng.integers(1, header_len // 8)) * 8
            vals = [0, 1, 7, 1 << 31, (1 << 63) - 1, (1 << 64) - 1]
            struct.pack_into("<Q", b, off, vals[int(rng.integers(0, len(vals)))])
        else:  # truncate
            b = b[:int(rng.integers(0, len(raw)))]
        try:
            g = W.Gguf(bytes(b))
            for t in g.tensors.values():  # every view must be readable
                if t.data.size:
                    int(t.data[0]) + int(t.data[-1])
            for v in g.metadata.values():
                repr(v)[:10]
            g.close()
            parsed += 1
        except W.WgmlError:
            refused += 1
    assert parsed + refused == 600 and refused > 100
