"""Test helper: writes GGUF v3 files (the container layout the reader in
wgml_amd/csrc/gguf.cpp parses; the reference has no writer) and re-parses them with
nothing but `struct`, as an independent check of the C++ reader."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B",
        U64: "<Q", I64: "<q", F64: "<d"}


def _s(text: str) -> bytes:
    b = text.encode()
    return struct.pack("<Q", len(b)) + b


def _value(vtype, v) -> bytes:
    if vtype == STRING:
        return _s(v)
    if vtype == ARRAY:
        etype, items = v
        out = struct.pack("<IQ", etype, len(items))
        for it in items:
            out += _value(etype, it)
        return out
    return struct.pack(_FMT[vtype], v)


def write_gguf(path, metadata, tensors, alignment=32):
    """metadata: list of (key, type, value) (arrays: value = (elem_type, list));
    tensors: list of (name, ggml_type, dims (GGML order: dims[0] contiguous), bytes-like)."""
    out = struct.pack("<IIQQ", 0x46554747, 3, len(tensors), len(metadata))
    for key, vtype, v in metadata:
        out += _s(key) + struct.pack("<I", vtype) + _value(vtype, v)
    offs, off = [], 0
    for _, _, _, data in tensors:
        offs.append(off)
        off += len(bytes(data))
        off += (-off) % alignment
    for (name, ttype, dims, _), o in zip(tensors, offs):
        out += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", ttype, o)
    out += b"\0" * ((-len(out)) % alignment)
    for (_, _, _, data), o in zip(tensors, offs):
        b = bytes(data)
        out += b + b"\0" * ((-len(b)) % alignment)
    with open(path, "wb") as f:
        f.write(out)
    return out


def parse_gguf(raw: bytes):
    """Independent restatement of the container layout: returns (version, metadata dict,
    tensors dict name -> (type, dims, absolute offset))."""
    pos = 0

    def rd(fmt):
        nonlocal pos
        v = struct.unpack_from(fmt, raw, pos)
        pos += struct.calcsize(fmt)
        return v[0] if len(v) == 1 else v

    def rs():
        nonlocal pos
        n = rd("<Q")
        s = raw[pos:pos + n].decode()
        pos += n
        return s

    def rv(t):
        if t == STRING:
            return rs()
        if t == ARRAY:
            et, n = rd("<I"), rd("<Q")
            return [rv(et) for _ in range(n)]
        v = rd(_FMT[t])
        return bool(v) if t == BOOL else v

    magic, version, nt, nm = rd("<I"), rd("<I"), rd("<Q"), rd("<Q")
    assert magic == 0x46554747
    md = {}
    for _ in range(nm):
        k = rs()
        md[k] = rv(rd("<I"))
    infos = []
    for _ in range(nt):
        name = rs()
        nd = rd("<I")
        dims = [rd("<Q") for _ in range(nd)]
        ttype, off = rd("<I"), rd("<Q")
        infos.append((name, ttype, dims, off))
    align = md.get("general.alignment", 32)
    start = pos + (-pos) % align
    return version, md, {n: (t, d + [1] * (4 - len(d)), start + o) for n, t, d, o in infos}


def llama_to_gguf(path, weights, model_name="llama", token_embd_type=0):
    """Writes LlamaHostWeights under the tensor and key names Llama2Weights::from_gguf and
    Llama2Config::from_gguf read (models/llama2/transformer.rs:161-172,235-237;
    models/llama2/cpu.rs:79-109)."""
    c = weights.config
    md = [("general.architecture", STRING, model_name),
          (f"{model_name}.embedding_length", U32, c.dim),
          (f"{model_name}.feed_forward_length", U32, c.hidden_dim),
          (f"{model_name}.block_count", U32, c.n_layers),
          (f"{model_name}.attention.head_count", U32, c.n_q_heads),
          (f"{model_name}.attention.head_count_kv", U32, c.n_kv_heads),
          (f"{model_name}.context_length", U32, c.seq_len),
          (f"{model_name}.rope.freq_base", F32, c.rope_base_freq),
          (f"{model_name}.attention.layer_norm_rms_epsilon", F32, c.rms_norm_eps),
          ("tokenizer.ggml.tokens", ARRAY, (STRING, [f"t{i}" for i in range(c.vocab_size)]))]
    tensors = []
    for l, layer in enumerate(weights.layers):
        for name, v in layer.items():
            if hasattr(v, "qtype"):
                tensors.append((f"blk.{l}.{name}.weight", v.qtype, [v.ncols, v.nrows],
                                np.ascontiguousarray(v.data).tobytes()))
            elif name.endswith("_bias"):
                tensors.append((f"blk.{l}.{name[:-5]}.bias", 0, [v.size], v.astype("<f4").tobytes()))
            else:
                tensors.append((f"blk.{l}.{name}.weight", 0, [v.size], v.astype("<f4").tobytes()))
    te = np.ascontiguousarray(weights.token_embd, dtype=np.float32)
    if token_embd_type == 0:
        tensors.append(("token_embd.weight", 0, [c.dim, c.vocab_size], te.tobytes()))
    else:
        import wgml_amd as W
        tensors.append(("token_embd.weight", token_embd_type, [c.dim, c.vocab_size],
                        W.quantize(token_embd_type, te.reshape(-1)).tobytes()))
    o = weights.output
    tensors.append(("output.weight", o.qtype, [o.ncols, o.nrows], np.ascontiguousarray(o.data).tobytes()))
    tensors.append(("output_norm.weight", 0, [weights.output_norm.size],
                    weights.output_norm.astype("<f4").tobytes()))
    return write_gguf(path, md, tensors)


def gpt2_to_gguf(path, weights, embd_type=0):
    """Writes Gpt2HostWeights under the tensor and key names Gpt2Weights::from_gguf and
    Gpt2Params::from_gguf read (models/gpt2/transformer.rs:115-127,179-188;
    models/gpt2/cpu.rs:34-47).  `embd_type`: GGUF type of token_embd / position_embd."""
    import wgml_amd as W

    p = weights.params
    md = [("general.architecture", STRING, "gpt2"), ("general.file_type", U32, 1),
          ("gpt2.context_length", U32, p.n_seq), ("gpt2.embedding_length", U32, p.n_embd),
          ("gpt2.attention.head_count", U32, p.n_head), ("gpt2.block_count", U32, p.n_layer),
          ("gpt2.feed_forward_length", U32, p.ff_len),
          ("tokenizer.ggml.tokens", ARRAY, (STRING, [f"t{i}" for i in range(p.n_vocab)]))]
    names = {"attn_w": "attn_qkv.weight", "attn_b": "attn_qkv.bias",
             "attn_proj_w": "attn_output.weight", "attn_proj_b": "attn_output.bias",
             "mlp_fc_w": "ffn_up.weight", "mlp_fc_b": "ffn_up.bias",
             "mlp_proj_w": "ffn_down.weight", "mlp_proj_b": "ffn_down.bias",
             "ln_1_g": "attn_norm.weight", "ln_1_b": "attn_norm.bias",
             "ln_2_g": "ffn_norm.weight", "ln_2_b": "ffn_norm.bias"}
    tensors = []
    for l, layer in enumerate(weights.layers):
        for name, v in layer.items():
            if hasattr(v, "qtype"):
                tensors.append((f"blk.{l}.{names[name]}", v.qtype, [v.ncols, v.nrows],
                                np.ascontiguousarray(v.data).tobytes()))
            else:
                tensors.append((f"blk.{l}.{names[name]}", 0, [v.size], v.astype("<f4").tobytes()))

    def embd(name, a):
        a = np.ascontiguousarray(a, dtype=np.float32)
        raw = a.tobytes() if embd_type == 0 else W.quantize(embd_type, a.reshape(-1)).tobytes()
        tensors.append((name, embd_type, [a.shape[1], a.shape[0]], raw))

    embd("token_embd.weight", weights.wte)
    embd("position_embd.weight", weights.wpe)
    tensors.append(("output_norm.weight", 0, [p.n_embd], weights.ln_f_g.astype("<f4").tobytes()))
    tensors.append(("output_norm.bias", 0, [p.n_embd], weights.ln_f_b.astype("<f4").tobytes()))
    return write_gguf(path, md, tensors)
