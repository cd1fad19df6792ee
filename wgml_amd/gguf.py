"""GGUF files: `Gguf` of the reference (gguf.rs:315-607) over the library's reader, and
the loaders that build models from one (models/llama2/cpu.rs:75-109,
models/llama2/transformer.rs:137-268)."""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass
from typing import Dict, Tuple, Union

import numpy as np

from . import _lib
from ._lib import GgufKv, GgufTensorInfo, call

# metadata value type -> numpy dtype (gguf.rs:330-361)
_SCALAR = {0: np.uint8, 1: np.int8, 2: np.uint16, 3: np.int16, 4: np.uint32, 5: np.int32,
           6: np.float32, 7: np.bool_, 10: np.uint64, 11: np.int64, 12: np.float64}
_STRING, _ARRAY = 8, 9


@dataclass
class GgufTensor:
    """GgufTensor (gguf.rs:288-305): dims in GGML order (dims[0] contiguous)."""
    name: str
    qtype: int
    dimensions: Tuple[int, int, int, int]
    offset: int
    data: np.ndarray  # uint8 view of the tensor's bytes inside the file mapping

    def as_f32(self) -> np.ndarray:
        """GgufTensorData::as_f32 (gguf.rs:105-110)."""
        if self.qtype != _lib.F32:
            raise ValueError(f"tensor '{self.name}' is not F32 (type {self.qtype})")
        return self.data.view(np.float32)


class Gguf:
    """Gguf::from_bytes: `version`, `metadata` (key -> value), `tensors` (name -> GgufTensor).
    Tensor data are views of the memory-mapped file: keep this object alive while they are used."""

    def __init__(self, source: Union[str, os.PathLike, bytes, bytearray, memoryview]):
        h = C.c_void_p()
        if isinstance(source, (str, os.PathLike)):
            call("wgml_gguf_open", os.fspath(source).encode(), C.byref(h))
            self._keep = None
        else:
            self._keep = np.frombuffer(bytes(source), dtype=np.uint8)
            call("wgml_gguf_open_bytes", self._keep.ctypes.data_as(C.c_void_p), self._keep.size,
                 C.byref(h))
        self._h = h
        self.version = _lib.lib.wgml_gguf_version(h)
        self.alignment = _lib.lib.wgml_gguf_alignment(h)
        self.metadata: Dict[str, object] = {}
        self.tensors: Dict[str, GgufTensor] = {}
        kv = GgufKv()
        for i in range(_lib.lib.wgml_gguf_n_metadata(h)):
            call("wgml_gguf_metadata", h, i, C.byref(kv))
            self.metadata[kv.key.decode("utf-8", "replace")] = self._value(i, kv)
        ti = GgufTensorInfo()
        for i in range(_lib.lib.wgml_gguf_n_tensors(h)):
            call("wgml_gguf_tensor", h, i, C.byref(ti))
            name = ti.name.decode("utf-8", "replace")
            data = (np.ctypeslib.as_array(C.cast(ti.data, C.POINTER(C.c_uint8)), shape=(ti.nbytes,))
                    if ti.nbytes else np.empty(0, np.uint8))
            self.tensors[name] = GgufTensor(name, ti.type, tuple(int(d) for d in ti.dims),
                                            int(ti.offset), data)

    def _value(self, i: int, kv: GgufKv):
        def raw(n):
            return C.string_at(kv.data, n) if n else b""

        if kv.type == _STRING:
            return raw(kv.nbytes).decode("utf-8", "replace")
        if kv.type == _ARRAY:
            if kv.array_type == _STRING:
                out, s, n = [], C.c_char_p(), C.c_uint64()
                for k in range(kv.array_len):
                    call("wgml_gguf_metadata_string", self._h, i, k, C.byref(s), C.byref(n))
                    out.append(C.string_at(s, n.value).decode("utf-8", "replace"))
                return out
            return np.frombuffer(raw(kv.nbytes), dtype=_SCALAR[kv.array_type]).copy()
        return np.frombuffer(raw(kv.nbytes), dtype=_SCALAR[kv.type])[0].item()

    def close(self) -> None:
        if self._h:
            self.tensors.clear()
            call("wgml_gguf_close", self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def llama2_config_from_gguf(gguf: Gguf, model_type: int = 0):
    """Llama2Config::from_gguf_with_model_type (models/llama2/cpu.rs:79-109)."""
    from .models import Llama2Config

    name = "qwen2" if model_type == 1 else "llama"  # LlamaModelType::gguf_model_name
    md = gguf.metadata
    return Llama2Config(
        dim=int(md[f"{name}.embedding_length"]),
        hidden_dim=int(md[f"{name}.feed_forward_length"]),
        n_layers=int(md[f"{name}.block_count"]),
        n_q_heads=int(md[f"{name}.attention.head_count"]),
        n_kv_heads=int(md[f"{name}.attention.head_count_kv"]),
        vocab_size=len(md["tokenizer.ggml.tokens"]),
        seq_len=int(md[f"{name}.context_length"]),
        rope_base_freq=float(md.get(f"{name}.rope.freq_base", 10000.0)),
        rms_norm_eps=float(md.get(f"{name}.attention.layer_norm_rms_epsilon", 1.0e-6)))


def llama2_weights_from_gguf(gguf: Gguf, config):
    """Llama2Weights::from_gguf (models/llama2/transformer.rs:137-268) as host weights: the
    matrices keep their GGUF quantization, token_embd is expanded to f32 (as the reference
    does), `output` falls back to token_embd when the file ties them."""
    from . import ops
    from .models import HostMatrix, LlamaHostWeights

    c = config
    shapes = {"attn_q": (c.dim, c.dim), "attn_k": (c.kv_dim, c.dim), "attn_v": (c.kv_dim, c.dim),
              "attn_output": (c.dim, c.dim), "ffn_down": (c.dim, c.hidden_dim),
              "ffn_gate": (c.hidden_dim, c.dim), "ffn_up": (c.hidden_dim, c.dim)}

    def matrix(tname: str, nrows: int, ncols: int) -> HostMatrix:
        t = gguf.tensors[tname]
        if t.dimensions[0] != ncols or t.dimensions[1] != nrows:
            raise ValueError(f"tensor '{tname}' is {t.dimensions[1]}x{t.dimensions[0]}, "
                             f"expected {nrows}x{ncols}")
        return HostMatrix(t.qtype, nrows, ncols, t.data)

    w = LlamaHostWeights(config=c)
    for l in range(c.n_layers):
        layer: Dict[str, object] = {}
        for name, (nr, nc) in shapes.items():
            layer[name] = matrix(f"blk.{l}.{name}.weight", nr, nc)
        for name in ("attn_norm", "ffn_norm"):
            layer[name] = gguf.tensors[f"blk.{l}.{name}.weight"].as_f32().copy()
        for name in ("attn_q", "attn_k", "attn_v"):
            t = gguf.tensors.get(f"blk.{l}.{name}.bias")
            if t is not None:
                layer[f"{name}_bias"] = t.as_f32().copy()
        w.layers.append(layer)
    te = gguf.tensors["token_embd.weight"]
    w.token_embd = ops.dequantize_host(te.qtype, te.data, c.vocab_size * c.dim).reshape(
        c.vocab_size, c.dim)
    out = gguf.tensors.get("output.weight", te)
    w.output = HostMatrix(out.qtype, c.vocab_size, c.dim, out.data)
    w.output_norm = gguf.tensors["output_norm.weight"].as_f32().copy()
    return w


# reference tensor name -> host weight name (models/gpt2/transformer.rs:115-127)
_GPT2_MATS = {"attn_qkv": "attn_w", "attn_output": "attn_proj_w", "ffn_up": "mlp_fc_w",
              "ffn_down": "mlp_proj_w"}
_GPT2_BIAS = {"attn_qkv": "attn_b", "attn_output": "attn_proj_b", "ffn_up": "mlp_fc_b",
              "ffn_down": "mlp_proj_b"}
_GPT2_NORMS = {"attn_norm": "ln_1", "ffn_norm": "ln_2"}


def gpt2_params_from_gguf(gguf: Gguf):
    """Gpt2Params::from_gguf (models/gpt2/cpu.rs:34-47)."""
    from .models import Gpt2Params

    md = gguf.metadata
    return Gpt2Params(n_vocab=len(md["tokenizer.ggml.tokens"]),
                      n_seq=int(md["gpt2.context_length"]),
                      n_embd=int(md["gpt2.embedding_length"]),
                      n_head=int(md["gpt2.attention.head_count"]),
                      n_layer=int(md["gpt2.block_count"]),
                      ff_len=int(md["gpt2.feed_forward_length"]),
                      attn_b=int(gguf.tensors["blk.0.attn_qkv.bias"].dimensions[0]))


def gpt2_weights_from_gguf(gguf: Gguf, params):
    """Gpt2Weights::from_gguf (models/gpt2/transformer.rs:108-205) as host weights.  The
    reference expands every matrix to f32; here a matrix keeps its GGUF quantization where the
    GEMV reads it directly, the values are the same.  wte and wpe are expanded to f32 (they
    are looked up, not multiplied); lm_head is the token_embd tensor itself (GPT-2 ties them)."""
    from . import ops
    from .models import Gpt2HostWeights, HostMatrix

    p = params

    def matrix(tname: str, nrows: int, ncols: int) -> HostMatrix:
        t = gguf.tensors[tname]
        if t.dimensions[0] != ncols or t.dimensions[1] != nrows:
            raise ValueError(f"tensor '{tname}' is {t.dimensions[1]}x{t.dimensions[0]}, "
                             f"expected {nrows}x{ncols}")
        return HostMatrix(t.qtype, nrows, ncols, t.data)

    def f32(tname: str, n: int) -> np.ndarray:
        a = gguf.tensors[tname].as_f32()
        if a.size != n:
            raise ValueError(f"tensor '{tname}' has {a.size} elements, expected {n}")
        return a.copy()

    def expanded(tname: str, nrows: int, ncols: int) -> np.ndarray:
        m = matrix(tname, nrows, ncols)
        if m.qtype == _lib.F32:
            return np.asarray(m.data).view(np.float32).reshape(nrows, ncols).copy()
        return ops.dequantize_host(m.qtype, m.data, nrows * ncols).reshape(nrows, ncols)

    shapes = {"attn_qkv": (p.attn_b, p.n_embd), "attn_output": (p.n_embd, p.n_embd),
              "ffn_up": (p.ff_len, p.n_embd), "ffn_down": (p.n_embd, p.ff_len)}
    w = Gpt2HostWeights(params=p)
    for l in range(p.n_layer):
        layer: Dict[str, object] = {}
        for tname, (nr, nc) in shapes.items():
            layer[_GPT2_MATS[tname]] = matrix(f"blk.{l}.{tname}.weight", nr, nc)
            layer[_GPT2_BIAS[tname]] = f32(f"blk.{l}.{tname}.bias", nr)
        for tname, name in _GPT2_NORMS.items():
            layer[name + "_g"] = f32(f"blk.{l}.{tname}.weight", p.n_embd)
            layer[name + "_b"] = f32(f"blk.{l}.{tname}.bias", p.n_embd)
        w.layers.append(layer)
    w.ln_f_g = f32("output_norm.weight", p.n_embd)
    w.ln_f_b = f32("output_norm.bias", p.n_embd)
    w.wte = expanded("token_embd.weight", p.n_vocab, p.n_embd)
    w.wpe = expanded("position_embd.weight", p.n_seq, p.n_embd)
    w.lm_head = matrix("token_embd.weight", p.n_vocab, p.n_embd)
    return w
