"""Llama-family and GPT-2 decoders over the HIP library, plus synthetic weight
builders for the benchmark configurations.

`Llama2` / `Gpt2` mirror `wgml::models::{llama2,gpt2}`: weights are handed over
as GGUF-layout bytes per tensor (what `Llama2Weights::from_gguf` /
`Gpt2Weights::from_gguf` pull out of a file), `forward` enqueues one decode step
and `generate_greedy` runs the chat loop with temperature 0.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import numpy as np

from . import _lib
from ._lib import Gpt2ParamsC, Llama2ConfigC, call
from .ops import GpuInstance, GpuQuantMatrix, _ptr, quantize, rng_normal, rng_tokens

__all__ = ["Llama2Config", "LlamaModelType", "Llama2", "Gpt2Params", "Gpt2", "HostMatrix",
           "LlamaHostWeights", "Gpt2HostWeights", "synth_llama", "synth_gpt2", "use_more_bits",
           "TINY_LLAMA", "LLAMA2_7B", "LLAMA3_8B", "GPT2_124M"]


class LlamaModelType:
    Llama, Qwen2 = 0, 1  # models/llama2/mod.rs:13-33


@dataclass(frozen=True)
class Llama2Config:
    """models/llama2/cpu.rs:46-67"""
    dim: int
    hidden_dim: int
    n_layers: int
    n_q_heads: int
    n_kv_heads: int
    vocab_size: int
    seq_len: int
    rope_base_freq: float = 10000.0
    rms_norm_eps: float = 1.0e-6

    @property
    def kv_dim(self) -> int:
        return self.dim * self.n_kv_heads // self.n_q_heads

    @property
    def head_size(self) -> int:
        return self.dim // self.n_q_heads

    def to_c(self) -> Llama2ConfigC:
        return Llama2ConfigC(self.dim, self.hidden_dim, self.n_layers, self.n_q_heads,
                             self.n_kv_heads, self.vocab_size, self.seq_len, self.rope_base_freq,
                             self.rms_norm_eps)


@dataclass(frozen=True)
class Gpt2Params:
    """models/gpt2/cpu.rs:18-64"""
    n_vocab: int = 50257
    n_seq: int = 1024
    n_embd: int = 768
    n_head: int = 12
    n_layer: int = 12
    ff_len: int = 3072
    attn_b: int = 2304

    def to_c(self) -> Gpt2ParamsC:
        return Gpt2ParamsC(self.n_vocab, self.n_seq, self.n_embd, self.n_head, self.n_layer,
                           self.ff_len, self.attn_b)


@dataclass
class HostMatrix:
    """One GGUF tensor on the host: quantization tag, shape, raw bytes."""
    qtype: int
    nrows: int
    ncols: int
    data: np.ndarray  # uint8 GGUF bytes (or f32 viewed as bytes)

    def nbytes(self) -> int:
        return int(self.data.nbytes)


LLAMA_MATS = ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down")
_LLAMA_MAT_ID = {n: i for i, n in enumerate(LLAMA_MATS)}
_LLAMA_OUTPUT = 7
_LLAMA_VEC_ID = {"attn_norm": 0, "ffn_norm": 1, "attn_q_bias": 2, "attn_k_bias": 3,
                 "attn_v_bias": 4}
_LLAMA_OUTPUT_NORM = 5


@dataclass
class LlamaHostWeights:
    config: Llama2Config
    layers: List[Dict[str, object]] = field(default_factory=list)  # name -> HostMatrix | ndarray
    token_embd: Optional[np.ndarray] = None  # (vocab, dim) f32: row t = embedding of token t
    output: Optional[HostMatrix] = None
    output_norm: Optional[np.ndarray] = None

    def weight_bytes_per_token(self) -> int:
        """GGUF bytes of every matrix and norm vector one decode step reads."""
        total = self.output.nbytes() + self.output_norm.nbytes
        for l in self.layers:
            for v in l.values():
                total += v.nbytes() if isinstance(v, HostMatrix) else v.nbytes
        return total


class Llama2:
    """`Llama2` + `Llama2State` + `Llama2Weights` (models/llama2/transformer.rs)."""

    def __init__(self, gpu: GpuInstance, config: Llama2Config,
                 model_type: int = LlamaModelType.Llama):
        self.gpu, self.config = gpu, config
        h = C.c_void_p()
        cfg = config.to_c()
        call("wgml_llama2_create", gpu.handle, C.byref(cfg), model_type, C.byref(h))
        self._h = h
        self._mats: List[GpuQuantMatrix] = []  # keep the borrowed matrices alive

    def set_matrix(self, name: str, layer: int, hm: HostMatrix) -> None:
        qm = GpuQuantMatrix(self.gpu, hm.qtype, hm.nrows, hm.ncols, hm.data)
        self._mats.append(qm)
        which = _LLAMA_OUTPUT if name == "output" else _LLAMA_MAT_ID[name]
        call("wgml_llama2_set_matrix", self._h, which, layer, qm.handle)

    def set_vector(self, name: str, layer: int, v: np.ndarray) -> None:
        a = np.ascontiguousarray(v, dtype=np.float32)
        which = _LLAMA_OUTPUT_NORM if name == "output_norm" else _LLAMA_VEC_ID[name]
        call("wgml_llama2_set_vector", self._h, which, layer, _ptr(a), a.size)

    def load(self, w: LlamaHostWeights) -> "Llama2":
        for l, layer in enumerate(w.layers):
            for name, v in layer.items():
                if isinstance(v, HostMatrix):
                    self.set_matrix(name, l, v)
                else:
                    self.set_vector(name, l, v)
        self.set_matrix("output", 0, w.output)
        self.set_vector("output_norm", 0, w.output_norm)
        te = np.ascontiguousarray(w.token_embd, dtype=np.float32)
        assert te.shape == (self.config.vocab_size, self.config.dim)
        call("wgml_llama2_set_token_embd", self._h, _ptr(te))
        return self

    @classmethod
    def from_gguf(cls, gpu: GpuInstance, gguf, model_type: int = LlamaModelType.Llama) -> "Llama2":
        """Llama2Config::from_gguf + Llama2Weights::from_gguf (models/llama2/cpu.rs:75-109,
        models/llama2/transformer.rs:137-268) from a `wgml_amd.Gguf`."""
        from .gguf import llama2_config_from_gguf, llama2_weights_from_gguf

        config = llama2_config_from_gguf(gguf, model_type)
        return cls(gpu, config, model_type).load(llama2_weights_from_gguf(gguf, config))

    def generate_sampled(self, prompt, n_total: int, temperature: float, topp: float,
                         seed: int) -> np.ndarray:
        """Token loop with the CPU sampler (temperature / top-p), seeded."""
        p = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.empty(n_total, dtype=np.uint32)
        call("wgml_llama2_generate_sampled", self._h, _ptr(p), p.size, n_total, temperature, topp,
             seed, _ptr(out))
        return out

    def set_fusion(self, level: int) -> None:
        call("wgml_llama2_set_fusion", self._h, level)

    def forward(self, token: int, pos: int) -> None:
        call("wgml_llama2_forward", self._h, token, pos)

    def logits(self) -> np.ndarray:
        out = np.empty(self.config.vocab_size, dtype=np.float32)
        call("wgml_llama2_read_logits", self._h, _ptr(out))
        return out

    def forward_logits(self, pos: int, token: int) -> np.ndarray:
        """ChatLlama2::forward_logits (wgml-chat/src/chat_llama2.rs:155-228)."""
        self.forward(token, pos)
        return self.logits()

    def generate_greedy(self, prompt, n_total: int) -> np.ndarray:
        p = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.empty(n_total, dtype=np.uint32)
        call("wgml_llama2_generate_greedy", self._h, _ptr(p), p.size, n_total, _ptr(out))
        return out

    def prefill(self, tokens, start_pos: int = 0) -> None:
        """Batched prompt pass on the matrix cores: fills the KV cache for the tokens'
        positions and leaves the last token's logits (`logits()`).  The reference has no
        batched pass (it steps through the prompt, chat_llama2.rs:155-228)."""
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        call("wgml_llama2_prefill", self._h, _ptr(t), t.size, start_pos)

    def prefill_decode_greedy(self, prompt, n_new: int) -> np.ndarray:
        """`prefill(prompt)` then greedy decoding; returns the n_new generated tokens."""
        p = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.empty(n_new, dtype=np.uint32)
        call("wgml_llama2_prefill_decode_greedy", self._h, _ptr(p), p.size, n_new, _ptr(out))
        return out

    def decode_greedy(self, first_token: int, start_pos: int, n_steps: int) -> np.ndarray:
        out = np.empty(n_steps, dtype=np.uint32)
        call("wgml_llama2_decode_greedy", self._h, first_token, start_pos, n_steps, _ptr(out))
        return out

    def record_steps(self, start_pos: int, n_steps: int) -> None:
        """Records ahead of time the steps the token loops replay for positions
        start_pos .. start_pos + n_steps - 1 (otherwise the first run through a range of
        positions does it before its first launch)."""
        call("wgml_llama2_record_steps", self._h, start_pos, n_steps)

    def decode_greedy_sync(self, first_token: int, start_pos: int, n_steps: int) -> np.ndarray:
        """Same as decode_greedy with a host read-back of every token."""
        out = np.empty(n_steps, dtype=np.uint32)
        call("wgml_llama2_decode_greedy_sync", self._h, first_token, start_pos, n_steps, _ptr(out))
        return out

    def kv_upload(self, layer: int, which: int, first_pos: int, data: np.ndarray) -> None:
        a = np.ascontiguousarray(data, dtype=np.float32)
        n_pos = a.size // self.config.kv_dim
        call("wgml_llama2_kv_upload", self._h, layer, which, first_pos, n_pos, _ptr(a))

    def kv_download(self, layer: int, which: int, first_pos: int, n_pos: int) -> np.ndarray:
        out = np.empty((n_pos, self.config.kv_dim), dtype=np.float32)
        call("wgml_llama2_kv_download", self._h, layer, which, first_pos, n_pos, _ptr(out))
        return out

    def launches_per_token(self) -> int:
        return _lib.lib.wgml_llama2_launches_per_token(self._h)

    def close(self) -> None:
        if self._h:
            call("wgml_llama2_destroy", self._h)
            self._h = None
        self._mats.clear()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


GPT2_MATS = ("attn_w", "attn_proj_w", "mlp_fc_w", "mlp_proj_w")
_GPT2_MAT_ID = {n: i for i, n in enumerate(GPT2_MATS)}
_GPT2_LM_HEAD = 4
_GPT2_VEC_ID = {"ln_1_g": 0, "ln_1_b": 1, "ln_2_g": 2, "ln_2_b": 3, "attn_b": 4, "attn_proj_b": 5,
                "mlp_fc_b": 6, "mlp_proj_b": 7}
_GPT2_LN_F_G, _GPT2_LN_F_B = 8, 9


@dataclass
class Gpt2HostWeights:
    params: Gpt2Params
    layers: List[Dict[str, object]] = field(default_factory=list)
    wte: Optional[np.ndarray] = None  # (n_vocab, n_embd) f32
    wpe: Optional[np.ndarray] = None  # (n_seq, n_embd) f32
    lm_head: Optional[HostMatrix] = None
    ln_f_g: Optional[np.ndarray] = None
    ln_f_b: Optional[np.ndarray] = None

    def weight_bytes_per_token(self) -> int:
        total = self.lm_head.nbytes() + self.ln_f_g.nbytes + self.ln_f_b.nbytes
        for l in self.layers:
            for v in l.values():
                total += v.nbytes() if isinstance(v, HostMatrix) else v.nbytes
        return total


class Gpt2:
    """`Gpt2` + `Gpt2State` + `Gpt2Weights` (models/gpt2/transformer.rs)."""

    def __init__(self, gpu: GpuInstance, params: Gpt2Params):
        self.gpu, self.params = gpu, params
        h = C.c_void_p()
        p = params.to_c()
        call("wgml_gpt2_create", gpu.handle, C.byref(p), C.byref(h))
        self._h = h
        self._mats: List[GpuQuantMatrix] = []
        self._slots: Dict[Tuple[str, int], GpuQuantMatrix] = {}

    def load(self, w: Gpt2HostWeights) -> "Gpt2":
        for l, layer in enumerate(w.layers):
            for name, v in layer.items():
                if isinstance(v, HostMatrix):
                    self.set_matrix(name, l, v)
                else:
                    a = np.ascontiguousarray(v, dtype=np.float32)
                    call("wgml_gpt2_set_vector", self._h, _GPT2_VEC_ID[name], l, _ptr(a), a.size)
        self.set_matrix("lm_head", 0, w.lm_head)
        for which, v in ((_GPT2_LN_F_G, w.ln_f_g), (_GPT2_LN_F_B, w.ln_f_b)):
            a = np.ascontiguousarray(v, dtype=np.float32)
            call("wgml_gpt2_set_vector", self._h, which, 0, _ptr(a), a.size)
        wte = np.ascontiguousarray(w.wte, dtype=np.float32)
        wpe = np.ascontiguousarray(w.wpe, dtype=np.float32)
        call("wgml_gpt2_set_embeddings", self._h, _ptr(wte), _ptr(wpe))
        return self

    def set_matrix(self, name: str, layer: int, hm: HostMatrix) -> None:
        """Sets or replaces one matrix ("lm_head" or a per-layer name of GPT2_MATS); a matrix
        it replaces is released."""
        qm = GpuQuantMatrix(self.gpu, hm.qtype, hm.nrows, hm.ncols, hm.data)
        which = _GPT2_LM_HEAD if name == "lm_head" else _GPT2_MAT_ID[name]
        call("wgml_gpt2_set_matrix", self._h, which, layer, qm.handle)
        old = self._slots.get((name, layer))
        self._slots[(name, layer)] = qm
        self._mats.append(qm)
        if old is not None:
            self._mats.remove(old)

    @classmethod
    def from_gguf(cls, gpu: GpuInstance, gguf) -> "Gpt2":
        """Gpt2Params::from_gguf + Gpt2Weights::from_gguf (models/gpt2/cpu.rs:34-47,
        models/gpt2/transformer.rs:108-205) from a `wgml_amd.Gguf`."""
        from .gguf import gpt2_params_from_gguf, gpt2_weights_from_gguf

        params = gpt2_params_from_gguf(gguf)
        return cls(gpu, params).load(gpt2_weights_from_gguf(gguf, params))

    def set_fusion(self, level: int) -> None:
        call("wgml_gpt2_set_fusion", self._h, level)

    def launches_per_token(self) -> int:
        return _lib.lib.wgml_gpt2_launches_per_token(self._h)

    def forward(self, token: int, pos: int) -> None:
        call("wgml_gpt2_forward", self._h, token, pos)

    def logits(self) -> np.ndarray:
        out = np.empty(self.params.n_vocab, dtype=np.float32)
        call("wgml_gpt2_read_logits", self._h, _ptr(out))
        return out

    def generate_greedy(self, prompt, n_total: int) -> np.ndarray:
        p = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.empty(n_total, dtype=np.uint32)
        call("wgml_gpt2_generate_greedy", self._h, _ptr(p), p.size, n_total, _ptr(out))
        return out

    def record_steps(self, n_total: int) -> None:
        """Records ahead of time the steps `generate_greedy` replays for positions
        0 .. n_total - 1."""
        call("wgml_gpt2_record_steps", self._h, n_total)

    def close(self) -> None:
        if self._h:
            call("wgml_gpt2_destroy", self._h)
            self._h = None
        self._mats.clear()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


# ---- synthetic models of the benchmark configurations -------------------------

TINY_LLAMA = Llama2Config(dim=288, hidden_dim=768, n_layers=6, n_q_heads=6, n_kv_heads=6,
                          vocab_size=32000, seq_len=256, rope_base_freq=10000.0,
                          rms_norm_eps=1.0e-5)
LLAMA2_7B = Llama2Config(dim=4096, hidden_dim=11008, n_layers=32, n_q_heads=32, n_kv_heads=32,
                         vocab_size=32000, seq_len=512, rope_base_freq=10000.0,
                         rms_norm_eps=1.0e-5)
LLAMA3_8B = Llama2Config(dim=4096, hidden_dim=14336, n_layers=32, n_q_heads=32, n_kv_heads=8,
                         vocab_size=128256, seq_len=8448, rope_base_freq=500000.0,
                         rms_norm_eps=1.0e-5)
GPT2_124M = Gpt2Params()


def use_more_bits(i_layer: int, n_layers: int) -> bool:
    """llama.cpp's Q4_K_M rule for which ffn_down layers get Q6_K."""
    return (i_layer < n_layers // 8 or i_layer >= 7 * n_layers // 8
            or (i_layer - n_layers // 8) % 3 == 2)


def _seed(base: int, tensor_index: int) -> int:
    return (base << 20) + tensor_index


def _rand_matrix(seed: int, nrows: int, ncols: int, qtype: int, std: float = 0.02) -> HostMatrix:
    vals = rng_normal(seed, nrows * ncols, 0.0, std)
    if qtype == _lib.F32:
        return HostMatrix(qtype, nrows, ncols, vals.view(np.uint8))
    return HostMatrix(qtype, nrows, ncols, quantize(qtype, vals))


def synth_llama(config: Llama2Config, seed: int, scheme: str = "q8_0",
                progress=None) -> LlamaHostWeights:
    """Seeded N(0, 0.02) weights quantized with the ggml reference quantizers.

    scheme: "q8_0" | "q4_k" | "q6_k" (every matrix in that format) or "q4_k_m"
    (Q4_K, with Q6_K for attn_v, output and the ffn_down layers picked by
    use_more_bits).  Norm weights are 1.0; the embedding stays f32.
    Tensor order = Llama2Weights::from_gguf (models/llama2/transformer.rs:161-172,
    235-237): per layer q,k,v,output,down,gate,up, then token_embd, output.
    """
    c = config
    Q = {"q8_0": _lib.Q8_0, "q4_k": _lib.Q4_K, "q6_k": _lib.Q6_K, "f32": _lib.F32}
    w = LlamaHostWeights(config=c)
    idx = 0

    def pick(name: str, layer: int) -> int:
        if scheme != "q4_k_m":
            return Q[scheme]
        if name in ("attn_v", "output"):
            return _lib.Q6_K
        if name == "ffn_down" and use_more_bits(layer, c.n_layers):
            return _lib.Q6_K
        return _lib.Q4_K

    shapes = {"attn_q": (c.dim, c.dim), "attn_k": (c.kv_dim, c.dim), "attn_v": (c.kv_dim, c.dim),
              "attn_output": (c.dim, c.dim), "ffn_down": (c.dim, c.hidden_dim),
              "ffn_gate": (c.hidden_dim, c.dim), "ffn_up": (c.hidden_dim, c.dim)}
    order = ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_down", "ffn_gate", "ffn_up")
    for l in range(c.n_layers):
        layer: Dict[str, object] = {}
        for name in order:
            r, k = shapes[name]
            layer[name] = _rand_matrix(_seed(seed, idx), r, k, pick(name, l))
            idx += 1
        layer["attn_norm"] = np.ones(c.dim, dtype=np.float32)
        layer["ffn_norm"] = np.ones(c.dim, dtype=np.float32)
        w.layers.append(layer)
        if progress:
            progress(l)
    w.token_embd = rng_normal(_seed(seed, idx), c.vocab_size * c.dim, 0.0, 0.02).reshape(
        c.vocab_size, c.dim)
    idx += 1
    w.output = _rand_matrix(_seed(seed, idx), c.vocab_size, c.dim, pick("output", 0))
    w.output_norm = np.ones(c.dim, dtype=np.float32)
    return w


def synth_gpt2(params: Gpt2Params, seed: int, qtype: int = _lib.Q8_0) -> Gpt2HostWeights:
    """Seeded GPT-2 weights: 2-D weights N(0,0.02) quantized to `qtype`,
    biases N(0,0.02) f32, gamma = 1, beta = 0, wte/wpe f32; lm_head = wte
    quantized (GPT-2 ties them, models/gpt2/cpu.rs:195-196)."""
    p = params
    w = Gpt2HostWeights(params=p)
    idx = 0
    shapes = {"attn_w": (p.attn_b, p.n_embd), "attn_proj_w": (p.n_embd, p.n_embd),
              "mlp_fc_w": (p.ff_len, p.n_embd), "mlp_proj_w": (p.n_embd, p.ff_len)}
    bias = {"attn_b": p.attn_b, "attn_proj_b": p.n_embd, "mlp_fc_b": p.ff_len,
            "mlp_proj_b": p.n_embd}
    for _ in range(p.n_layer):
        layer: Dict[str, object] = {}
        for name, (r, k) in shapes.items():
            layer[name] = _rand_matrix(_seed(seed, idx), r, k, qtype)
            idx += 1
        for name, n in bias.items():
            layer[name] = rng_normal(_seed(seed, idx), n, 0.0, 0.02)
            idx += 1
        for g in ("ln_1_g", "ln_2_g"):
            layer[g] = np.ones(p.n_embd, dtype=np.float32)
        for b in ("ln_1_b", "ln_2_b"):
            layer[b] = np.zeros(p.n_embd, dtype=np.float32)
        w.layers.append(layer)
    w.wte = rng_normal(_seed(seed, idx), p.n_vocab * p.n_embd, 0.0, 0.02).reshape(p.n_vocab,
                                                                                   p.n_embd)
    idx += 1
    w.wpe = rng_normal(_seed(seed, idx), p.n_seq * p.n_embd, 0.0, 0.02).reshape(p.n_seq, p.n_embd)
    if qtype == _lib.F32:
        w.lm_head = HostMatrix(qtype, p.n_vocab, p.n_embd, w.wte.reshape(-1).view(np.uint8))
    else:
        w.lm_head = HostMatrix(qtype, p.n_vocab, p.n_embd, quantize(qtype, w.wte))
    w.ln_f_g = np.ones(p.n_embd, dtype=np.float32)
    w.ln_f_b = np.zeros(p.n_embd, dtype=np.float32)
    return w


def prompt_tokens(seed: int, n: int, vocab: int) -> np.ndarray:
    return rng_tokens(_seed(seed, 0xFF), n, vocab)
