"""ctypes binding of the CPU oracle (oracle/libwgml_oracle.so).

Test infrastructure only: nothing in the product imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from pathlib import Path

import numpy as np

ORACLE_DIR = Path(__file__).resolve().parent.parent / "oracle"
LIB = ORACLE_DIR / "libwgml_oracle.so"

F32, Q8_0, Q4_K, Q6_K = 0, 8, 12, 14
F16, Q4_0, Q4_1, Q5_0, Q5_1, Q5_K, Q8_K = 1, 2, 3, 6, 7, 13, 15


def build(force: bool = False) -> None:
    if force or not LIB.exists():
        subprocess.run(["make", "-C", os.fspath(ORACLE_DIR)] + (["-B"] if force else []),
                       check=True, capture_output=True)


build()
lib = C.CDLL(os.fspath(LIB))

_P, _i, _f, _u32 = C.c_void_p, C.c_int, C.c_float, C.c_uint32


class AttnParams(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("seq_len", "kv_dim", "kv_mul", "n_heads", "head_size",
                                          "pos")]


class Matrix(C.Structure):
    _fields_ = [("type", _i), ("data", _P), ("nrows", _i), ("ncols", _i)]


class LlamaConfig(C.Structure):
    _fields_ = [(n, _i) for n in ("dim", "hidden_dim", "n_layers", "n_q_heads", "n_kv_heads",
                                  "vocab_size", "seq_len")] + \
               [("rope_base_freq", _f), ("rms_norm_eps", _f), ("rope_variant", _i)]


class LlamaLayer(C.Structure):
    _fields_ = [(n, Matrix) for n in ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate",
                                      "ffn_up", "ffn_down")] + \
               [(n, _P) for n in ("attn_norm", "ffn_norm", "attn_q_bias", "attn_k_bias",
                                  "attn_v_bias")]


class Gpt2ParamsC(C.Structure):
    _fields_ = [(n, _i) for n in ("n_vocab", "n_seq", "n_embd", "n_head", "n_layer", "ff_len",
                                  "attn_b")]


class Gpt2Layer(C.Structure):
    _fields_ = [("ln_1_g", _P), ("ln_1_b", _P), ("ln_2_g", _P), ("ln_2_b", _P),
                ("c_attn_attn_w", Matrix), ("c_attn_attn_b", _P),
                ("c_attn_proj_w", Matrix), ("c_attn_proj_b", _P),
                ("c_mlp_fc_w", Matrix), ("c_mlp_fc_b", _P),
                ("c_mlp_proj_w", Matrix), ("c_mlp_proj_b", _P)]


lib.orc_decode_f16.restype = _f
lib.orc_decode_f16.argtypes = [C.c_uint16]
lib.orc_block_bytes.restype = C.c_size_t
lib.orc_block_bytes.argtypes = [_i]
lib.orc_block_elems.restype = C.c_size_t
lib.orc_block_elems.argtypes = [_i]
lib.orc_dequantize.restype = _i
lib.orc_dequantize.argtypes = [_i, _P, C.c_size_t, _P]
lib.orc_gemv_f32.argtypes = [_P, _P, _P, _i, _i]
lib.orc_gemv_f32_colmajor.argtypes = [_P, _P, _P, _i, _i]
lib.orc_gemv_f64.argtypes = [_P, _P, _P, _i, _i]
lib.orc_set_threads.restype = None
lib.orc_set_threads.argtypes = [_i]
lib.orc_get_threads.restype = _i


def set_threads(n: int) -> None:
    """Threads for the rows of matrix-vector products (timing mode of the benchmark's CPU
    baseline; 1 = single-threaded as the reference, results do not depend on it)."""
    lib.orc_set_threads(int(n))


lib.orc_gemv_quant.restype = _i
lib.orc_gemv_quant.argtypes = [_i, _P, _i, _i, _P, _P, _P]
lib.orc_rms_norm.argtypes = [_P, _P, _P, _i, _f]
lib.orc_layernorm.argtypes = [_P, _P, _i]
lib.orc_softmax.argtypes = [_P, _i]
lib.orc_silu.argtypes = [_P, _P, _i]
lib.orc_gelu.argtypes = [_P, _i]
lib.orc_rope.argtypes = [_P, _P, _i, _i, _i, _i, _f, _i]
lib.orc_attention.argtypes = [C.POINTER(AttnParams), _P, _P, _P, _P, _P]
lib.orc_argmax.restype = _u32
lib.orc_argmax.argtypes = [_P, _i]
lib.orc_llama2_new.restype = _P
lib.orc_llama2_new.argtypes = [C.POINTER(LlamaConfig), C.POINTER(LlamaLayer), _P,
                               C.POINTER(Matrix), _P]
lib.orc_llama2_free.argtypes = [_P]
lib.orc_llama2_predequantize.restype = _i
lib.orc_llama2_predequantize.argtypes = [_P]
lib.orc_llama2_forward.argtypes = [_P, _i, _i]
lib.orc_llama2_logits.restype = C.POINTER(C.c_float)
lib.orc_llama2_logits.argtypes = [_P]
lib.orc_llama2_key_cache.restype = C.POINTER(C.c_float)
lib.orc_llama2_key_cache.argtypes = [_P, _i]
lib.orc_llama2_value_cache.restype = C.POINTER(C.c_float)
lib.orc_llama2_value_cache.argtypes = [_P, _i]
lib.orc_llama2_x.restype = C.POINTER(C.c_float)
lib.orc_llama2_x.argtypes = [_P]
lib.orc_gpt2_new.restype = _P
lib.orc_gpt2_new.argtypes = [C.POINTER(Gpt2ParamsC), C.POINTER(Gpt2Layer), _P, _P,
                             C.POINTER(Matrix), _P, _P]
lib.orc_gpt2_free.argtypes = [_P]
lib.orc_gpt2_predequantize.restype = _i
lib.orc_gpt2_predequantize.argtypes = [_P]
lib.orc_gpt2_forward.argtypes = [_P, _i, _i]
lib.orc_gpt2_logits.restype = C.POINTER(C.c_float)
lib.orc_gpt2_logits.argtypes = [_P]


def _p(a: np.ndarray):
    return C.c_void_p(a.ctypes.data)


def f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def decode_f16(bits: int) -> float:
    return lib.orc_decode_f16(bits)


def dequantize(qtype: int, raw: np.ndarray, nelems: int) -> np.ndarray:
    raw = np.ascontiguousarray(raw).view(np.uint8)
    out = np.empty(nelems, dtype=np.float32)
    rc = lib.orc_dequantize(qtype, _p(raw), nelems, _p(out))
    assert rc == 0, "unsupported type"
    return out


def gemv_quant(qtype: int, raw: np.ndarray, nrows: int, ncols: int, x: np.ndarray):
    """Returns (f32 sequential sum as the reference's CPU gemv, f64 sum)."""
    raw = np.ascontiguousarray(raw).view(np.uint8)
    x = f32(x)
    o32 = np.empty(nrows, dtype=np.float32)
    o64 = np.empty(nrows, dtype=np.float64)
    rc = lib.orc_gemv_quant(qtype, _p(raw), nrows, ncols, _p(x), _p(o32), _p(o64))
    assert rc == 0
    return o32, o64


def gemv_f32(w: np.ndarray, x: np.ndarray) -> np.ndarray:
    w, x = f32(w), f32(x)
    out = np.empty(w.shape[0], dtype=np.float32)
    lib.orc_gemv_f32(_p(out), _p(w), _p(x), w.shape[0], w.shape[1])
    return out


def gemv_f64(w: np.ndarray, x: np.ndarray) -> np.ndarray:
    w, x = f32(w), f32(x)
    out = np.empty(w.shape[0], dtype=np.float64)
    lib.orc_gemv_f64(_p(out), _p(w), _p(x), w.shape[0], w.shape[1])
    return out


def rms_norm(a, w, eps) -> np.ndarray:
    a, w = f32(a), f32(w)
    out = np.empty_like(a)
    lib.orc_rms_norm(_p(out), _p(a), _p(w), a.size, eps)
    return out


def layernorm(v) -> np.ndarray:
    v = f32(v)
    out = np.empty_like(v)
    lib.orc_layernorm(_p(out), _p(v), v.size)
    return out


def softmax(v) -> np.ndarray:
    v = f32(v).copy()
    lib.orc_softmax(_p(v), v.size)
    return v


def silu(h1, h2) -> np.ndarray:
    h1, h2 = f32(h1).copy(), f32(h2)
    lib.orc_silu(_p(h1), _p(h2), h1.size)
    return h1


def gelu(x) -> np.ndarray:
    x = f32(x).copy()
    lib.orc_gelu(_p(x), x.size)
    return x


def rope(q, k, head_size, kv_dim, pos, base_freq, variant=0):
    q, k = f32(q).copy(), f32(k).copy()
    lib.orc_rope(_p(q), _p(k), head_size, q.size, kv_dim, pos, base_freq, variant)
    return q, k


def attention(seq_len, kv_dim, kv_mul, n_heads, head_size, pos, q, key_cache, value_cache):
    """Returns (xb, attn[n_heads, seq_len])."""
    p = AttnParams(seq_len, kv_dim, kv_mul, n_heads, head_size, pos)
    q, kc, vc = f32(q), f32(key_cache), f32(value_cache)
    att = np.zeros((n_heads, seq_len), dtype=np.float32)
    xb = np.zeros(n_heads * head_size, dtype=np.float32)
    lib.orc_attention(C.byref(p), _p(q), _p(kc), _p(vc), _p(att), _p(xb))
    return xb, att


def argmax(v) -> int:
    v = f32(v)
    return lib.orc_argmax(_p(v), v.size)


def _matrix(hm) -> Matrix:
    return Matrix(hm.qtype, hm.data.ctypes.data, hm.nrows, hm.ncols)


class Llama2:
    """Oracle transformer over the same host weights the GPU model loads."""

    def __init__(self, w, rope_variant: int = 0, predequantize: bool = False):
        c = w.config
        self.w = w  # keeps every numpy array alive
        self.cfg = LlamaConfig(c.dim, c.hidden_dim, c.n_layers, c.n_q_heads, c.n_kv_heads,
                               c.vocab_size, c.seq_len, c.rope_base_freq, c.rms_norm_eps,
                               rope_variant)
        self._keep = []
        layers = (LlamaLayer * c.n_layers)()
        for i, l in enumerate(w.layers):
            for name in ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up",
                         "ffn_down"):
                setattr(layers[i], name, _matrix(l[name]))
            for name in ("attn_norm", "ffn_norm", "attn_q_bias", "attn_k_bias", "attn_v_bias"):
                v = l.get(name)
                if v is not None:
                    v = f32(v)
                    self._keep.append(v)
                    setattr(layers[i], name, v.ctypes.data)
        self._layers = layers
        self._te = f32(w.token_embd)
        self._on = f32(w.output_norm)
        self._out = _matrix(w.output)
        self._h = lib.orc_llama2_new(C.byref(self.cfg), layers, _p(self._te), C.byref(self._out),
                                     _p(self._on))
        if predequantize:
            assert lib.orc_llama2_predequantize(self._h) == 0

    def forward(self, token: int, pos: int) -> np.ndarray:
        lib.orc_llama2_forward(self._h, int(token), int(pos))
        return np.ctypeslib.as_array(lib.orc_llama2_logits(self._h),
                                     shape=(self.cfg.vocab_size,)).copy()

    def key_cache(self, layer: int) -> np.ndarray:
        kv_dim = self.cfg.dim * self.cfg.n_kv_heads // self.cfg.n_q_heads
        return np.ctypeslib.as_array(lib.orc_llama2_key_cache(self._h, layer),
                                     shape=(self.cfg.seq_len, kv_dim))

    def value_cache(self, layer: int) -> np.ndarray:
        kv_dim = self.cfg.dim * self.cfg.n_kv_heads // self.cfg.n_q_heads
        return np.ctypeslib.as_array(lib.orc_llama2_value_cache(self._h, layer),
                                     shape=(self.cfg.seq_len, kv_dim))

    def generate_greedy(self, prompt, n_total: int):
        """Same loop contract as wgml_llama2_generate_greedy.  Also returns the
        top-2 logit margin of every step."""
        out = np.empty(n_total, dtype=np.uint32)
        margins = np.empty(n_total, dtype=np.float32)
        token = int(prompt[0])
        for pos in range(n_total):
            logits = self.forward(token, pos)
            best = argmax(logits)
            top2 = np.partition(logits, -2)[-2:]
            margins[pos] = top2[1] - top2[0]
            out[pos] = best
            token = int(prompt[pos + 1]) if pos + 1 < len(prompt) else best
        return out, margins

    def __del__(self):
        try:
            lib.orc_llama2_free(self._h)
        except Exception:
            pass


class Gpt2:
    def __init__(self, w, predequantize: bool = False):
        p = w.params
        self.w = w
        self.p = Gpt2ParamsC(p.n_vocab, p.n_seq, p.n_embd, p.n_head, p.n_layer, p.ff_len, p.attn_b)
        self._keep = []
        layers = (Gpt2Layer * p.n_layer)()
        mats = {"attn_w": "c_attn_attn_w", "attn_proj_w": "c_attn_proj_w",
                "mlp_fc_w": "c_mlp_fc_w", "mlp_proj_w": "c_mlp_proj_w"}
        vecs = {"ln_1_g": "ln_1_g", "ln_1_b": "ln_1_b", "ln_2_g": "ln_2_g", "ln_2_b": "ln_2_b",
                "attn_b": "c_attn_attn_b", "attn_proj_b": "c_attn_proj_b",
                "mlp_fc_b": "c_mlp_fc_b", "mlp_proj_b": "c_mlp_proj_b"}
        for i, l in enumerate(w.layers):
            for k, field in mats.items():
                setattr(layers[i], field, _matrix(l[k]))
            for k, field in vecs.items():
                v = f32(l[k])
                self._keep.append(v)
                setattr(layers[i], field, v.ctypes.data)
        self._layers = layers
        self._wte, self._wpe = f32(w.wte), f32(w.wpe)
        self._g, self._b = f32(w.ln_f_g), f32(w.ln_f_b)
        self._head = _matrix(w.lm_head)
        self._h = lib.orc_gpt2_new(C.byref(self.p), layers, _p(self._wte), _p(self._wpe),
                                   C.byref(self._head), _p(self._g), _p(self._b))
        if predequantize:
            assert lib.orc_gpt2_predequantize(self._h) == 0

    def forward(self, token: int, pos: int) -> np.ndarray:
        lib.orc_gpt2_forward(self._h, int(token), int(pos))
        return np.ctypeslib.as_array(lib.orc_gpt2_logits(self._h),
                                     shape=(self.p.n_vocab,)).copy()

    def generate_greedy(self, prompt, n_total: int):
        out = np.empty(n_total, dtype=np.uint32)
        margins = np.empty(n_total, dtype=np.float32)
        token = int(prompt[0])
        for pos in range(n_total):
            logits = self.forward(token, pos)
            best = argmax(logits)
            top2 = np.partition(logits, -2)[-2:]
            margins[pos] = top2[1] - top2[0]
            out[pos] = best
            token = int(prompt[pos + 1]) if pos + 1 < len(prompt) else best
        return out, margins

    def __del__(self):
        try:
            lib.orc_gpt2_free(self._h)
        except Exception:
            pass


lib.orc_sample.restype = C.c_uint32
lib.orc_sample.argtypes = [_P, _i, C.c_float, C.c_float, C.c_float]
lib.orc_sample_mult.restype = C.c_uint32
lib.orc_sample_mult.argtypes = [_P, _i, C.c_float]
lib.orc_sample_topp.restype = C.c_uint32
lib.orc_sample_topp.argtypes = [_P, _i, C.c_float, C.c_float]


def sample(logits: np.ndarray, temperature: float, topp: float, coin: float) -> int:
    """Sampler::sample (models/sampler.rs:32-52) on a copy of `logits`."""
    v = np.ascontiguousarray(logits, dtype=np.float32).copy()
    return int(lib.orc_sample(_p(v), v.size, temperature, topp, coin))


def sample_mult(p: np.ndarray, coin: float) -> int:
    v = np.ascontiguousarray(p, dtype=np.float32)
    return int(lib.orc_sample_mult(_p(v), v.size, coin))


def sample_topp(p: np.ndarray, topp: float, coin: float) -> int:
    v = np.ascontiguousarray(p, dtype=np.float32)
    return int(lib.orc_sample_topp(_p(v), v.size, topp, coin))
