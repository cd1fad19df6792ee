"""ctypes binding of libwgml_hip.so (the C ABI declared in include/wgml_hip.h).

The library is the product; this module only loads it and declares prototypes.
There is no fallback: if the shared library is missing, importing raises.
"""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path

_PKG = Path(__file__).resolve().parent
LIB_PATH = _PKG / "lib" / "libwgml_hip.so"


class WgmlError(RuntimeError):
    """A call into libwgml_hip returned a non-zero status."""

    def __init__(self, code: int, message: str):
        super().__init__(f"[wgml status {code}] {message}")
        self.code = code
        self.message = message


OK, E_INVALID, E_UNSUPPORTED, E_HIP, E_NO_DEVICE, E_OOM = range(6)

# GGUF tensor-type ids (gguf.rs:70-103 of the reference)
F32, F16, Q4_0, Q4_1, Q5_0, Q5_1, Q8_0 = 0, 1, 2, 3, 6, 7, 8
Q4_K, Q5_K, Q6_K, Q8_K = 12, 13, 14, 15
TYPE_NAMES = {F32: "F32", Q8_0: "Q8_0", Q4_K: "Q4_K", Q6_K: "Q6_K"}


class View(C.Structure):
    """wgml_view: an f32 vector view (buffer, element offset, length)."""

    _fields_ = [("buf", C.c_void_p), ("offset", C.c_uint64), ("len", C.c_uint32)]


class RopeConfig(C.Structure):
    """wgml_rope_config == RoPEConfig (ops/rope.rs:30-35)."""

    _fields_ = [("head_size", C.c_uint32), ("kv_dim", C.c_uint32), ("pos", C.c_uint32),
                ("base_freq", C.c_float)]


class AttnParams(C.Structure):
    """wgml_attn_params == BatchedMultiqueryAttentionParams
    (ops/batched_multiquery_attention.rs:30-37)."""

    _fields_ = [("seq_len", C.c_uint32), ("kv_dim", C.c_uint32), ("kv_mul", C.c_uint32),
                ("n_heads", C.c_uint32), ("head_size", C.c_uint32), ("pos", C.c_uint32)]


class Llama2ConfigC(C.Structure):
    _fields_ = [("dim", C.c_uint32), ("hidden_dim", C.c_uint32), ("n_layers", C.c_uint32),
                ("n_q_heads", C.c_uint32), ("n_kv_heads", C.c_uint32), ("vocab_size", C.c_uint32),
                ("seq_len", C.c_uint32), ("rope_base_freq", C.c_float),
                ("rms_norm_eps", C.c_float)]


class Gpt2ParamsC(C.Structure):
    _fields_ = [("n_vocab", C.c_uint32), ("n_seq", C.c_uint32), ("n_embd", C.c_uint32),
                ("n_head", C.c_uint32), ("n_layer", C.c_uint32), ("ff_len", C.c_uint32),
                ("attn_b", C.c_uint32)]


class GgufKv(C.Structure):
    """wgml_gguf_kv"""

    _fields_ = [("key", C.c_char_p), ("type", C.c_int), ("array_type", C.c_int),
                ("array_len", C.c_uint64), ("data", C.c_void_p), ("nbytes", C.c_uint64)]


class GgufTensorInfo(C.Structure):
    """wgml_gguf_tensor_info"""

    _fields_ = [("name", C.c_char_p), ("type", C.c_int), ("ndims", C.c_uint32),
                ("dims", C.c_uint64 * 4), ("offset", C.c_uint64), ("nbytes", C.c_uint64),
                ("data", C.c_void_p)]


_P = C.c_void_p
_PP = C.POINTER(C.c_void_p)
_u32, _u64, _i, _f = C.c_uint32, C.c_uint64, C.c_int, C.c_float
_u32p = C.POINTER(C.c_uint32)
_fp = C.POINTER(C.c_float)

# name -> (restype, argtypes).  Every symbol declared in include/wgml_hip.h.
PROTOTYPES = {
    "wgml_last_error": (C.c_char_p, []),
    "wgml_version": (C.c_char_p, []),
    "wgml_ctx_create": (_i, [_i, _PP]),
    "wgml_ctx_destroy": (_i, [_P]),
    "wgml_ctx_synchronize": (_i, [_P]),
    "wgml_ctx_stream": (_i, [_P, _PP]),
    "wgml_ctx_info": (_i, [_P, C.c_char_p, C.c_size_t, C.POINTER(_i)]),
    "wgml_timer_start": (_i, [_P]),
    "wgml_timer_stop": (_i, [_P, _fp]),
    "wgml_buf_create": (_i, [_P, _u64, _PP]),
    "wgml_buf_destroy": (_i, [_P]),
    "wgml_buf_size": (_u64, [_P]),
    "wgml_buf_upload": (_i, [_P, _u64, _P, _u64]),
    "wgml_buf_download": (_i, [_P, _u64, _P, _u64]),
    "wgml_buf_copy": (_i, [_P, _u64, _P, _u64, _u64]),
    "wgml_buf_zero": (_i, [_P]),
    "wgml_quant_matrix_create": (_i, [_P, _i, _u32, _u32, _P, _PP]),
    "wgml_quant_matrix_destroy": (_i, [_P]),
    "wgml_quant_matrix_shape": (_i, [_P, C.POINTER(_i), _u32p, _u32p]),
    "wgml_quant_matrix_gguf_bytes": (_u64, [_P]),
    "wgml_quant_matrix_weight_bound": (_i, [_P, _fp]),
    "wgml_quant_bytes": (_u64, [_i, _u64]),
    "wgml_quant_block_elems": (_u32, [_i]),
    "wgml_gemv_quant": (_i, [_P, View, _P, View]),
    "wgml_gemm_quant": (_i, [_P, View, _P, View, _u32]),
    "wgml_ctx_set_gemm_precision": (_i, [_P, _i]),
    "wgml_dequantize": (_i, [_P, View, _P]),
    "wgml_f16_to_f32": (_i, [_P, View, _P, _u64]),
    "wgml_gemv_f32": (_i, [_P, View, View, _u32, _u32, _i, View]),
    "wgml_rms_norm": (_i, [_P, _f, View, View, View]),
    "wgml_layernorm": (_i, [_P, View, View]),
    "wgml_rope": (_i, [_P, _i, C.POINTER(RopeConfig), View, View]),
    "wgml_softmax": (_i, [_P, View, _u32, _u32, _u32]),
    "wgml_attention": (_i, [_P, C.POINTER(AttnParams), View, View, View, View, View]),
    "wgml_attention_noalloc": (_i, [_P, C.POINTER(AttnParams), View, View, View, View]),
    "wgml_attention_gemv_quant": (_i, [_P, C.POINTER(AttnParams), View, View, View, View, _P, View, _i]),
    "wgml_silu": (_i, [_P, View, View]),
    "wgml_unary_inplace": (_i, [_P, _i, View, _fp]),
    "wgml_op_assign": (_i, [_P, _i, View, View]),
    "wgml_argmax": (_i, [_P, View, _u32p]),
    "wgml_llama2_create": (_i, [_P, C.POINTER(Llama2ConfigC), _i, _PP]),
    "wgml_llama2_destroy": (_i, [_P]),
    "wgml_llama2_set_matrix": (_i, [_P, _i, _u32, _P]),
    "wgml_llama2_set_vector": (_i, [_P, _i, _u32, _P, _u32]),
    "wgml_llama2_set_token_embd": (_i, [_P, _P]),
    "wgml_llama2_forward": (_i, [_P, _u32, _u32]),
    "wgml_llama2_read_logits": (_i, [_P, _P]),
    "wgml_llama2_generate_greedy": (_i, [_P, _P, _u32, _u32, _P]),
    "wgml_llama2_prefill": (_i, [_P, _P, _u32, _u32]),
    "wgml_llama2_prefill_decode_greedy": (_i, [_P, _P, _u32, _u32, _P]),
    "wgml_llama2_decode_greedy": (_i, [_P, _u32, _u32, _u32, _P]),
    "wgml_llama2_record_steps": (_i, [_P, _u32, _u32]),
    "wgml_gpt2_record_steps": (_i, [_P, _u32]),
    "wgml_llama2_decode_greedy_sync": (_i, [_P, _u32, _u32, _u32, _P]),
    "wgml_llama2_kv_upload": (_i, [_P, _u32, _i, _u32, _u32, _P]),
    "wgml_llama2_kv_download": (_i, [_P, _u32, _i, _u32, _u32, _P]),
    "wgml_llama2_launches_per_token": (_i, [_P]),
    "wgml_llama2_set_fusion": (_i, [_P, _i]),
    "wgml_gpt2_create": (_i, [_P, C.POINTER(Gpt2ParamsC), _PP]),
    "wgml_gpt2_destroy": (_i, [_P]),
    "wgml_gpt2_set_matrix": (_i, [_P, _i, _u32, _P]),
    "wgml_gpt2_set_vector": (_i, [_P, _i, _u32, _P, _u32]),
    "wgml_gpt2_set_embeddings": (_i, [_P, _P, _P]),
    "wgml_gpt2_forward": (_i, [_P, _u32, _u32]),
    "wgml_gpt2_read_logits": (_i, [_P, _P]),
    "wgml_gpt2_generate_greedy": (_i, [_P, _P, _u32, _u32, _P]),
    "wgml_gpt2_set_fusion": (_i, [_P, _i]),
    "wgml_gpt2_launches_per_token": (_i, [_P]),
    "wgml_bench_gemv_quant": (_i, [_P, _PP, _u32, View, View, _u32, _i, _fp]),
    "wgml_bench_read_chain": (_i, [_P, _u32, _u32, _i, _fp]),
    "wgml_bench_gemv_fused": (_i, [_P, _PP, _PP, C.POINTER(C.c_int), _u32, _u32, View, _u32, View,
                                   C.POINTER(View), _u32, _fp]),
    "wgml_bench_attention": (_i, [_P, C.POINTER(AttnParams), _u32, View, C.POINTER(View), C.POINTER(View),
                                  _u32, View, _u32, _fp]),
    "wgml_sample": (_i, [_P, _u32, _f, _f, _f, _u32p]),
    "wgml_llama2_generate_sampled": (_i, [_P, _P, _u32, _u32, _f, _f, _u64, _P]),
    "wgml_gguf_open": (_i, [C.c_char_p, _PP]),
    "wgml_gguf_open_bytes": (_i, [_P, _u64, _PP]),
    "wgml_gguf_close": (_i, [_P]),
    "wgml_gguf_version": (_u32, [_P]),
    "wgml_gguf_alignment": (_u32, [_P]),
    "wgml_gguf_n_metadata": (_u64, [_P]),
    "wgml_gguf_n_tensors": (_u64, [_P]),
    "wgml_gguf_find_metadata": (C.c_int64, [_P, C.c_char_p]),
    "wgml_gguf_find_tensor": (C.c_int64, [_P, C.c_char_p]),
    "wgml_gguf_metadata": (_i, [_P, _u64, C.POINTER(GgufKv)]),
    "wgml_gguf_metadata_string": (_i, [_P, _u64, _u64, C.POINTER(C.c_char_p), C.POINTER(_u64)]),
    "wgml_gguf_tensor": (_i, [_P, _u64, C.POINTER(GgufTensorInfo)]),
    "wgml_llama_tokenizer_create": (_i, [_P, _P, _u32, _P, _u32, _u32, _u32, _PP]),
    "wgml_gpt2_tokenizer_create": (_i, [_P, _P, _u32, _P, _P, _u32, _u32, _u32, _PP]),
    "wgml_tokenizer_destroy": (_i, [_P]),
    "wgml_tokenizer_vocab_size": (_u32, [_P]),
    "wgml_tokenizer_bos": (_u32, [_P]),
    "wgml_tokenizer_eos": (_u32, [_P]),
    "wgml_tokenizer_unk": (_u32, [_P]),
    "wgml_tokenizer_token": (_i, [_P, _u32, C.POINTER(C.c_char_p), C.POINTER(_u64)]),
    "wgml_llama_tokenizer_encode": (_i, [_P, _P, _u64, _i, _i, _P, _u64, C.POINTER(_u64)]),
    "wgml_llama_tokenizer_decode": (_i, [_P, _u32, _u32, _P, _u64, C.POINTER(_u64)]),
    "wgml_gpt2_tokenizer_encode": (_i, [_P, _P, _u64, _P, _u64, C.POINTER(_u64)]),
    "wgml_gpt2_tokenizer_decode": (_i, [_P, _P, _u64, _i, _P, _u64, C.POINTER(_u64)]),
    "wgml_quantize": (_i, [_i, _P, _P, _u64, _i]),
    "wgml_dequantize_host": (_i, [_i, _P, _P, _u64, _i]),
    "wgml_rng_normal": (_i, [_u64, _P, _u64, _f, _f, _i]),
    "wgml_rng_uniform_f32": (_i, [_u64, _P, _u64]),
    "wgml_rng_uniform_u32": (_i, [_u64, _P, _u64, _u32]),
    "wgml_ctx_set_tuning": (_i, [_P, _i, _i]),
}

# calls whose return value is not a status code
_NON_STATUS = {"wgml_last_error", "wgml_version", "wgml_buf_size", "wgml_quant_matrix_gguf_bytes",
               "wgml_quant_bytes", "wgml_quant_block_elems", "wgml_llama2_launches_per_token",
               "wgml_gpt2_launches_per_token",
               "wgml_tokenizer_vocab_size", "wgml_tokenizer_bos", "wgml_tokenizer_eos",
               "wgml_tokenizer_unk",
               "wgml_gguf_version", "wgml_gguf_alignment", "wgml_gguf_n_metadata",
               "wgml_gguf_n_tensors", "wgml_gguf_find_metadata", "wgml_gguf_find_tensor"}


def _load() -> C.CDLL:
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build it first (python -c 'import __graft_entry__ as g; "
            f"g.build()' or make -C wgml_amd/csrc). There is no CPU fallback.")
    lib = C.CDLL(os.fspath(LIB_PATH))
    for name, (res, args) in PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def check(status: int) -> None:
    if status != OK:
        raise WgmlError(status, lib.wgml_last_error().decode("utf-8", "replace"))


def call(name: str, *args):
    """Calls a status-returning entry point and raises WgmlError on failure."""
    rc = getattr(lib, name)(*args)
    if name in _NON_STATUS:
        return rc
    check(rc)
    return rc
