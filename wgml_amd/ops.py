"""Host-side mirror of wgml's operator surface over the HIP library.

Names and argument meaning follow the reference (`wgml::ops`, `wgcore` tensors):
ops are constructed once per device (`X.from_device(gpu)`), `dispatch` enqueues
work on the context's stream and returns, tensors are views into device
buffers, and only `read()` blocks.  All compute happens in libwgml_hip.so.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np

from . import _lib
from ._lib import AttnParams, RopeConfig, View, WgmlError, call

__all__ = [
    "GpuInstance", "GpuVector", "GpuMatrix", "GpuQuantMatrix", "GemvQuant", "GemmQuant", "Gemv", "Quantization",
    "RmsNorm", "RmsNormConfig", "LayerNorm", "RoPE", "RoPEConfig", "RoPEVariant", "SoftMax",
    "BatchedMultiqueryAttention", "BatchedMultiqueryAttentionParams", "Silu", "UnaryOp",
    "UnaryInplace", "OpAssign", "OpAssignVariant", "Sampler", "quantize", "dequantize_host",
    "quant_bytes",
    "rng_normal", "rng_uniform", "rng_tokens", "WgmlError",
]


def _ptr(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


class GpuInstance:
    """A device + one in-order stream (wgcore `GpuInstance`)."""

    def __init__(self, device: int = 0):
        h = C.c_void_p()
        call("wgml_ctx_create", device, C.byref(h))
        self._h = h

    @property
    def handle(self) -> C.c_void_p:
        return self._h

    def synchronize(self) -> None:
        call("wgml_ctx_synchronize", self._h)

    def stream(self) -> int:
        """The context's HIP stream (a hipStream_t as an integer), on which every call of this
        context enqueues its work in call order."""
        st = C.c_void_p()
        call("wgml_ctx_stream", self._h, C.byref(st))
        return st.value or 0

    # keys of set_tuning (enum WGML_TUNE_* of the C header, same order)
    (TUNE_GEMV_ROWS_PER_WAVE, TUNE_GEMV_WAVES_PER_WG, TUNE_GEMV_WG_PER_CU, TUNE_GEMV_DEPTH,
     TUNE_GEMV_F32_ACTIVATIONS, TUNE_GEMM_K_SPLIT, TUNE_PREFILL_ATTENTION_PER_TOKEN,
     TUNE_ATTN_WIDE_POSITIONS, TUNE_ATTN_SPLITS, TUNE_ATTN_MERGE) = range(10)

    def set_tuning(self, key: int, value: int) -> None:
        """Launch-shape override of this context (0 = heuristic); for sweeps and tests."""
        call("wgml_ctx_set_tuning", self._h, key, value)

    def set_gemm_precision(self, level: int) -> None:
        """Batched products (GemmQuant, Llama2.prefill): 1 = split-f16 operands, results to fp32
        rounding (default); 0 = plain f16 operands, faster, about 3e-4 of a row's magnitude."""
        call("wgml_ctx_set_gemm_precision", self._h, level)

    def info(self):
        name = C.create_string_buffer(128)
        n_cu = C.c_int()
        call("wgml_ctx_info", self._h, name, 128, C.byref(n_cu))
        return name.value.decode(), n_cu.value

    def timer_start(self) -> None:
        call("wgml_timer_start", self._h)

    def timer_stop(self) -> float:
        ms = C.c_float()
        call("wgml_timer_stop", self._h, C.byref(ms))
        return ms.value

    def close(self) -> None:
        if self._h:
            call("wgml_ctx_destroy", self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class GpuVector:
    """An owned f32 device vector (wgcore `GpuVector<f32>`); slicing gives views."""

    def __init__(self, gpu: GpuInstance, length: int, _buf=None, _offset: int = 0,
                 _owner: Optional["GpuVector"] = None, nbytes: Optional[int] = None):
        self.gpu = gpu
        self.len = int(length)
        self.offset = int(_offset)
        self._owner = _owner
        if _buf is None:
            h = C.c_void_p()
            call("wgml_buf_create", gpu.handle, int(nbytes if nbytes is not None else 4 * max(1, length)),
                 C.byref(h))
            self._buf = h
        else:
            self._buf = _buf

    @classmethod
    def init(cls, gpu: GpuInstance, data) -> "GpuVector":
        a = np.ascontiguousarray(data, dtype=np.float32).reshape(-1)
        v = cls(gpu, a.size)
        if a.size:
            call("wgml_buf_upload", v._buf, 0, _ptr(a), a.nbytes)
        return v

    @classmethod
    def uninit(cls, gpu: GpuInstance, length: int) -> "GpuVector":
        return cls(gpu, length)

    @classmethod
    def from_bytes(cls, gpu: GpuInstance, raw: np.ndarray) -> "GpuVector":
        """Uploads arbitrary bytes (e.g. u16 half patterns); `len` counts f32 slots."""
        a = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        v = cls(gpu, a.size // 4, nbytes=max(4, a.size))
        call("wgml_buf_upload", v._buf, 0, _ptr(a), a.nbytes)
        return v

    def view(self) -> View:
        return View(self._buf, self.offset, self.len)

    def rows(self, start: int, count: int) -> "GpuVector":
        """`.rows(start, count)` sub-view (wgcore GpuVector::rows)."""
        return GpuVector(self.gpu, count, _buf=self._buf, _offset=self.offset + start,
                         _owner=self._owner or self)

    def write(self, data) -> None:
        a = np.ascontiguousarray(data, dtype=np.float32).reshape(-1)
        assert a.size == self.len
        call("wgml_buf_upload", self._buf, 4 * self.offset, _ptr(a), a.nbytes)

    def read(self) -> np.ndarray:
        out = np.empty(self.len, dtype=np.float32)
        if self.len:
            call("wgml_buf_download", self._buf, 4 * self.offset, _ptr(out), out.nbytes)
        return out

    def copy_from(self, src: "GpuVector") -> None:
        assert src.len == self.len
        call("wgml_buf_copy", self._buf, 4 * self.offset, src._buf, 4 * src.offset, 4 * self.len)

    def __del__(self):
        try:
            if self._owner is None and self._buf:
                _lib.lib.wgml_buf_destroy(self._buf)
                self._buf = None
        except Exception:
            pass


class GpuMatrix(GpuVector):
    """Column-addressable f32 matrix: column c at [c*nrows, (c+1)*nrows)
    (wgcore `GpuMatrix<f32>` as used for KV caches and embeddings)."""

    def __init__(self, gpu: GpuInstance, nrows: int, ncols: int):
        super().__init__(gpu, nrows * ncols)
        self.nrows, self.ncols = nrows, ncols

    @classmethod
    def init(cls, gpu: GpuInstance, columns: np.ndarray) -> "GpuMatrix":
        """`columns[c]` is column c (shape ncols x nrows, C-contiguous)."""
        a = np.ascontiguousarray(columns, dtype=np.float32)
        m = cls(gpu, a.shape[1], a.shape[0])
        call("wgml_buf_upload", m._buf, 0, _ptr(a), a.nbytes)
        return m

    def column(self, c: int) -> GpuVector:
        return self.rows(c * self.nrows, self.nrows)


class GpuQuantMatrix:
    """`GpuQuantMatrix` (quantized_matrix.rs:9-75): a tagged quantized matrix
    created from GGUF bytes as `GgufTensorData::to_gpu_matrix` does
    (gguf.rs:131-184), minus the fall-back to f32."""

    def __init__(self, gpu: GpuInstance, qtype: int, nrows: int, ncols: int, gguf_bytes):
        raw = np.ascontiguousarray(gguf_bytes).view(np.uint8).reshape(-1)
        expect = _lib.lib.wgml_quant_bytes(qtype, nrows * ncols)
        if expect and raw.size != expect:
            raise ValueError(f"expected {expect} GGUF bytes for {nrows}x{ncols}, got {raw.size}")
        h = C.c_void_p()
        call("wgml_quant_matrix_create", gpu.handle, qtype, nrows, ncols, _ptr(raw), C.byref(h))
        self.gpu, self._h = gpu, h
        self.qtype, self.nrows, self.ncols = qtype, nrows, ncols

    @property
    def handle(self):
        return self._h

    def shape(self):
        t, r, c = C.c_int(), C.c_uint32(), C.c_uint32()
        call("wgml_quant_matrix_shape", self._h, C.byref(t), C.byref(r), C.byref(c))
        return t.value, r.value, c.value

    def gguf_bytes(self) -> int:
        return _lib.lib.wgml_quant_matrix_gguf_bytes(self._h)

    def weight_bound(self) -> float:
        """Upper bound on |w| of the dequantized matrix, from its block scales (the nine
        quantized formats; 0 for f32 matrices): what the batched product checks against its
        limit of 255.875."""
        b = C.c_float()
        call("wgml_quant_matrix_weight_bound", self._h, C.byref(b))
        return b.value

    def __del__(self):
        try:
            if self._h:
                _lib.lib.wgml_quant_matrix_destroy(self._h)
                self._h = None
        except Exception:
            pass


class _Op:
    def __init__(self, gpu: GpuInstance):
        self.gpu = gpu

    @classmethod
    def from_device(cls, gpu: GpuInstance):
        return cls(gpu)


class GemvQuant(_Op):
    """ops/gemv_quant.rs:103-348"""

    def dispatch(self, out: GpuVector, m: GpuQuantMatrix, v: GpuVector) -> None:
        call("wgml_gemv_quant", self.gpu.handle, out.view(), m.handle, v.view())


class GemmQuant(_Op):
    """The product of a quantized matrix with up to 128 vectors at once, on the matrix cores
    (f16 operands, fp32 sums).  The reference multiplies one vector at a time
    (ops/gemv_quant.rs:243-348); this is that product for the tokens of a prompt."""

    MAX_TOKENS = 128

    def dispatch(self, out: GpuVector, m: GpuQuantMatrix, x: GpuVector, n_tokens: int) -> None:
        call("wgml_gemm_quant", self.gpu.handle, out.view(), m.handle, x.view(), n_tokens)


class Gemv(_Op):
    """wgebra `Gemv` on f32 (row-major matrix)."""

    def dispatch(self, out: GpuVector, a: GpuVector, nrows: int, ncols: int, v: GpuVector,
                 transposed: bool = False) -> None:
        call("wgml_gemv_f32", self.gpu.handle, out.view(), a.view(), nrows, ncols, int(transposed),
             v.view())


class Quantization(_Op):
    """ops/quantization.rs: the dequantization kernels."""

    def dequantize(self, out: GpuVector, m: GpuQuantMatrix) -> None:
        call("wgml_dequantize", self.gpu.handle, out.view(), m.handle)

    def f16_to_f32(self, out: GpuVector, halves: GpuVector, offset_bytes: int = 0) -> None:
        call("wgml_f16_to_f32", self.gpu.handle, out.view(), halves._buf, offset_bytes)


@dataclass
class RmsNormConfig:
    nudge_factor: float  # ops/rms_norm.rs:19-21


class RmsNorm(_Op):
    """ops/rms_norm.rs:13-63"""

    def dispatch(self, config: RmsNormConfig, result: GpuVector, value: GpuVector,
                 weight: GpuVector) -> None:
        call("wgml_rms_norm", self.gpu.handle, float(config.nudge_factor), result.view(),
             value.view(), weight.view())


class LayerNorm(_Op):
    """ops/layernorm.rs:13-53"""

    def dispatch(self, out_vec: GpuVector, in_vec: GpuVector) -> None:
        call("wgml_layernorm", self.gpu.handle, out_vec.view(), in_vec.view())


class RoPEVariant:
    Original, Neox = 0, 1  # ops/rope.rs:10-16


@dataclass
class RoPEConfig:
    head_size: int
    kv_dim: int
    pos: int
    base_freq: float  # ops/rope.rs:30-35


class RoPE(_Op):
    """ops/rope.rs:18-76"""

    def dispatch(self, variant: int, config: RoPEConfig, in_out_q: GpuVector,
                 in_out_k: GpuVector) -> None:
        cfg = RopeConfig(config.head_size, config.kv_dim, config.pos, config.base_freq)
        call("wgml_rope", self.gpu.handle, variant, C.byref(cfg), in_out_q.view(), in_out_k.view())


class SoftMax(_Op):
    """ops/softmax.rs:10-49: softmax of every column of an nrows x ncols matrix."""

    def dispatch(self, in_out_mat: GpuVector, nrows: Optional[int] = None, ncols: int = 1,
                 col_stride: Optional[int] = None) -> None:
        nrows = in_out_mat.len if nrows is None else nrows
        col_stride = nrows if col_stride is None else col_stride
        call("wgml_softmax", self.gpu.handle, in_out_mat.view(), nrows, ncols, col_stride)


@dataclass
class BatchedMultiqueryAttentionParams:
    seq_len: int
    kv_dim: int
    kv_mul: int
    n_heads: int
    head_size: int
    pos: int  # ops/batched_multiquery_attention.rs:30-37


class BatchedMultiqueryAttention(_Op):
    """ops/batched_multiquery_attention.rs:20-139"""

    def dispatch(self, params: BatchedMultiqueryAttentionParams, q: GpuVector,
                 key_cache: GpuVector, value_cache: GpuVector, attn: Optional[GpuVector],
                 xb: GpuVector) -> None:
        p = AttnParams(params.seq_len, params.kv_dim, params.kv_mul, params.n_heads,
                       params.head_size, params.pos)
        att = attn.view() if attn is not None else View(None, 0, 0)
        call("wgml_attention", self.gpu.handle, C.byref(p), q.view(), key_cache.view(),
             value_cache.view(), att, xb.view())

    def dispatch_multi(self, params, q, key_cache, value_cache, xb) -> None:
        self.dispatch(params, q, key_cache, value_cache, None, xb)

    def dispatch_with_projection(self, params: BatchedMultiqueryAttentionParams, q: GpuVector,
                                 key_cache: GpuVector, value_cache: GpuVector, xb: GpuVector,
                                 m: "GpuQuantMatrix", out: GpuVector, accumulate: bool = False) -> None:
        """`dispatch_multi` followed by `GemvQuant::dispatch(out, m, xb)` (and the `add_assign`
        into `out` when `accumulate`), the pair of models/llama2/transformer.rs:366-383, as one
        call: the product merges attention's partial results itself where the format allows.
        `xb` is scratch."""
        p = AttnParams(params.seq_len, params.kv_dim, params.kv_mul, params.n_heads,
                       params.head_size, params.pos)
        call("wgml_attention_gemv_quant", self.gpu.handle, C.byref(p), q.view(), key_cache.view(),
             value_cache.view(), xb.view(), m.handle, out.view(), 1 if accumulate else 0)

    def dispatch_noalloc(self, params: BatchedMultiqueryAttentionParams, q: GpuVector,
                         key_cache: GpuVector, value_cache: GpuVector, xb: GpuVector) -> None:
        """`dispatch_multi` through the entry point that allocates nothing: partial results go
        to the library's fixed scratch array (no counterpart in the reference)."""
        p = AttnParams(params.seq_len, params.kv_dim, params.kv_mul, params.n_heads,
                       params.head_size, params.pos)
        call("wgml_attention_noalloc", self.gpu.handle, C.byref(p), q.view(), key_cache.view(),
             value_cache.view(), xb.view())


class Silu(_Op):
    """ops/silu.rs:10-44"""

    def dispatch(self, in_out_h1: GpuVector, in_h2: GpuVector) -> None:
        call("wgml_silu", self.gpu.handle, in_out_h1.view(), in_h2.view())


class UnaryOp:
    """ops/unary.rs:16-38 (same order)."""
    (Abs, Sgn, Neg, Step, Elu, Gelu, GeluQuick, Silu, Tanh, Relu, Sigmoid, HardSigmoid, HardSwish,
     Sqr, Sqrt, Log, LeakyRelu, Clamp, Scale, AddScalar) = range(20)


class UnaryInplace:
    """ops/unary.rs:207-261"""

    def __init__(self, gpu: GpuInstance, op: int):
        self.gpu, self.op = gpu, op

    def dispatch(self, dest: GpuVector, args: Optional[Sequence[float]] = None) -> None:
        a = None
        if args is not None:
            a = (C.c_float * 4)(*(list(args) + [0.0] * (4 - len(args))))
        call("wgml_unary_inplace", self.gpu.handle, self.op, dest.view(), a)


class OpAssignVariant:
    Add, Mul, Copy = 0, 1, 2


class OpAssign:
    """wgebra `OpAssign`: a op= b."""

    def __init__(self, gpu: GpuInstance, variant: int):
        self.gpu, self.variant = gpu, variant

    def dispatch(self, a: GpuVector, b: GpuVector) -> None:
        call("wgml_op_assign", self.gpu.handle, self.variant, a.view(), b.view())


class Sampler:
    """models/sampler.rs: `sample_argmax` on the device (the greedy branch); `sample` is the
    CPU sampler (temperature, top-p) with the random number passed in."""

    def __init__(self, gpu: Optional[GpuInstance] = None, temperature: float = 0.0,
                 topp: float = 0.0):
        self.gpu, self.temperature, self.topp = gpu, temperature, topp

    def sample(self, logits: np.ndarray, coin: float) -> int:
        """Sampler::sample (models/sampler.rs:32-52); `logits` is modified in place."""
        assert logits.dtype == np.float32 and logits.flags.c_contiguous
        out = C.c_uint32()
        call("wgml_sample", _ptr(logits), logits.size, self.temperature, self.topp, coin,
             C.byref(out))
        return out.value

    def sample_argmax(self, logits: GpuVector) -> int:
        out = C.c_uint32()
        call("wgml_argmax", self.gpu.handle, logits.view(), C.byref(out))
        return out.value


# ---- host-side input makers --------------------------------------------------

def quant_bytes(qtype: int, nelems: int) -> int:
    return _lib.lib.wgml_quant_bytes(qtype, nelems)


def dequantize_host(qtype: int, data: np.ndarray, nelems: int, nthreads: int = 0) -> np.ndarray:
    """GGUF bytes (F32 / F16 / Q8_0 / Q4_K / Q6_K) -> f32 values, on the host."""
    src = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
    out = np.empty(nelems, dtype=np.float32)
    call("wgml_dequantize_host", qtype, src.ctypes.data_as(C.c_void_p),
         out.ctypes.data_as(C.c_void_p), nelems, nthreads)
    return out


def quantize(qtype: int, values: np.ndarray, nthreads: int = 0) -> np.ndarray:
    """ggml reference quantizer (Q8_0 / Q4_K / Q6_K) -> GGUF bytes (uint8)."""
    a = np.ascontiguousarray(values, dtype=np.float32).reshape(-1)
    n = quant_bytes(qtype, a.size)
    if n == 0:
        raise WgmlError(_lib.E_UNSUPPORTED, f"cannot quantize {a.size} elements as type {qtype}")
    out = np.empty(n, dtype=np.uint8)
    call("wgml_quantize", qtype, _ptr(a), _ptr(out), a.size, nthreads)
    return out


def rng_normal(seed: int, n: int, mean: float = 0.0, std: float = 1.0,
               nthreads: int = 0) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    call("wgml_rng_normal", seed, _ptr(out), n, mean, std, nthreads)
    return out


def rng_uniform(seed: int, n: int) -> np.ndarray:
    """Uniform f32 in [0, 1): the sampler's coins."""
    out = np.empty(n, dtype=np.float32)
    call("wgml_rng_uniform_f32", seed, _ptr(out), n)
    return out


def rng_tokens(seed: int, n: int, vocab: int) -> np.ndarray:
    out = np.empty(n, dtype=np.uint32)
    call("wgml_rng_uniform_u32", seed, _ptr(out), n, vocab)
    return out
