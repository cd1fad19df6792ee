/*
 * wgml_hip — C ABI of the MI355X (gfx950) batch-1 token-decode path behind
 * dimforge/wgml's operator API.
 *
 * The reference has no FFI layer: its boundary is the Rust API of `wgml::ops`,
 * `wgml::models` and `wgml::quantized_matrix` running on wgpu.  Each entry
 * point below names the reference interface it replaces (paths relative to the
 * reference's `crates/wgml/src/`).  A Rust `wgml-hip-sys` crate would bind
 * exactly these symbols with `extern "C"` declarations.
 *
 * Conventions
 *   - every call returns a status (0 = WGML_OK); wgml_last_error() returns the
 *     message of the last failure on the calling thread;
 *   - handles are opaque, owned by the caller, freed by the matching _destroy;
 *   - a context owns one in-order HIP stream: ops are *enqueued* in program
 *     order and return immediately, like `dispatch()` recording into one
 *     wgpu compute pass.  Only *_download, *_read_*, wgml_argmax, the timers'
 *     stop call and wgml_ctx_synchronize block;
 *   - tensors are f32 *views*: buffer + element offset + length, so an output
 *     may alias a sub-range such as one KV-cache column
 *     (models/llama2/transformer.rs:326-341);
 *   - a context is not thread-safe; use one per thread;
 *   - there is no CPU fallback: without a HIP device wgml_ctx_create fails.
 */
#ifndef WGML_HIP_H
#define WGML_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define WGML_API __attribute__((visibility("default")))

/* ---- status ------------------------------------------------------------ */
enum {
    WGML_OK = 0,
    WGML_E_INVALID = 1,     /* bad argument / shape mismatch (the reference panics) */
    WGML_E_UNSUPPORTED = 2, /* quantization tag or op outside this path */
    WGML_E_HIP = 3,         /* a HIP runtime call failed */
    WGML_E_NO_DEVICE = 4,   /* no usable gfx950 device */
    WGML_E_OOM = 5,
};

WGML_API const char *wgml_last_error(void);
WGML_API const char *wgml_version(void);

/* ---- quantization tags (GGUF tensor-type ids, gguf.rs:70-103) ------------ */
enum {
    WGML_F32 = 0,
    WGML_F16 = 1,
    WGML_Q4_0 = 2,
    WGML_Q4_1 = 3,
    WGML_Q5_0 = 6,
    WGML_Q5_1 = 7,
    WGML_Q8_0 = 8,
    WGML_Q4_K = 12,
    WGML_Q5_K = 13,
    WGML_Q6_K = 14,
    WGML_Q8_K = 15,
};

typedef struct wgml_ctx wgml_ctx;
typedef struct wgml_buf wgml_buf;
typedef struct wgml_qmat wgml_qmat;

/* An f32 vector view: GpuVectorView<f32> (wgcore), `.column()`, `.rows()`. */
typedef struct {
    wgml_buf *buf;
    uint64_t offset; /* in f32 elements */
    uint32_t len;    /* in f32 elements */
} wgml_view;

/* ---- context: GpuInstance::new + every `X::from_device` ------------------ */
WGML_API int wgml_ctx_create(int device, wgml_ctx **out);
WGML_API int wgml_ctx_destroy(wgml_ctx *ctx);
WGML_API int wgml_ctx_synchronize(wgml_ctx *ctx);
/* The HIP stream (a hipStream_t) on which every call of this context enqueues its work, in
 * call order: the counterpart of the wgpu queue / compute pass the reference's dispatch calls
 * record into (e.g. ops/gemv_quant.rs:243-250).  For callers that order HIP work of their own
 * against the library's, or capture its launches into a HIP graph. */
WGML_API int wgml_ctx_stream(wgml_ctx *ctx, void **stream);
/* Launch-shape overrides of one context, for kernel sweeps and for tests that must reach every
 * kernel variant; value 0 restores the heuristic.  The reference has compile-time constants in
 * this role (USE_OPTIMIZED, ops/gemv_quant.rs:15; USE_MATMUL_ATTN, models/llama2/transformer.rs:444).
 * Results stay within the documented tolerances for every setting.  Values outside a key's range
 * are refused.  A model re-records its decode step the next time it runs after a change (launch
 * sequences recorded under other settings are dropped). */
enum {
    WGML_TUNE_GEMV_ROWS_PER_WAVE = 0,        /* 1 or 2 rows of a quantized GEMV per wave and step */
    WGML_TUNE_GEMV_WAVES_PER_WG,             /* 4, 8 or 16; 12 for the multi-matrix launches only
                                                (single-matrix launches then use 16) */
    WGML_TUNE_GEMV_WG_PER_CU,                /* cap on resident workgroups per compute unit, 1..8 */
    WGML_TUNE_GEMV_DEPTH,                    /* weight tiles in flight per wave, 1..4 */
    WGML_TUNE_GEMV_F32_ACTIVATIONS,          /* 1: fp32 activations instead of 16-bit block fixed point */
    WGML_TUNE_GEMM_K_SPLIT,                  /* 1..8 workgroups share the K range of a batched product */
    WGML_TUNE_PREFILL_ATTENTION_PER_TOKEN,   /* 1: one workgroup per (head, token) in the prompt pass */
    WGML_TUNE_ATTN_WIDE_POSITIONS,           /* decode attention planned for up to this many positions
                                                (at most 2^20) runs as one workgroup per head group,
                                                without partial results */
    WGML_TUNE_ATTN_SPLITS,                   /* workgroups that share the positions of a head group, 2..64 */
    WGML_TUNE_ATTN_MERGE,                    /* attention followed by a quantized GEMV on its output
                                                (wgml_attention_gemv_quant, the decoders' layers): 1 = the
                                                GEMV merges attention's partial results itself while it
                                                stages its input (up to 16 per head) instead of a merge
                                                launch.  Off by default: every workgroup of the GEMV then
                                                reads all partial results, which costs more than the launch */
    WGML_TUNE_COUNT
};
WGML_API int wgml_ctx_set_tuning(wgml_ctx *ctx, int key, int value);
/* Device name and compute-unit count (diagnostics). */
WGML_API int wgml_ctx_info(wgml_ctx *ctx, char *name, size_t name_len, int *n_cu);

/* GPU timestamps over the context's stream (wgcore GpuTimestamps as used by
 * wgml-bench/src/main.rs:201,225-244).  stop() blocks and returns milliseconds. */
WGML_API int wgml_timer_start(wgml_ctx *ctx);
WGML_API int wgml_timer_stop(wgml_ctx *ctx, float *ms);

/* ---- buffers: GpuVector / GpuMatrix / GpuScalar -------------------------- */
WGML_API int wgml_buf_create(wgml_ctx *ctx, uint64_t bytes, wgml_buf **out); /* ::uninit */
WGML_API int wgml_buf_destroy(wgml_buf *buf);
WGML_API uint64_t wgml_buf_size(const wgml_buf *buf);
WGML_API int wgml_buf_upload(wgml_buf *buf, uint64_t offset_bytes, const void *src,
                             uint64_t bytes); /* ::init / queue.write_buffer */
WGML_API int wgml_buf_download(wgml_buf *buf, uint64_t offset_bytes, void *dst,
                               uint64_t bytes); /* ::read / read_to (blocks) */
WGML_API int wgml_buf_copy(wgml_buf *dst, uint64_t dst_offset_bytes, const wgml_buf *src,
                           uint64_t src_offset_bytes, uint64_t bytes); /* copy_from{,_view} */
WGML_API int wgml_buf_zero(wgml_buf *buf);

/* ---- quantized matrices: GpuQuantMatrix (quantized_matrix.rs:9-75) and
 *      GgufTensorData::to_gpu_matrix (gguf.rs:131-184) ---------------------- *
 * `gguf_bytes` is the tensor exactly as stored in a GGUF file: row-major,
 * nrows rows of ncols/elems_per_block blocks.  Every block format the reference keeps
 * quantized on the GPU (gguf.rs:172-182) stays quantized here: WGML_Q8_0 and WGML_Q6_K are
 * re-laid out into aligned planes on the device (same bytes in total, see the layout
 * notes in csrc/common.h), WGML_Q4_K, WGML_Q4_0, WGML_Q4_1, WGML_Q5_0, WGML_Q5_1,
 * WGML_Q5_K and WGML_Q8_K keep the GGUF bytes unchanged; the values are those of
 * Block*::dequantize in every case.  WGML_F16 is expanded to f32 on the device at
 * creation, as to_gpu_matrix does (the matrix then reports WGML_F32).  Other tags give
 * WGML_E_UNSUPPORTED.  Unlike the reference there is no pairing rule (ncols % 64 /
 * % 512): any ncols that is a multiple of the block length stays quantized. */
WGML_API int wgml_quant_matrix_create(wgml_ctx *ctx, int type, uint32_t nrows, uint32_t ncols,
                                      const void *gguf_bytes, wgml_qmat **out);
WGML_API int wgml_quant_matrix_destroy(wgml_qmat *m);
WGML_API int wgml_quant_matrix_shape(const wgml_qmat *m, int *type, uint32_t *nrows,
                                     uint32_t *ncols); /* GpuQuantMatrix::shape */
/* Size of the tensor in GGUF bytes (the algorithmic weight traffic of one GEMV). */
WGML_API uint64_t wgml_quant_matrix_gguf_bytes(const wgml_qmat *m);
/* An upper bound on the magnitude of the matrix's dequantized weights, computed on the device
 * when the matrix is created (Q8_0 / Q4_K / Q6_K; 0 for other formats; infinity when a block
 * scale is NaN or infinite).  The reference has no counterpart: it is what decides whether the
 * batched product (wgml_gemm_quant) takes the matrix. */
WGML_API int wgml_quant_matrix_weight_bound(const wgml_qmat *m, float *bound);

/* Host helpers (no device needed): bytes of `nelems` elements in a format
 * (0 if unsupported / not a whole number of blocks). */
WGML_API uint64_t wgml_quant_bytes(int type, uint64_t nelems);
WGML_API uint32_t wgml_quant_block_elems(int type); /* QuantizedValue::DEQUANTIZED_LEN per GGUF block */

/* ---- ops ------------------------------------------------------------------ */

/* GemvQuant::dispatch (ops/gemv_quant.rs:243-348): out = m * v, fp32 accumulate.
 * out.len == nrows, v.len == ncols. */
WGML_API int wgml_gemv_quant(wgml_ctx *ctx, wgml_view out, const wgml_qmat *m, wgml_view v);

/* The same product for n_tokens <= 128 vectors at once, on the matrix cores:
 * out[t] = m * x[t], with x n_tokens x ncols and out n_tokens x nrows, both row-major.
 * No counterpart in the reference, which multiplies one vector at a time
 * (GemvQuant::dispatch above); it is the building block of wgml_llama2_prefill.
 * The weights are expanded with the reference's dequantization arithmetic (fp32).
 * Precision (wgml_ctx_set_gemm_precision): level 1, the default, feeds the matrix
 * cores pairs of f16 numbers per operand (high part + low part), three MFMAs per
 * product term group, fp32 sums: results agree with n_tokens calls of
 * wgml_gemv_quant to fp32 rounding (about 1e-6 of a row's magnitude).  Level 0 rounds
 * weights and vectors to f16 once: 1.4x faster, about 3e-4 of a row's magnitude
 * (up to 1.4e-3 for single elements).  m: any of the nine quantized block formats
 * (Q8_0, Q4_K, Q6_K, Q4_0, Q4_1, Q5_0, Q5_1, Q5_K, Q8_K); not F32 / F16.
 * Vectors of any magnitude are taken (scaled per vector by a power of two); the
 * dequantized weights must not exceed 255.875 in magnitude (they pass through f16 times 2^8,
 * and 65504 is the largest finite f16): a bound on the largest weight is computed when the
 * matrix is created, and a matrix whose bound is larger is refused with WGML_E_UNSUPPORTED
 * (wgml_gemv_quant takes any value;
 * wgml_llama2_prefill steps through the prompt token by token for such a model). */
WGML_API int wgml_ctx_set_gemm_precision(wgml_ctx *ctx, int level);
WGML_API int wgml_gemm_quant(wgml_ctx *ctx, wgml_view out, const wgml_qmat *m, wgml_view x,
                             uint32_t n_tokens);

/* Quantization shader `dequantize_*` (ops/quantization.wgsl, exercised by
 * ops/quantization.rs:37-408) == Block*::dequantize (quantization.rs): writes
 * the nrows*ncols f32 values, row-major, bit-exact with the CPU twin. */
WGML_API int wgml_dequantize(wgml_ctx *ctx, wgml_view out, const wgml_qmat *m);

/* BlockF16::dequantize (quantization.rs:16-24): n IEEE half bit patterns
 * (uint16, at `in_offset_bytes` of `in`) -> f32. */
WGML_API int wgml_f16_to_f32(wgml_ctx *ctx, wgml_view out, const wgml_buf *in,
                             uint64_t in_offset_bytes);

/* wgebra Gemv / GemvTr on f32 (call sites ops/gemv_quant.rs:119,305,
 * models/gpt2/transformer.rs:243-476).  `a` is row-major nrows x ncols;
 * transposed != 0 computes out = a^T v (out.len == ncols, v.len == nrows). */
WGML_API int wgml_gemv_f32(wgml_ctx *ctx, wgml_view out, wgml_view a, uint32_t nrows,
                           uint32_t ncols, int transposed, wgml_view v);

/* RmsNorm::dispatch (ops/rms_norm.rs:24-53); eps = RmsNormConfig.nudge_factor. */
WGML_API int wgml_rms_norm(wgml_ctx *ctx, float eps, wgml_view out, wgml_view x, wgml_view w);

/* LayerNorm::dispatch (ops/layernorm.rs:18-41): no affine, eps 1e-5. */
WGML_API int wgml_layernorm(wgml_ctx *ctx, wgml_view out, wgml_view x);

enum { WGML_ROPE_ORIGINAL = 0, WGML_ROPE_NEOX = 1 }; /* ops/rope.rs:10-16 */
typedef struct {
    uint32_t head_size, kv_dim, pos;
    float base_freq;
} wgml_rope_config; /* ops/rope.rs:30-35 */
/* RoPE::dispatch (ops/rope.rs:38-76): rotates q (all pairs) and k (pairs below
 * kv_dim) in place.  Errors where the reference asserts: odd lengths, q shorter
 * than k. */
WGML_API int wgml_rope(wgml_ctx *ctx, int variant, const wgml_rope_config *cfg, wgml_view q,
                       wgml_view k);

/* SoftMax::dispatch (ops/softmax.rs:18-30): independent softmax of each of the
 * ncols columns of length nrows; column j starts at offset + j*col_stride. */
WGML_API int wgml_softmax(wgml_ctx *ctx, wgml_view mat, uint32_t nrows, uint32_t ncols,
                          uint32_t col_stride);

typedef struct {
    uint32_t seq_len, kv_dim, kv_mul, n_heads, head_size, pos;
} wgml_attn_params; /* ops/batched_multiquery_attention.rs:30-37 */
/* BatchedMultiqueryAttention::{dispatch, dispatch_multi}
 * (ops/batched_multiquery_attention.rs:55-139).  key/value cache: position t at
 * [t*kv_dim, (t+1)*kv_dim).  If att.buf != NULL the normalised weights of head
 * h are also written to att[h*seq_len + t] as `dispatch` does; pass a null
 * view to skip them (as `dispatch_multi`, whose scratch layout is private). */
WGML_API int wgml_attention(wgml_ctx *ctx, const wgml_attn_params *p, wgml_view q,
                            wgml_view key_cache, wgml_view value_cache, wgml_view att,
                            wgml_view xb);
/* The pair BatchedMultiqueryAttention::dispatch_multi + GemvQuant::dispatch that every decoder
 * layer runs (models/llama2/transformer.rs:366-383, models/gpt2/transformer.rs:355-395):
 * out = m * attention(q, caches), or out += ... when accumulate != 0 (the add_assign that
 * follows in the reference).  m is n x (n_heads * head_size).  The two launches run as they
 * would on their own; with WGML_TUNE_ATTN_MERGE = 1 and m in Q8_0 / Q4_K / Q6_K the
 * attention launch leaves per-workgroup partial results and the product merges them while it
 * stages its input (no merge launch, `xb` not written).  xb: n_heads * head_size floats of
 * scratch whose contents after the call are unspecified. */
WGML_API int wgml_attention_gemv_quant(wgml_ctx *ctx, const wgml_attn_params *p, wgml_view q,
                                       wgml_view key_cache, wgml_view value_cache, wgml_view xb,
                                       const wgml_qmat *m, wgml_view out, int accumulate);
/* No counterpart in the reference.  wgml_attention without the `att` output, for callers
 * that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): the partial results of the position-split launches live
 * in a fixed 2 MiB array inside the library (one copy per GPU, held until the process ends)
 * instead of a workspace from hipMalloc, and the call allocates and frees nothing.  A shape
 * whose partial results (n_heads * workgroups per head * (head_size rounded up to 64, + 2)
 * floats; 1.06 MB for 32 heads of 128 at 8192 positions) exceed the array is refused with
 * WGML_E_UNSUPPORTED.  Results equal
 * wgml_attention's.  Every call on a GPU uses that GPU's one array: calls that overlap on
 * one GPU (two contexts, two streams) race.  The array's address is looked up when the context
 * is created; the call itself only launches kernels, so it may be recorded under stream capture
 * (wgml_ctx_stream) and replayed. */
WGML_API int wgml_attention_noalloc(wgml_ctx *ctx, const wgml_attn_params *p, wgml_view q,
                                    wgml_view key_cache, wgml_view value_cache, wgml_view xb);

/* Silu::dispatch (ops/silu.rs:18-34): h1 = h2 * h1 / (1 + exp(-h1)). */
WGML_API int wgml_silu(wgml_ctx *ctx, wgml_view h1, wgml_view h2);

/* UnaryOp (ops/unary.rs:16-38), same order.  Each follows the shader (ops/unary.wgsl); where the
 * reference's CPU twin differs from its shader the shader wins, this being the device op:
 * WGML_UNARY_SGN is WGSL `sign` (ops/unary.wgsl:27): 0 at +0 and -0 (and for NaN), whereas
 * UnaryOp::eval's f32::signum (ops/unary.rs:90) gives +1 / -1 at the two zeros. */
enum {
    WGML_UNARY_ABS = 0, WGML_UNARY_SGN, WGML_UNARY_NEG, WGML_UNARY_STEP, WGML_UNARY_ELU,
    WGML_UNARY_GELU, WGML_UNARY_GELU_QUICK, WGML_UNARY_SILU, WGML_UNARY_TANH, WGML_UNARY_RELU,
    WGML_UNARY_SIGMOID, WGML_UNARY_HARD_SIGMOID, WGML_UNARY_HARD_SWISH, WGML_UNARY_SQR,
    WGML_UNARY_SQRT, WGML_UNARY_LOG, WGML_UNARY_LEAKY_RELU, WGML_UNARY_CLAMP, WGML_UNARY_SCALE,
    WGML_UNARY_ADD_SCALAR,
};
/* UnaryInplace::dispatch (ops/unary.rs:207-261); args may be NULL for ops
 * without arguments. */
WGML_API int wgml_unary_inplace(wgml_ctx *ctx, int op, wgml_view x, const float *args4);

enum { WGML_ASSIGN_ADD = 0, WGML_ASSIGN_MUL = 1, WGML_ASSIGN_COPY = 2 };
/* wgebra OpAssign (call sites models/llama2/transformer.rs:293,344-353,383,406;
 * models/gpt2/transformer.rs:277-452): a op= b elementwise. */
WGML_API int wgml_op_assign(wgml_ctx *ctx, int op, wgml_view a, wgml_view b);

/* Sampler::sample_argmax (models/sampler.rs:54-56): first index of the
 * maximum, computed on the device; blocks and returns it. */
WGML_API int wgml_argmax(wgml_ctx *ctx, wgml_view logits, uint32_t *out_index);

/* ---- Llama-family model: Llama2 / Llama2State / Llama2Weights ------------- */
typedef struct {
    uint32_t dim, hidden_dim, n_layers, n_q_heads, n_kv_heads, vocab_size, seq_len;
    float rope_base_freq, rms_norm_eps;
} wgml_llama2_config; /* models/llama2/cpu.rs:46-67 */

enum { WGML_MODEL_LLAMA = 0, WGML_MODEL_QWEN2 = 1 }; /* models/llama2/mod.rs:13-33 */

enum { /* matrices of Llama2LayerWeights / Llama2Weights (transformer.rs:128-148) */
    WGML_LLAMA2_ATTN_Q = 0, WGML_LLAMA2_ATTN_K, WGML_LLAMA2_ATTN_V, WGML_LLAMA2_ATTN_OUTPUT,
    WGML_LLAMA2_FFN_GATE, WGML_LLAMA2_FFN_UP, WGML_LLAMA2_FFN_DOWN,
    WGML_LLAMA2_OUTPUT, /* layer ignored */
};
enum { /* f32 vectors */
    WGML_LLAMA2_ATTN_NORM = 0, WGML_LLAMA2_FFN_NORM,
    WGML_LLAMA2_ATTN_Q_BIAS, WGML_LLAMA2_ATTN_K_BIAS, WGML_LLAMA2_ATTN_V_BIAS,
    WGML_LLAMA2_OUTPUT_NORM, /* layer ignored */
};

typedef struct wgml_llama2 wgml_llama2;

/* Llama2::new + Llama2State::new (models/llama2/transformer.rs:47-105,283-296):
 * allocates activations and the per-layer f32 KV caches (kv_dim x seq_len). */
WGML_API int wgml_llama2_create(wgml_ctx *ctx, const wgml_llama2_config *cfg, int model_type,
                                wgml_llama2 **out);
WGML_API int wgml_llama2_destroy(wgml_llama2 *m);
/* Llama2Weights fields (models/llama2/transformer.rs:151-268).  The model
 * borrows the matrix; it must outlive the model.  Shapes are checked. */
WGML_API int wgml_llama2_set_matrix(wgml_llama2 *m, int which, uint32_t layer,
                                    const wgml_qmat *mat);
WGML_API int wgml_llama2_set_vector(wgml_llama2 *m, int which, uint32_t layer, const float *host,
                                    uint32_t len);
/* token_embd: f32, dim x vocab, token t at [t*dim, (t+1)*dim)
 * (models/llama2/transformer.rs:239-242). */
WGML_API int wgml_llama2_set_token_embd(wgml_llama2 *m, const float *host);
/* One decode step: ChatLlama2::forward_logits minus the read-back
 * (wgml-chat/src/chat_llama2.rs:155-213) = embedding copy + Llama2::dispatch
 * (models/llama2/transformer.rs:298-431).  Enqueues and returns. */
WGML_API int wgml_llama2_forward(wgml_llama2 *m, uint32_t token, uint32_t pos);
/* logits_readback.read_to (chat_llama2.rs:216-220): blocks. */
WGML_API int wgml_llama2_read_logits(wgml_llama2 *m, float *host_out);
/* The token loop of ChatLlama2::forward + sample_next_token with temperature 0
 * (chat_llama2.rs:51-153, wgml-chat/src/sampler.rs:91-111): positions
 * 0..n_total-1; position p consumes prompt[p] while p < n_prompt, else the
 * arg-max of the previous step.  out_tokens[p] receives the arg-max after
 * position p (n_total entries).  Sampling and the loop bookkeeping run on the
 * device: one recorded step (a HIP graph) is replayed per token and the host
 * synchronises once, at the end. */
WGML_API int wgml_llama2_generate_greedy(wgml_llama2 *m, const uint32_t *prompt,
                                         uint32_t n_prompt, uint32_t n_total,
                                         uint32_t *out_tokens);
/* As above from an arbitrary start position with the KV cache already filled
 * for positions < start_pos; first consumed token is `first_token`. */
WGML_API int wgml_llama2_decode_greedy(wgml_llama2 *m, uint32_t first_token, uint32_t start_pos,
                                       uint32_t n_steps, uint32_t *out_tokens);
/* Records, ahead of time, the steps that the token loops replay for positions
 * start_pos .. start_pos + n_steps - 1 (one capture per range of positions, limits 256, 512,
 * 1024, ...: what the first run through such a range would otherwise do before its first
 * launch, a few milliseconds per range).  No counterpart in the reference, which has nothing
 * to record; KV caches and logits are left as they were.  Without graphs
 * (WGML_DISABLE_GRAPHS) it only reserves the attention workspace. */
WGML_API int wgml_llama2_record_steps(wgml_llama2 *m, uint32_t start_pos, uint32_t n_steps);
/* The same loop with a blocking read-back of the sampled token after every
 * step, as the reference's chat loop does (chat_llama2.rs:205-220). */
WGML_API int wgml_llama2_decode_greedy_sync(wgml_llama2 *m, uint32_t first_token,
                                            uint32_t start_pos, uint32_t n_steps,
                                            uint32_t *out_tokens);
/* Batched prompt pass ("prefill").  No counterpart in the reference, which feeds the
 * prompt through the single-token step one position at a time with the sampled
 * token overridden (chat_llama2.rs:155-228, sampler.rs:102-107); this produces the
 * state those n_tokens steps leave behind -- KV-cache rows start_pos ..
 * start_pos + n_tokens - 1 of every layer and the logits of the last token (read
 * them with wgml_llama2_read_logits) -- with every matrix-vector product of the
 * step replaced by one product with up to 128 token vectors on the matrix cores
 * (wgml_gemm_quant; longer prompts go through in runs of 128).  The layer matrices
 * are multiplied at the precision set with wgml_ctx_set_gemm_precision (default:
 * to fp32 rounding); norms, RoPE, attention and the output matrix are fp32 as in
 * the step, so with the default the logits agree with the step-by-step pass as two
 * fp32 implementations do (2e-4 of their range is the bound the tests use); with
 * level 0 a product is within about 3e-4 and a whole model adds that up (3e-3 of
 * the logits' range on 2-layer models, 6e-3 on the 32-layer 7B shape).  The batched
 * products exist for the nine quantized block formats: a model with a layer matrix that is
 * F32 / F16, or whose weights exceed what the products take (see wgml_gemm_quant), takes the
 * prompt one step per token, as the reference does.
 * Enqueues and returns. */
WGML_API int wgml_llama2_prefill(wgml_llama2 *m, const uint32_t *tokens, uint32_t n_tokens,
                                 uint32_t start_pos);
/* wgml_llama2_prefill of the prompt at position 0 followed by greedy decoding:
 * out_tokens[0] is the arg-max after the last prompt token, out_tokens[i] the
 * arg-max after out_tokens[i-1] was consumed (n_new entries): the tokens
 * wgml_llama2_generate_greedy returns from index n_prompt - 1 on. */
WGML_API int wgml_llama2_prefill_decode_greedy(wgml_llama2 *m, const uint32_t *prompt,
                                               uint32_t n_prompt, uint32_t n_new,
                                               uint32_t *out_tokens);
/* Direct KV-cache access (tests; pre-filled long-context runs). which: 0 = key,
 * 1 = value; `n_pos` positions starting at `first_pos`, kv_dim floats each. */
WGML_API int wgml_llama2_kv_upload(wgml_llama2 *m, uint32_t layer, int which, uint32_t first_pos,
                                   uint32_t n_pos, const float *host);
WGML_API int wgml_llama2_kv_download(wgml_llama2 *m, uint32_t layer, int which,
                                     uint32_t first_pos, uint32_t n_pos, float *host);
/* Number of kernel launches one forward enqueues (diagnostics). */
WGML_API int wgml_llama2_launches_per_token(const wgml_llama2 *m);
/* 0: one launch per reference op (mirrors Llama2::dispatch one to one);
 * 1: bias and residual adds folded into the GEMV epilogues; 2: also every
 * RMSNorm folded into the GEMVs that consume it; 3 (default): also Q, K and V
 * (with bias, RoPE and the KV-cache write) in one launch and gate and up (with
 * the SiLU gating) in one launch.  All levels give the same results to fp32
 * rounding. */
WGML_API int wgml_llama2_set_fusion(wgml_llama2 *m, int level);

/* ---- GPT-2: Gpt2 / Gpt2State / Gpt2Weights -------------------------------- */
typedef struct {
    uint32_t n_vocab, n_seq, n_embd, n_head, n_layer, ff_len, attn_b;
} wgml_gpt2_params; /* models/gpt2/cpu.rs:18-33 */

enum { /* matrices (models/gpt2/transformer.rs:72-106) */
    WGML_GPT2_ATTN_W = 0, WGML_GPT2_ATTN_PROJ_W, WGML_GPT2_MLP_FC_W, WGML_GPT2_MLP_PROJ_W,
    WGML_GPT2_LM_HEAD, /* layer ignored */
};
enum { /* f32 vectors */
    WGML_GPT2_LN_1_G = 0, WGML_GPT2_LN_1_B, WGML_GPT2_LN_2_G, WGML_GPT2_LN_2_B,
    WGML_GPT2_ATTN_B, WGML_GPT2_ATTN_PROJ_B, WGML_GPT2_MLP_FC_B, WGML_GPT2_MLP_PROJ_B,
    WGML_GPT2_LN_F_G, WGML_GPT2_LN_F_B, /* layer ignored */
};

typedef struct wgml_gpt2 wgml_gpt2;

/* Gpt2::new + Gpt2State::new (+ the per-layer KV caches of Gpt2LayerWeights,
 * models/gpt2/transformer.rs:27-57,86-87,252-263). */
WGML_API int wgml_gpt2_create(wgml_ctx *ctx, const wgml_gpt2_params *p, wgml_gpt2 **out);
WGML_API int wgml_gpt2_destroy(wgml_gpt2 *m);
WGML_API int wgml_gpt2_set_matrix(wgml_gpt2 *m, int which, uint32_t layer, const wgml_qmat *mat);
WGML_API int wgml_gpt2_set_vector(wgml_gpt2 *m, int which, uint32_t layer, const float *host,
                                  uint32_t len);
/* wte: n_embd x n_vocab, wpe: n_embd x n_seq, column c at [c*n_embd ..]. */
WGML_API int wgml_gpt2_set_embeddings(wgml_gpt2 *m, const float *wte, const float *wpe);
/* Gpt2::dispatch (models/gpt2/transformer.rs:265-477). */
WGML_API int wgml_gpt2_forward(wgml_gpt2 *m, uint32_t token, uint32_t pos);
WGML_API int wgml_gpt2_read_logits(wgml_gpt2 *m, float *host_out);
/* ChatGpt2::forward's loop with greedy sampling (wgml-chat/src/chat_gpt2.rs:43-151). */
WGML_API int wgml_gpt2_generate_greedy(wgml_gpt2 *m, const uint32_t *prompt, uint32_t n_prompt,
                                       uint32_t n_total, uint32_t *out_tokens);
/* As wgml_llama2_record_steps, for positions 0 .. n_total - 1. */
WGML_API int wgml_gpt2_record_steps(wgml_gpt2 *m, uint32_t n_total);
/* 0: layernorm, GELU and the q/k/v copies are launches of their own and the token
 * loop reads every token back (mirrors Gpt2::dispatch and chat_gpt2.rs one to
 * one); 1 (default): LayerNorm folded into the GEMV that consumes it, bias /
 * residual / GELU into GEMV epilogues, k and v written straight into their cache
 * columns, and the token loop replays one recorded step per token.  Same results
 * to fp32 rounding. */
WGML_API int wgml_gpt2_set_fusion(wgml_gpt2 *m, int level);
/* Number of kernel launches of one decode step (diagnostics). */
WGML_API int wgml_gpt2_launches_per_token(const wgml_gpt2 *m);

/* ---- measurement: wgml-bench's bench_gemv (wgml-bench/src/main.rs:187-250) ---- *
 * Enqueues out = mats[i % n_mats] * v for i in 0..iters back to back between two
 * GPU timestamps and returns the elapsed milliseconds.  Rotating over several
 * matrices keeps the weights out of the last-level cache.  use_graph != 0
 * records the launches into a HIP graph first, so host launch time is not
 * part of the measurement. */
WGML_API int wgml_bench_gemv_quant(wgml_ctx *ctx, const wgml_qmat *const *mats, uint32_t n_mats,
                                   wgml_view out, wgml_view v, uint32_t iters, int use_graph,
                                   float *total_ms);

/* The machine's own ceiling for such a chain of launches (no counterpart in the reference):
 * `iters` launches of a kernel that only reads, with the access pattern of the Q4_K GEMV
 * (rows of 4096 columns = 2304 bytes, a wave per row, one 64-element tile per lane in
 * flight, one workgroup of 16 waves per compute unit), each launch over its own `nrows` rows
 * of a 1.5 GB pool that the call allocates and frees.  nrows 4096 / 11008 / 22016 / 46400 read
 * 9.4 / 25.4 / 50.7 / 106.9 MB per launch.  Returns the elapsed milliseconds between two GPU
 * timestamps; use_graph != 0 records the launches into a HIP graph first.  Time per launch as a
 * function of the bytes gives what a launch boundary costs and what loads sustain. */
WGML_API int wgml_bench_read_chain(wgml_ctx *ctx, uint32_t nrows, uint32_t iters, int use_graph,
                                   float *total_ms);

/* The same loop for the fused launches of the decoder: launch i covers the
 * `njobs` (1..3) matrices a[(i % nsets) * njobs + j], all consuming `v` (RMS-
 * normalised with `norm_w` first when norm_w->buf is non-null), job j writing
 * out[j * stride ..].  modes[j]: 0 plain rows, 1 adjacent row pairs rotated as by
 * RoPE at position 0 with head size 128, 2 SiLU-gated: b[...] holds the `up`
 * matrix that goes with the `gate` matrix in a[...] (null entries otherwise).
 * These are the launches Llama2::dispatch's Q/K/V and gate/up GEMVs
 * (models/llama2/transformer.rs:261-374) are folded into. */
WGML_API int wgml_bench_gemv_fused(wgml_ctx *ctx, const wgml_qmat *const *a,
                                   const wgml_qmat *const *b, const int *modes, uint32_t njobs,
                                   uint32_t nsets, wgml_view out, uint32_t stride, wgml_view v,
                                   const wgml_view *norm_w, uint32_t iters, float *total_ms);

/* The same loop for the decode attention of one layer (BatchedMultiqueryAttention::dispatch,
 * ops/batched_multiquery_attention.rs:99-136): launch i reads the KV caches of set i % n_sets
 * (seq_len x kv_dim each), the position p->pos comes from device memory as in a recorded decode
 * step, and the launch grid is the one a recorded step planned for `plan_positions` positions
 * (p->pos < plan_positions <= p->seq_len) would use. */
WGML_API int wgml_bench_attention(wgml_ctx *ctx, const wgml_attn_params *p, uint32_t plan_positions,
                                  wgml_view q, const wgml_view *key_caches,
                                  const wgml_view *value_caches, uint32_t n_sets, wgml_view xb,
                                  uint32_t iters, float *total_ms);

/* ---- tokenizers (host only) ------------------------------------------------ *
 * The vocabulary is handed over as one block of UTF-8 bytes plus n + 1 offsets
 * (token i is bytes offsets[i] .. offsets[i+1]), the way the string arrays
 * `tokenizer.ggml.tokens` / `tokenizer.ggml.merges` lie in a GGUF file.
 * encode/decode follow the two-call pattern: *n_out is the full length, at most
 * `cap` elements are written (out / buf may be NULL with cap 0). */
typedef struct wgml_tokenizer wgml_tokenizer;
/* LlamaTokenizer::from_gguf (models/llama2/tokenizer.rs:23-51): tokens, scores
 * (`tokenizer.ggml.scores`) and the bos / eos / unknown ids. */
WGML_API int wgml_llama_tokenizer_create(const char *tokens, const uint64_t *offsets,
                                         uint32_t n_tokens, const float *scores, uint32_t bos,
                                         uint32_t eos, uint32_t unk, wgml_tokenizer **out);
/* Gpt2Tokenizer::from_gguf (models/gpt2/tokenizer.rs:54-95): tokens and the ranked
 * merges ("first second" per entry). */
WGML_API int wgml_gpt2_tokenizer_create(const char *tokens, const uint64_t *token_offsets,
                                        uint32_t n_tokens, const char *merges,
                                        const uint64_t *merge_offsets, uint32_t n_merges,
                                        uint32_t bos, uint32_t eos, wgml_tokenizer **out);
WGML_API int wgml_tokenizer_destroy(wgml_tokenizer *t);
/* eos() / bos() / unk() and bos_str() / eos_str() (llama2/tokenizer.rs:53-71,
 * gpt2/tokenizer.rs:97-152): the ids, and the string of any id. */
WGML_API uint32_t wgml_tokenizer_vocab_size(const wgml_tokenizer *t);
WGML_API uint32_t wgml_tokenizer_bos(const wgml_tokenizer *t);
WGML_API uint32_t wgml_tokenizer_eos(const wgml_tokenizer *t);
WGML_API uint32_t wgml_tokenizer_unk(const wgml_tokenizer *t);
WGML_API int wgml_tokenizer_token(const wgml_tokenizer *t, uint32_t id, const char **str,
                                  uint64_t *len);
/* LlamaTokenizer::encode(text, bos, eos) (llama2/tokenizer.rs:73-166).  Where the
 * reference panics (nothing to merge: empty text without bos; a fallback byte id
 * beyond the vocabulary) this returns WGML_E_INVALID. */
WGML_API int wgml_llama_tokenizer_encode(const wgml_tokenizer *t, const char *text,
                                         uint64_t text_len, int bos, int eos, uint32_t *out,
                                         uint64_t cap, uint64_t *n_out);
/* LlamaTokenizer::decode(prev_token, token) (llama2/tokenizer.rs:168-180): the text
 * of one token given the one before it. */
WGML_API int wgml_llama_tokenizer_decode(const wgml_tokenizer *t, uint32_t prev_token,
                                         uint32_t token, char *buf, uint64_t cap, uint64_t *n_out);
/* Gpt2Tokenizer::encode(text) (gpt2/tokenizer.rs:105-144).  A "<...>" string that is
 * not in the vocabulary is WGML_E_INVALID (the reference panics). */
WGML_API int wgml_gpt2_tokenizer_encode(const wgml_tokenizer *t, const char *text,
                                        uint64_t text_len, uint32_t *out, uint64_t cap,
                                        uint64_t *n_out);
/* Gpt2Tokenizer::decode(tokens) (gpt2/tokenizer.rs:154-166).  raw_bytes 0: every
 * decoded byte becomes the character of that value, as the reference does (text
 * beyond ASCII comes out as Latin-1); 1: the bytes themselves (UTF-8 stays UTF-8). */
WGML_API int wgml_gpt2_tokenizer_decode(const wgml_tokenizer *t, const uint32_t *tokens,
                                        uint64_t n_tokens, int raw_bytes, char *buf, uint64_t cap,
                                        uint64_t *n_out);

/* ---- sampling beyond greedy: Sampler::sample (models/sampler.rs:32-130), host only ---- *
 * temperature 0: arg-max.  Otherwise the logits are divided by the temperature,
 * turned into probabilities (in place) and a token is drawn with `coin` in [0, 1):
 * from the whole distribution if topp <= 0 or >= 1, else from the smallest set of
 * most likely tokens whose probability exceeds topp. */
WGML_API int wgml_sample(float *logits, uint32_t n, float temperature, float topp, float coin,
                         uint32_t *out_token);
/* The token loop of ChatLlama2::forward with that sampler (chat_llama2.rs:51-153;
 * the reference uses temperature 0.7, top-p 0.95 there, wgml-chat/src/sampler.rs:109):
 * logits are read back after every step and sampled on the host; the coin of position
 * p is the p-th output of the library's counter-based generator for `seed`. */
WGML_API int wgml_llama2_generate_sampled(wgml_llama2 *m, const uint32_t *prompt,
                                          uint32_t n_prompt, uint32_t n_total, float temperature,
                                          float topp, uint64_t seed, uint32_t *out_tokens);

/* ---- GGUF container: Gguf::from_bytes (gguf.rs:450-607), host only -------- *
 * The file is memory-mapped (or the caller's bytes are used in place); the
 * pointers handed out below point into it and stay valid until close.
 * Metadata value types: 0 u8, 1 i8, 2 u16, 3 i16, 4 u32, 5 i32, 6 f32, 7 bool,
 * 8 string, 9 array, 10 u64, 11 i64, 12 f64 (gguf.rs:330-361).  Tensor types are
 * the WGML_* tags above (gguf.rs:70-103). */
typedef struct wgml_gguf wgml_gguf;
typedef struct {
    const char *key;
    int type;           /* metadata value type */
    int array_type;     /* element type when type == 9 */
    uint64_t array_len; /* element count when type == 9 */
    const void *data;   /* scalar: its bytes; string: its bytes (not terminated);
                           array of scalars: the elements; array of strings: null */
    uint64_t nbytes;    /* bytes at `data` */
} wgml_gguf_kv;
typedef struct {
    const char *name;
    int type;
    uint32_t ndims;
    uint64_t dims[4]; /* dims[0] is the contiguous one (GGML order); unused ones are 1 */
    uint64_t offset;  /* from the start of the file */
    uint64_t nbytes;  /* 0 for tensor types whose block size is not known here */
    const void *data;
} wgml_gguf_tensor_info;
WGML_API int wgml_gguf_open(const char *path, wgml_gguf **out);
WGML_API int wgml_gguf_open_bytes(const void *bytes, uint64_t size, wgml_gguf **out);
WGML_API int wgml_gguf_close(wgml_gguf *g);
WGML_API uint32_t wgml_gguf_version(const wgml_gguf *g);
WGML_API uint32_t wgml_gguf_alignment(const wgml_gguf *g); /* general.alignment, default 32 */
WGML_API uint64_t wgml_gguf_n_metadata(const wgml_gguf *g);
WGML_API uint64_t wgml_gguf_n_tensors(const wgml_gguf *g);
/* Index of a key / tensor name, -1 if absent (Gguf::metadata / Gguf::tensors lookups). */
WGML_API int64_t wgml_gguf_find_metadata(const wgml_gguf *g, const char *key);
WGML_API int64_t wgml_gguf_find_tensor(const wgml_gguf *g, const char *name);
WGML_API int wgml_gguf_metadata(const wgml_gguf *g, uint64_t i, wgml_gguf_kv *out);
/* Element k of a string array. */
WGML_API int wgml_gguf_metadata_string(const wgml_gguf *g, uint64_t i, uint64_t k, const char **s,
                                       uint64_t *len);
WGML_API int wgml_gguf_tensor(const wgml_gguf *g, uint64_t i, wgml_gguf_tensor_info *out);

/* ---- host-side input makers (no device needed) ---------------------------- *
 * The reference only de-quantizes; its inputs come from GGUF files written by
 * ggml.  These restate ggml's reference quantizers (quantize_row_q8_0_ref,
 * quantize_row_q4_K_ref, quantize_row_q6_K_ref) so that synthetic weights can
 * be produced in-process.  nthreads <= 0 picks the available cores. */
WGML_API int wgml_quantize(int type, const float *src, void *dst, uint64_t nelems, int nthreads);
/* Block*::dequantize on the host (quantization.rs:16-42, 204-244, 322-389) for
 * F32, F16, Q8_0, Q4_K, Q6_K: what the reference does at load for tensors it
 * keeps in f32 (token_embd, models/llama2/transformer.rs:239-242). */
WGML_API int wgml_dequantize_host(int type, const void *src, float *dst, uint64_t nelems,
                                  int nthreads);
/* Counter-based generator: element i depends only on (seed, i).
 * normal: mean + std * N(0,1) by Box-Muller in f32. */
WGML_API int wgml_rng_normal(uint64_t seed, float *out, uint64_t n, float mean, float std,
                             int nthreads);
/* uniform floats in [0, 1) (24 random bits each). */
WGML_API int wgml_rng_uniform_f32(uint64_t seed, float *out, uint64_t n);
/* uniform integers in [0, bound). */
WGML_API int wgml_rng_uniform_u32(uint64_t seed, uint32_t *out, uint64_t n, uint32_t bound);

#ifdef __cplusplus
}
#endif
#endif
