/*
 * wgml_oracle — TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C, single-threaded CPU restatement of dimforge/wgml's batch-1
 * token-decode path (its CPU twins `run_cpu` / `cpu.rs`).  It exists so the
 * HIP kernels can be checked against the reference's arithmetic.  Nothing in
 * the product library links, loads or calls this file: only the test-suite,
 * the smoke check and the benchmark's CPU-baseline leg may use it.
 *
 * Every function cites the reference source (paths relative to the
 * reference tree's `crates/wgml/src/`) whose arithmetic it follows.
 *
 * How each function is pinned (what would fail if it were wrong):
 *   orc_decode_f16        all 65 536 inputs vs numpy float16->float32
 *   orc_dequantize_*      the reference's own deterministic test blocks
 *                         (ops/quantization.rs:79-86,179-222) with hand-
 *                         computed anchors, + an independent vectorised numpy
 *                         restatement, bit for bit, on random block bits
 *   orc_gemv_*            definition (dequantize, then dot); one-hot vectors
 *                         return dequantized columns; brute force
 *   orc_rms_norm, orc_layernorm, orc_softmax, orc_silu, orc_gelu
 *                         torch.nn.functional closed forms
 *   orc_rope              complex-rotation closed form + invariants
 *   orc_attention         torch softmax(qK^T/sqrt(d))V with the GQA head map
 *   orc_llama2_* / orc_gpt2_*
 *                         composition of the above; an independent numpy
 *                         float64 forward agrees to 1e-4.  The reference
 *                         holds no end-to-end logits, so the greedy ids are
 *                         pinned by construction only.
 *   tokenizers            restated in oracle/tokenizers.py (Python); pinned by merge
 *                         sequences traced by hand on small vocabularies and by the
 *                         library's independent scanner; ids on a real vocabulary are
 *                         parity unpinned (no vocabulary or golden ids exist offline)
 *   parity unpinned:      the exact f32 summation order of nalgebra's gemv
 *                         (source not in the reference tree; restated from
 *                         its documented column-sweep axpy form).
 */
#ifndef WGML_ORACLE_H
#define WGML_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Quantization tags: same numeric values as the GGUF tensor-type ids used by
 * gguf.rs:70-103. */
enum {
    ORC_F32 = 0,
    ORC_F16 = 1,
    ORC_Q4_0 = 2,
    ORC_Q4_1 = 3,
    ORC_Q5_0 = 6,
    ORC_Q5_1 = 7,
    ORC_Q8_0 = 8,
    ORC_Q4_K = 12,
    ORC_Q5_K = 13,
    ORC_Q6_K = 14,
    ORC_Q8_K = 15,
};

/* quantization.rs:392-409 */
float orc_decode_f16(uint16_t half_bits);

/* Bytes per block / elements per block for a tag (0 if unknown). */
size_t orc_block_bytes(int type);
size_t orc_block_elems(int type);

/* quantization.rs:38-41 (Q8_0), :347-378 (Q4_K), :214-243 (Q6_K).
 * `blocks` is the GGUF byte stream; `out` receives nblocks*elems floats. */
void orc_dequantize_q8_0(const void *blocks, size_t nblocks, float *out);
void orc_dequantize_q4_k(const void *blocks, size_t nblocks, float *out);
void orc_dequantize_q6_k(const void *blocks, size_t nblocks, float *out);
/* quantization.rs:53-68, 82-98, 112-131, 146-167, 195-201, 274-317 */
void orc_dequantize_q4_0(const void *blocks, size_t nblocks, float *out);
void orc_dequantize_q4_1(const void *blocks, size_t nblocks, float *out);
void orc_dequantize_q5_0(const void *blocks, size_t nblocks, float *out);
void orc_dequantize_q5_1(const void *blocks, size_t nblocks, float *out);
void orc_dequantize_q8_k(const void *blocks, size_t nblocks, float *out);
void orc_dequantize_q5_k(const void *blocks, size_t nblocks, float *out);
/* gguf.rs:114-129: dispatch on the tag; returns 0, or -1 for an unsupported tag. */
int orc_dequantize(int type, const void *blocks, size_t nelems, float *out);

/* models/llama2/cpu.rs:368-374 — `out.gemv(1.0, w, x, 0.0)` on a dequantized
 * matrix: every out[i] is the f32 sum over columns j = 0..n in order, each
 * term a separately rounded product (no fused multiply-add).  `w` is row-major
 * nrows x ncols. */
/* threads for the rows of matrix-vector products (1 = as the reference; results do not depend on it) */
void orc_set_threads(int n);
int orc_get_threads(void);
void orc_gemv_f32(float *out, const float *w, const float *x, int nrows, int ncols);
/* Same product accumulated in double: the tolerance anchor for GPU GEMVs. */
void orc_gemv_f64(double *out, const float *w, const float *x, int nrows, int ncols);
/* out = dequantize(m) * x, rows dequantized on the fly (same arithmetic per
 * element as dequantize-all-then-gemv).  Either output may be NULL. */
int orc_gemv_quant(int type, const void *blocks, int nrows, int ncols, const float *x,
                   float *out_f32, double *out_f64);

/* ops/rms_norm.rs:55-63 with the nudge factor taken from the config as the GPU
 * path does (models/llama2/transformer.rs:312-320, ops/rms_norm.wgsl:60-66). */
void orc_rms_norm(float *out, const float *a, const float *w, int n, float eps);
/* ops/layernorm.rs:46-53 */
void orc_layernorm(float *out, const float *v, int n);
/* ops/softmax.rs:36-49 */
void orc_softmax(float *vals, int n);
/* ops/silu.rs:36-44 */
void orc_silu(float *h1, const float *h2, int n);
/* ops/unary.rs:106-110 (UnaryOp::Gelu) */
void orc_gelu(float *x, int n);
/* ops/rope.rs:79-116, with base_freq from the config as ops/rope.wgsl:38-41
 * does.  variant 0 = Original (adjacent pairs), 1 = Neox (ops/rope.wgsl:59-78).
 * `dim` = len(q). */
void orc_rope(float *q, float *k, int head_size, int dim, int kv_dim, int pos, float base_freq,
              int variant);

typedef struct {
    uint32_t seq_len, kv_dim, kv_mul, n_heads, head_size, pos;
} orc_attn_params; /* ops/batched_multiquery_attention.rs:30-37 */

/* ops/batched_multiquery_attention.rs:141-195.  key/value cache: position t at
 * [t*kv_dim .. (t+1)*kv_dim).  attn: head h at [h*seq_len ..]. */
void orc_attention(const orc_attn_params *p, const float *q, const float *key_cache,
                   const float *value_cache, float *attn, float *xb);

/* models/sampler.rs:54-56: index of the first maximum. */
uint32_t orc_argmax(const float *v, int n);
/* models/sampler.rs:32-130 with the random number passed in (`coin` in [0, 1)). */
uint32_t orc_sample_mult(const float *p, int n, float coin);
uint32_t orc_sample_topp(const float *p, int n, float topp, float coin);
uint32_t orc_sample(float *logits, int n, float temperature, float topp, float coin);

/* A matrix as the oracle sees it: a tag plus GGUF bytes (or f32 values). */
typedef struct {
    int type;
    const void *data;
    int nrows, ncols;
} orc_matrix;

typedef struct {
    /* models/llama2/cpu.rs:46-67 */
    int dim, hidden_dim, n_layers, n_q_heads, n_kv_heads, vocab_size, seq_len;
    float rope_base_freq, rms_norm_eps;
    int rope_variant; /* models/llama2/mod.rs:26-32 */
} orc_llama2_config;

typedef struct {
    /* models/llama2/cpu.rs:160-170 (+ optional q/k/v bias, transformer.rs:133-135) */
    orc_matrix attn_q, attn_k, attn_v, attn_output, ffn_gate, ffn_up, ffn_down;
    const float *attn_norm, *ffn_norm;
    const float *attn_q_bias, *attn_k_bias, *attn_v_bias; /* may be NULL */
} orc_llama2_layer;

typedef struct orc_llama2 orc_llama2;

/* `token_embd`: f32, column `tok` at [tok*dim ..] (models/llama2/cpu.rs:244).
 * All pointers are borrowed and must outlive the model. */
orc_llama2 *orc_llama2_new(const orc_llama2_config *cfg, const orc_llama2_layer *layers,
                           const float *token_embd, const orc_matrix *output,
                           const float *output_norm);
void orc_llama2_free(orc_llama2 *m);
/* Expand every matrix to f32 once, as models/llama2/cpu.rs:198-204 does at load
 * (faithful timing mode).  Results are identical with or without it. */
int orc_llama2_predequantize(orc_llama2 *m);
/* models/llama2/cpu.rs:377-444 */
void orc_llama2_forward(orc_llama2 *m, int token, int pos);
float *orc_llama2_logits(orc_llama2 *m);
float *orc_llama2_key_cache(orc_llama2 *m, int layer);
float *orc_llama2_value_cache(orc_llama2 *m, int layer);
float *orc_llama2_x(orc_llama2 *m);

typedef struct {
    /* models/gpt2/cpu.rs:18-33 */
    int n_vocab, n_seq, n_embd, n_head, n_layer, ff_len, attn_b;
} orc_gpt2_params;

typedef struct {
    /* models/gpt2/cpu.rs:66-88 */
    const float *ln_1_g, *ln_1_b, *ln_2_g, *ln_2_b;
    orc_matrix c_attn_attn_w;
    const float *c_attn_attn_b;
    orc_matrix c_attn_proj_w;
    const float *c_attn_proj_b;
    orc_matrix c_mlp_fc_w;
    const float *c_mlp_fc_b;
    orc_matrix c_mlp_proj_w;
    const float *c_mlp_proj_b;
} orc_gpt2_layer;

typedef struct orc_gpt2 orc_gpt2;

/* wte/wpe f32 with column c at [c*n_embd ..]; lm_head is its own matrix
 * (n_vocab x n_embd) so that a quantized head can be checked as well
 * (models/gpt2/cpu.rs:193-196 uses wte^T). */
orc_gpt2 *orc_gpt2_new(const orc_gpt2_params *p, const orc_gpt2_layer *layers, const float *wte,
                       const float *wpe, const orc_matrix *lm_head, const float *ln_f_g,
                       const float *ln_f_b);
void orc_gpt2_free(orc_gpt2 *m);
int orc_gpt2_predequantize(orc_gpt2 *m);
/* models/gpt2/cpu.rs:224-381 */
void orc_gpt2_forward(orc_gpt2 *m, int token, int pos);
float *orc_gpt2_logits(orc_gpt2 *m);

/* Timing helper for the CPU-baseline leg: nalgebra-shaped GEMV on a
 * column-major f32 copy (one axpy per column, models/llama2/cpu.rs:211-217 +
 * :368-374).  Same values as orc_gemv_f32. */
void orc_gemv_f32_colmajor(float *out, const float *w_colmajor, const float *x, int nrows,
                           int ncols);

#ifdef __cplusplus
}
#endif
#endif
