/*
 * wgml_oracle — TEST INFRASTRUCTURE ONLY (see wgml_oracle.h).
 *
 * C restatement of the reference's CPU arithmetic, single-threaded unless orc_set_threads
 * asks otherwise (a timing mode with identical results).  Compile
 * with -ffp-contract=off so that no multiply-add is fused: the reference is
 * Rust, which never contracts a*b+c.
 */
#include "wgml_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ f16 -- */

/* quantization.rs:392-409.  powi(2, e) is exact for these exponents, so ldexpf
 * gives the same value. */
float orc_decode_f16(uint16_t half) {
    uint16_t exp = (half >> 10) & 0x1f;
    uint16_t mant = half & 0x3ff;
    float val;
    if (exp == 0) {
        val = ldexpf((float)mant, -24);
    } else if (exp != 31) {
        val = ldexpf((float)mant + 1024.0f, (int)exp - 25);
    } else if (mant == 0) {
        val = INFINITY;
    } else {
        val = NAN;
    }
    return (half & 0x8000) ? -val : val;
}

/* --------------------------------------------------------------- blocks -- */

#define QK8_0 32
#define QK_K 256
#define K_SCALE_SIZE 12

#pragma pack(push, 1)
typedef struct { /* quantization.rs:29-32 */
    uint16_t scale;
    int8_t data[QK8_0];
} block_q8_0;
typedef struct { /* quantization.rs:322-327 */
    uint16_t d, dmin;
    uint8_t scales[K_SCALE_SIZE];
    uint8_t qs[QK_K / 2];
} block_q4_k;
typedef struct { /* quantization.rs:204-209 */
    uint8_t ql[QK_K / 2];
    uint8_t qh[QK_K / 4];
    int8_t scales[QK_K / 16];
    uint16_t d;
} block_q6_k;
typedef struct { /* quantization.rs:47-50 */
    uint16_t d;
    uint8_t qs[16];
} block_q4_0;
typedef struct { /* quantization.rs:75-79 */
    uint16_t d, m;
    uint8_t qs[16];
} block_q4_1;
typedef struct { /* quantization.rs:105-109 */
    uint16_t d;
    uint8_t qh[4];
    uint8_t qs[16];
} block_q5_0;
typedef struct { /* quantization.rs:138-143 */
    uint16_t d, m;
    uint8_t qh[4];
    uint8_t qs[16];
} block_q5_1;
typedef struct { /* quantization.rs:174-178 */
    float d;
    int8_t qs[QK_K];
    int16_t bsums[QK_K / 16];
} block_q8_k;
typedef struct { /* quantization.rs:249-255 */
    uint16_t d, dmin;
    uint8_t scales[K_SCALE_SIZE];
    uint8_t qh[QK_K / 8];
    uint8_t qs[QK_K / 2];
} block_q5_k;
#pragma pack(pop)

_Static_assert(sizeof(block_q4_0) == 18, "q4_0 block size");
_Static_assert(sizeof(block_q4_1) == 20, "q4_1 block size");
_Static_assert(sizeof(block_q5_0) == 22, "q5_0 block size");
_Static_assert(sizeof(block_q5_1) == 24, "q5_1 block size");
_Static_assert(sizeof(block_q8_k) == 292, "q8_k block size");
_Static_assert(sizeof(block_q5_k) == 176, "q5_k block size");
_Static_assert(sizeof(block_q8_0) == 34, "q8_0 block size");
_Static_assert(sizeof(block_q4_k) == 144, "q4_k block size");
_Static_assert(sizeof(block_q6_k) == 210, "q6_k block size");

size_t orc_block_bytes(int type) {
    switch (type) {
    case ORC_F32: return 4;
    case ORC_F16: return 2;
    case ORC_Q4_0: return sizeof(block_q4_0);
    case ORC_Q4_1: return sizeof(block_q4_1);
    case ORC_Q5_0: return sizeof(block_q5_0);
    case ORC_Q5_1: return sizeof(block_q5_1);
    case ORC_Q8_0: return sizeof(block_q8_0);
    case ORC_Q4_K: return sizeof(block_q4_k);
    case ORC_Q5_K: return sizeof(block_q5_k);
    case ORC_Q6_K: return sizeof(block_q6_k);
    case ORC_Q8_K: return sizeof(block_q8_k);
    default: return 0;
    }
}

size_t orc_block_elems(int type) {
    switch (type) {
    case ORC_F32: return 1;
    case ORC_F16: return 1;
    case ORC_Q4_0: case ORC_Q4_1: case ORC_Q5_0: case ORC_Q5_1: return 32;
    case ORC_Q8_0: return QK8_0;
    case ORC_Q4_K: case ORC_Q5_K: case ORC_Q6_K: case ORC_Q8_K: return QK_K;
    default: return 0;
    }
}

/* quantization.rs:38-41 */
void orc_dequantize_q8_0(const void *blocks, size_t nblocks, float *out) {
    const block_q8_0 *b = (const block_q8_0 *)blocks;
    for (size_t i = 0; i < nblocks; ++i) {
        float scale = orc_decode_f16(b[i].scale);
        for (int j = 0; j < QK8_0; ++j)
            out[i * QK8_0 + j] = (float)b[i].data[j] * scale;
    }
}

/* quantization.rs:381-389 */
static void get_scale_min_k4(int j, const uint8_t *q, uint8_t *d, uint8_t *m) {
    if (j < 4) {
        *d = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *d = (uint8_t)((q[j + 4] & 0xf) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* quantization.rs:347-378 */
void orc_dequantize_q4_k(const void *blocks, size_t nblocks, float *out) {
    const block_q4_k *b = (const block_q4_k *)blocks;
    for (size_t i = 0; i < nblocks; ++i) {
        float *res = out + i * QK_K;
        float d = orc_decode_f16(b[i].d);
        float min = orc_decode_f16(b[i].dmin);
        int is = 0, iq = 0;
        uint8_t sc, m;
        for (int j = 0; j < QK_K; j += 64) {
            get_scale_min_k4(is, b[i].scales, &sc, &m);
            float d1 = d * (float)sc;
            float m1 = min * (float)m;
            get_scale_min_k4(is + 1, b[i].scales, &sc, &m);
            float d2 = d * (float)sc;
            float m2 = min * (float)m;
            for (int l = 0; l < 32; ++l)
                res[j + l] = d1 * (float)(b[i].qs[iq + l] & 0xF) - m1;
            for (int l = 0; l < 32; ++l)
                res[j + l + 32] = d2 * (float)(b[i].qs[iq + l] >> 4) - m2;
            iq += 32;
            is += 2;
        }
    }
}

/* quantization.rs:214-243 */
void orc_dequantize_q6_k(const void *blocks, size_t nblocks, float *out) {
    const block_q6_k *b = (const block_q6_k *)blocks;
    for (size_t n = 0; n < nblocks; ++n) {
        float *res = out + n * QK_K;
        float d = orc_decode_f16(b[n].d);
        for (int i = 0; i < 2; ++i) {
            for (int l = 0; l < 32; ++l) {
                int is = l / 16;
                uint8_t ql0 = b[n].ql[i * 64 + l];
                uint8_t ql32 = b[n].ql[i * 64 + l + 32];
                uint8_t qh = b[n].qh[i * 32 + l];
                int8_t q1 = (int8_t)((ql0 & 0xF) | (((qh >> 0) & 3) << 4)) - 32;
                int8_t q2 = (int8_t)((ql32 & 0xF) | (((qh >> 2) & 3) << 4)) - 32;
                int8_t q3 = (int8_t)((ql0 >> 4) | (((qh >> 4) & 3) << 4)) - 32;
                int8_t q4 = (int8_t)((ql32 >> 4) | (((qh >> 6) & 3) << 4)) - 32;
                const int8_t *s = b[n].scales + i * 8 + is;
                res[i * 128 + l + 0] = d * (float)s[0] * (float)q1;
                res[i * 128 + l + 32] = d * (float)s[2] * (float)q2;
                res[i * 128 + l + 64] = d * (float)s[4] * (float)q3;
                res[i * 128 + l + 96] = d * (float)s[6] * (float)q4;
            }
        }
    }
}

/* quantization.rs:53-68 */
void orc_dequantize_q4_0(const void *blocks, size_t nblocks, float *out) {
    const block_q4_0 *b = (const block_q4_0 *)blocks;
    for (size_t i = 0; i < nblocks; ++i, out += 32) {
        const float d = orc_decode_f16(b[i].d);
        for (int j = 0; j < 16; ++j) {
            const int x0 = (int)(b[i].qs[j] & 0x0F) - 8, x1 = (int)(b[i].qs[j] >> 4) - 8;
            out[j] = (float)x0 * d;
            out[j + 16] = (float)x1 * d;
        }
    }
}

/* quantization.rs:82-98 */
void orc_dequantize_q4_1(const void *blocks, size_t nblocks, float *out) {
    const block_q4_1 *b = (const block_q4_1 *)blocks;
    for (size_t i = 0; i < nblocks; ++i, out += 32) {
        const float d = orc_decode_f16(b[i].d), m = orc_decode_f16(b[i].m);
        for (int j = 0; j < 16; ++j) {
            out[j] = (float)(b[i].qs[j] & 0x0F) * d + m;
            out[j + 16] = (float)(b[i].qs[j] >> 4) * d + m;
        }
    }
}

/* quantization.rs:112-131 */
void orc_dequantize_q5_0(const void *blocks, size_t nblocks, float *out) {
    const block_q5_0 *b = (const block_q5_0 *)blocks;
    for (size_t i = 0; i < nblocks; ++i, out += 32) {
        const float d = orc_decode_f16(b[i].d);
        uint32_t qh;
        memcpy(&qh, b[i].qh, 4);
        for (int j = 0; j < 16; ++j) {
            const uint32_t xh_0 = ((qh >> j) << 4) & 0x10, xh_1 = (qh >> (j + 12)) & 0x10;
            const int x0 = (int)((b[i].qs[j] & 0x0Fu) | xh_0) - 16;
            const int x1 = (int)((uint32_t)(b[i].qs[j] >> 4) | xh_1) - 16;
            out[j] = (float)x0 * d;
            out[j + 16] = (float)x1 * d;
        }
    }
}

/* quantization.rs:146-167 */
void orc_dequantize_q5_1(const void *blocks, size_t nblocks, float *out) {
    const block_q5_1 *b = (const block_q5_1 *)blocks;
    for (size_t i = 0; i < nblocks; ++i, out += 32) {
        const float d = orc_decode_f16(b[i].d), m = orc_decode_f16(b[i].m);
        uint32_t qh;
        memcpy(&qh, b[i].qh, 4);
        for (int j = 0; j < 16; ++j) {
            const uint32_t xh_0 = ((qh >> j) << 4) & 0x10, xh_1 = (qh >> (j + 12)) & 0x10;
            const uint32_t x0 = (b[i].qs[j] & 0x0Fu) | xh_0, x1 = (uint32_t)(b[i].qs[j] >> 4) | xh_1;
            out[j] = (float)x0 * d + m;
            out[j + 16] = (float)x1 * d + m;
        }
    }
}

/* quantization.rs:195-201 */
void orc_dequantize_q8_k(const void *blocks, size_t nblocks, float *out) {
    const block_q8_k *b = (const block_q8_k *)blocks;
    for (size_t i = 0; i < nblocks; ++i, out += QK_K)
        for (int j = 0; j < QK_K; ++j) out[j] = b[i].d * (float)b[i].qs[j];
}

/* quantization.rs:274-317 */
void orc_dequantize_q5_k(const void *blocks, size_t nblocks, float *out) {
    const block_q5_k *b = (const block_q5_k *)blocks;
    for (size_t i = 0; i < nblocks; ++i, out += QK_K) {
        const float d = orc_decode_f16(b[i].d), min = orc_decode_f16(b[i].dmin);
        int iq = 0, is = 0;
        uint8_t u1 = 1, u2 = 2, sc, m;
        for (int j = 0; j < QK_K; j += 64) {
            get_scale_min_k4(is, b[i].scales, &sc, &m);
            const float d1 = d * (float)sc, m1 = min * (float)m;
            get_scale_min_k4(is + 1, b[i].scales, &sc, &m);
            const float d2 = d * (float)sc, m2 = min * (float)m;
            for (int l = 0; l < 32; ++l)
                out[j + l] = d1 * (float)((b[i].qs[iq + l] & 0xF) + ((b[i].qh[l] & u1) ? 16 : 0)) - m1;
            for (int l = 0; l < 32; ++l)
                out[j + l + 32] =
                    d2 * (float)((b[i].qs[iq + l] >> 4) + ((b[i].qh[l] & u2) ? 16 : 0)) - m2;
            iq += 32;
            is += 2;
            u1 = (uint8_t)(u1 << 2);
            u2 = (uint8_t)(u2 << 2);
        }
    }
}

/* gguf.rs:114-129 */
int orc_dequantize(int type, const void *blocks, size_t nelems, float *out) {
    switch (type) {
    case ORC_F32: memcpy(out, blocks, nelems * sizeof(float)); return 0;
    case ORC_F16:
        for (size_t i = 0; i < nelems; ++i) out[i] = orc_decode_f16(((const uint16_t *)blocks)[i]);
        return 0;
    case ORC_Q4_0: orc_dequantize_q4_0(blocks, nelems / 32, out); return 0;
    case ORC_Q4_1: orc_dequantize_q4_1(blocks, nelems / 32, out); return 0;
    case ORC_Q5_0: orc_dequantize_q5_0(blocks, nelems / 32, out); return 0;
    case ORC_Q5_1: orc_dequantize_q5_1(blocks, nelems / 32, out); return 0;
    case ORC_Q5_K: orc_dequantize_q5_k(blocks, nelems / QK_K, out); return 0;
    case ORC_Q8_K: orc_dequantize_q8_k(blocks, nelems / QK_K, out); return 0;
    case ORC_Q8_0: orc_dequantize_q8_0(blocks, nelems / QK8_0, out); return 0;
    case ORC_Q4_K: orc_dequantize_q4_k(blocks, nelems / QK_K, out); return 0;
    case ORC_Q6_K: orc_dequantize_q6_k(blocks, nelems / QK_K, out); return 0;
    default: return -1;
    }
}

/* ----------------------------------------------------------------- BLAS -- */

/* nalgebra's `dot` as used by norm_squared()/dot() in ops/rms_norm.rs:61,
 * ops/layernorm.rs:50 and ops/batched_multiquery_attention.rs:175: eight
 * running sums over strides of 8, folded as (0+4)+(1+5)+(2+6)+(3+7), then the
 * tail in order.  nalgebra's source is not in the reference tree; this is its
 * published form (parity unpinned at the last-bit level). */
static float dot8(const float *a, const float *b, int n) {
    float res = 0.0f;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    int i = 0;
    while (n - i >= 8) {
        for (int k = 0; k < 8; ++k) acc[k] += a[i + k] * b[i + k];
        i += 8;
    }
    res += acc[0] + acc[4];
    res += acc[1] + acc[5];
    res += acc[2] + acc[6];
    res += acc[3] + acc[7];
    for (; i < n; ++i) res += a[i] * b[i];
    return res;
}

/* models/llama2/cpu.rs:373: out.gemv(1.0, w, x, 0.0) — one axpy per column, so
 * out[i] = (..((x0*w[i][0]) + x1*w[i][1]) + ..), each product rounded. */
/* Timing mode only (the benchmark's all-cores CPU baseline): rows of a matrix-vector
 * product are shared out over n threads.  Every row's sum keeps its sequential order, so
 * results are identical to the single-threaded ones; the reference itself has no threading
 * (models/llama2/cpu.rs), so 1 is the faithful setting and the default. */
static int g_threads = 1;
void orc_set_threads(int n) { g_threads = n > 1 ? n : 1; }
int orc_get_threads(void) { return g_threads; }

void orc_gemv_f32(float *out, const float *w, const float *x, int nrows, int ncols) {
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1 && nrows >= 64) schedule(static)
    for (int i = 0; i < nrows; ++i) {
        const float *row = w + (size_t)i * ncols;
        float acc = (1.0f * x[0]) * row[0];
        for (int j = 1; j < ncols; ++j) acc = (1.0f * x[j]) * row[j] + acc;
        out[i] = acc;
    }
}

void orc_gemv_f32_colmajor(float *out, const float *w, const float *x, int nrows, int ncols) {
    {
        const float a = 1.0f * x[0];
        for (int i = 0; i < nrows; ++i) out[i] = a * w[i];
    }
    for (int j = 1; j < ncols; ++j) {
        const float a = 1.0f * x[j];
        const float *col = w + (size_t)j * nrows;
        for (int i = 0; i < nrows; ++i) out[i] = a * col[i] + out[i];
    }
}

void orc_gemv_f64(double *out, const float *w, const float *x, int nrows, int ncols) {
    for (int i = 0; i < nrows; ++i) {
        const float *row = w + (size_t)i * ncols;
        double acc = 0.0;
        for (int j = 0; j < ncols; ++j) acc += (double)row[j] * (double)x[j];
        out[i] = acc;
    }
}

int orc_gemv_quant(int type, const void *blocks, int nrows, int ncols, const float *x,
                   float *out_f32, double *out_f64) {
    size_t be = orc_block_elems(type), bb = orc_block_bytes(type);
    if (!be || ncols % (int)be) return -1;
    size_t row_bytes = (size_t)ncols / be * bb;
    int failed = 0;
#pragma omp parallel num_threads(g_threads) if (g_threads > 1 && nrows >= 64)
    {
        float *row = (float *)malloc((size_t)ncols * sizeof(float));
        if (!row) {
#pragma omp atomic write
            failed = 1;
        } else {
#pragma omp for schedule(static)
            for (int i = 0; i < nrows; ++i) {
                orc_dequantize(type, (const uint8_t *)blocks + (size_t)i * row_bytes, (size_t)ncols,
                               row);
                if (out_f32) orc_gemv_f32(out_f32 + i, row, x, 1, ncols);
                if (out_f64) orc_gemv_f64(out_f64 + i, row, x, 1, ncols);
            }
            free(row);
        }
    }
    return failed ? -2 : 0;
}

/* ------------------------------------------------------------------ ops -- */

/* ops/rms_norm.rs:55-63 */
void orc_rms_norm(float *out, const float *a, const float *w, int n, float eps) {
    float rms = 1.0f / sqrtf(dot8(a, a, n) / (float)n + eps);
    for (int i = 0; i < n; ++i) out[i] = (a[i] * rms) * w[i];
}

/* ops/layernorm.rs:46-53 */
void orc_layernorm(float *res, const float *v, int n) {
    float sum = 0.0f;
    for (int i = 0; i < n; ++i) sum += v[i];
    float mean = sum / (float)n;
    for (int i = 0; i < n; ++i) res[i] = v[i] - mean;
    float variance = dot8(res, res, n) / (float)n;
    float scale = 1.0f / sqrtf(variance + 1.0e-5f);
    for (int i = 0; i < n; ++i) res[i] *= scale;
}

/* ops/softmax.rs:36-49 */
void orc_softmax(float *vals, int n) {
    float max_val = vals[0];
    for (int i = 1; i < n; ++i)
        if (vals[i] > max_val) max_val = vals[i];
    float sum = 0.0f;
    for (int i = 0; i < n; ++i) {
        vals[i] = expf(vals[i] - max_val);
        sum += vals[i];
    }
    for (int i = 0; i < n; ++i) vals[i] /= sum;
}

/* ops/silu.rs:36-44 */
void orc_silu(float *h1, const float *h2, int n) {
    for (int i = 0; i < n; ++i) {
        float x = h1[i];
        float swish = x / (1.0f + expf(-1.0f * x));
        h1[i] = h2[i] * swish;
    }
}

/* ops/unary.rs:106-110 */
void orc_gelu(float *v, int n) {
    const float GELU_COEF_A = 0.044715f;
    const float SQRT_2_OVER_PI = 0.7978846f;
    for (int i = 0; i < n; ++i) {
        float x = v[i];
        v[i] = 0.5f * x * (1.0f + tanhf(SQRT_2_OVER_PI * x * (1.0f + GELU_COEF_A * x * x)));
    }
}

/* ops/rope.rs:79-116 (pair layout) and ops/rope.wgsl:35-78 (base frequency from
 * the config, Neox pairing). */
void orc_rope(float *q, float *k, int head_size, int dim, int kv_dim, int pos, float base_freq,
              int variant) {
    for (int i = 0; i < dim; i += 2) {
        float head_dim = (float)(i % head_size);
        float theta = powf(base_freq, -head_dim / (float)head_size);
        float m_theta = (float)pos * theta;
        float c = cosf(m_theta), s = sinf(m_theta);
        int a, b;
        if (variant == 0) {
            a = i;
            b = i + 1;
        } else {
            int head_id = i / head_size;
            a = i / 2 + head_id * head_size / 2;
            b = a + head_size / 2;
        }
        float x = q[a], y = q[b];
        q[a] = c * x - s * y;
        q[b] = s * x + c * y;
        if (i < kv_dim) {
            x = k[a];
            y = k[b];
            k[a] = c * x - s * y;
            k[b] = s * x + c * y;
        }
    }
}

/* ops/batched_multiquery_attention.rs:141-195 */
void orc_attention(const orc_attn_params *p, const float *q, const float *key_cache,
                   const float *value_cache, float *attn, float *xb) {
    int head_size = (int)p->head_size, kv_mul = (int)p->kv_mul, kv_dim = (int)p->kv_dim;
    int pos = (int)p->pos;
    for (int h = 0; h < (int)p->n_heads; ++h) {
        const float *qh = q + (size_t)h * head_size;
        float *att = attn + (size_t)h * p->seq_len;
        for (int t = 0; t <= pos; ++t) {
            const float *kh = key_cache + (size_t)t * kv_dim + (size_t)(h / kv_mul) * head_size;
            float score = dot8(qh, kh, head_size);
            score /= sqrtf((float)head_size);
            att[t] = score;
        }
        orc_softmax(att, pos + 1);
        float *o = xb + (size_t)h * head_size;
        for (int i = 0; i < head_size; ++i) o[i] = 0.0f;
        for (int t = 0; t <= pos; ++t) {
            const float *vh = value_cache + (size_t)t * kv_dim + (size_t)(h / kv_mul) * head_size;
            float a = att[t];
            for (int i = 0; i < head_size; ++i) o[i] = a * vh[i] + o[i];
        }
    }
}

/* models/sampler.rs:58-76: `probabilities` sum to 1, coin in [0, 1). */
uint32_t orc_sample_mult(const float *p, int n, float coin) {
    float cdf = 0.0f;
    for (int i = 0; i < n; ++i) {
        cdf += p[i];
        if (coin < cdf) return (uint32_t)i;
    }
    return (uint32_t)(n - 1);
}

/* models/sampler.rs:78-130.  Candidates with p >= (1 - topp) / (n - 1), sorted by
 * decreasing probability (stable: ties keep index order, as Rust's sort_by_key),
 * cut where the running sum first exceeds topp, then sampled with coin * sum. */
uint32_t orc_sample_topp(const float *p, int n, float topp, float coin) {
    const float cutoff = (1.0f - topp) / ((float)n - 1.0f);
    int *idx = (int *)malloc(sizeof(int) * (size_t)n);
    int n0 = 0;
    for (int i = 0; i < n; ++i)
        if (p[i] >= cutoff) idx[n0++] = i;
    if (n0 == 0) { /* the reference would index out of bounds here; it cannot happen for
                      probabilities that sum to 1 */
        free(idx);
        return (uint32_t)(n - 1);
    }
    for (int i = 1; i < n0; ++i) { /* stable insertion sort, descending */
        const int v = idx[i];
        int j = i - 1;
        while (j >= 0 && p[idx[j]] < p[v]) {
            idx[j + 1] = idx[j];
            --j;
        }
        idx[j + 1] = v;
    }
    float cumulative = 0.0f;
    int last = n0 - 1;
    for (int i = 0; i < n0; ++i) {
        cumulative += p[idx[i]];
        if (cumulative > topp) {
            last = i;
            break;
        }
    }
    const float r = coin * cumulative;
    float cdf = 0.0f;
    uint32_t out = (uint32_t)idx[last];
    for (int i = 0; i <= last; ++i) {
        cdf += p[idx[i]];
        if (r < cdf) {
            out = (uint32_t)idx[i];
            break;
        }
    }
    free(idx);
    return out;
}

/* models/sampler.rs:32-52: logits are modified in place (scaled, then softmax). */
uint32_t orc_sample(float *logits, int n, float temperature, float topp, float coin) {
    if (temperature == 0.0f) return orc_argmax(logits, n);
    for (int i = 0; i < n; ++i) logits[i] /= temperature;
    orc_softmax(logits, n);
    if (topp <= 0.0f || topp >= 1.0f) return orc_sample_mult(logits, n, coin);
    return orc_sample_topp(logits, n, topp, coin);
}

/* models/sampler.rs:54-56 */
uint32_t orc_argmax(const float *v, int n) {
    int best = 0;
    for (int i = 1; i < n; ++i)
        if (v[i] > v[best]) best = i;
    return (uint32_t)best;
}

/* --------------------------------------------------------------- models -- */

typedef struct {
    orc_matrix m;
    float *f32; /* optional dequantized copy */
} omat;

static int omat_predequantize(omat *w) {
    if (w->f32 || w->m.type == ORC_F32) return 0;
    size_t n = (size_t)w->m.nrows * w->m.ncols;
    w->f32 = (float *)malloc(n * sizeof(float));
    if (!w->f32) return -1;
    return orc_dequantize(w->m.type, w->m.data, n, w->f32);
}

/* models/llama2/cpu.rs:368-374 */
static void matmul(float *out, const float *x, const omat *w, float *row_tmp) {
    const orc_matrix *m = &w->m;
    if (m->type == ORC_F32) {
        orc_gemv_f32(out, (const float *)m->data, x, m->nrows, m->ncols);
    } else if (w->f32) {
        orc_gemv_f32(out, w->f32, x, m->nrows, m->ncols);
    } else {
        size_t be = orc_block_elems(m->type), bb = orc_block_bytes(m->type);
        size_t row_bytes = (size_t)m->ncols / be * bb;
        for (int i = 0; i < m->nrows; ++i) {
            orc_dequantize(m->type, (const uint8_t *)m->data + (size_t)i * row_bytes,
                           (size_t)m->ncols, row_tmp);
            orc_gemv_f32(out + i, row_tmp, x, 1, m->ncols);
        }
    }
}

typedef struct {
    omat attn_q, attn_k, attn_v, attn_output, ffn_gate, ffn_up, ffn_down;
    const float *attn_norm, *ffn_norm, *bq, *bk, *bv;
} llayer;

struct orc_llama2 {
    orc_llama2_config cfg;
    llayer *layers;
    const float *token_embd;
    omat output;
    const float *output_norm;
    /* models/llama2/cpu.rs:259-280 */
    float *x, *xb, *xb2, *hb, *hb2, *q, *att, *logits, *row_tmp;
    float **key_cache, **value_cache;
};

orc_llama2 *orc_llama2_new(const orc_llama2_config *cfg, const orc_llama2_layer *layers,
                           const float *token_embd, const orc_matrix *output,
                           const float *output_norm) {
    orc_llama2 *m = (orc_llama2 *)calloc(1, sizeof(*m));
    m->cfg = *cfg;
    int L = cfg->n_layers;
    int kv_dim = cfg->dim * cfg->n_kv_heads / cfg->n_q_heads;
    m->layers = (llayer *)calloc((size_t)L, sizeof(llayer));
    for (int l = 0; l < L; ++l) {
        llayer *d = &m->layers[l];
        const orc_llama2_layer *s = &layers[l];
        d->attn_q.m = s->attn_q;
        d->attn_k.m = s->attn_k;
        d->attn_v.m = s->attn_v;
        d->attn_output.m = s->attn_output;
        d->ffn_gate.m = s->ffn_gate;
        d->ffn_up.m = s->ffn_up;
        d->ffn_down.m = s->ffn_down;
        d->attn_norm = s->attn_norm;
        d->ffn_norm = s->ffn_norm;
        d->bq = s->attn_q_bias;
        d->bk = s->attn_k_bias;
        d->bv = s->attn_v_bias;
    }
    m->token_embd = token_embd;
    m->output.m = *output;
    m->output_norm = output_norm;
    int maxc = cfg->dim > cfg->hidden_dim ? cfg->dim : cfg->hidden_dim;
    m->x = (float *)calloc((size_t)cfg->dim, 4);
    m->xb = (float *)calloc((size_t)cfg->dim, 4);
    m->xb2 = (float *)calloc((size_t)cfg->dim, 4);
    m->hb = (float *)calloc((size_t)cfg->hidden_dim, 4);
    m->hb2 = (float *)calloc((size_t)cfg->hidden_dim, 4);
    m->q = (float *)calloc((size_t)cfg->dim, 4);
    m->att = (float *)calloc((size_t)cfg->seq_len * cfg->n_q_heads, 4);
    m->logits = (float *)calloc((size_t)cfg->vocab_size, 4);
    m->row_tmp = (float *)calloc((size_t)maxc, 4);
    m->key_cache = (float **)calloc((size_t)L, sizeof(float *));
    m->value_cache = (float **)calloc((size_t)L, sizeof(float *));
    for (int l = 0; l < L; ++l) {
        m->key_cache[l] = (float *)calloc((size_t)kv_dim * cfg->seq_len, 4);
        m->value_cache[l] = (float *)calloc((size_t)kv_dim * cfg->seq_len, 4);
    }
    return m;
}

void orc_llama2_free(orc_llama2 *m) {
    if (!m) return;
    for (int l = 0; l < m->cfg.n_layers; ++l) {
        llayer *d = &m->layers[l];
        free(d->attn_q.f32);
        free(d->attn_k.f32);
        free(d->attn_v.f32);
        free(d->attn_output.f32);
        free(d->ffn_gate.f32);
        free(d->ffn_up.f32);
        free(d->ffn_down.f32);
        free(m->key_cache[l]);
        free(m->value_cache[l]);
    }
    free(m->output.f32);
    free(m->layers);
    free(m->key_cache);
    free(m->value_cache);
    free(m->x);
    free(m->xb);
    free(m->xb2);
    free(m->hb);
    free(m->hb2);
    free(m->q);
    free(m->att);
    free(m->logits);
    free(m->row_tmp);
    free(m);
}

int orc_llama2_predequantize(orc_llama2 *m) {
    int rc = 0;
    for (int l = 0; l < m->cfg.n_layers; ++l) {
        llayer *d = &m->layers[l];
        rc |= omat_predequantize(&d->attn_q);
        rc |= omat_predequantize(&d->attn_k);
        rc |= omat_predequantize(&d->attn_v);
        rc |= omat_predequantize(&d->attn_output);
        rc |= omat_predequantize(&d->ffn_gate);
        rc |= omat_predequantize(&d->ffn_up);
        rc |= omat_predequantize(&d->ffn_down);
    }
    rc |= omat_predequantize(&m->output);
    return rc;
}

float *orc_llama2_logits(orc_llama2 *m) { return m->logits; }
float *orc_llama2_key_cache(orc_llama2 *m, int layer) { return m->key_cache[layer]; }
float *orc_llama2_value_cache(orc_llama2 *m, int layer) { return m->value_cache[layer]; }
float *orc_llama2_x(orc_llama2 *m) { return m->x; }

/* models/llama2/cpu.rs:377-444; q/k/v bias as models/llama2/transformer.rs:343-354 */
void orc_llama2_forward(orc_llama2 *m, int token, int pos) {
    const orc_llama2_config *c = &m->cfg;
    int dim = c->dim;
    int kv_dim = c->dim * c->n_kv_heads / c->n_q_heads;
    int head_size = dim / c->n_q_heads;
    memcpy(m->x, m->token_embd + (size_t)token * dim, (size_t)dim * 4);

    for (int l = 0; l < c->n_layers; ++l) {
        llayer *wl = &m->layers[l];
        orc_rms_norm(m->xb, m->x, wl->attn_norm, dim, c->rms_norm_eps);

        float *k_cache = m->key_cache[l] + (size_t)pos * kv_dim;
        float *v_cache = m->value_cache[l] + (size_t)pos * kv_dim;
        matmul(m->q, m->xb, &wl->attn_q, m->row_tmp);
        matmul(k_cache, m->xb, &wl->attn_k, m->row_tmp);
        matmul(v_cache, m->xb, &wl->attn_v, m->row_tmp);
        if (wl->bq)
            for (int i = 0; i < dim; ++i) m->q[i] += wl->bq[i];
        if (wl->bk)
            for (int i = 0; i < kv_dim; ++i) k_cache[i] += wl->bk[i];
        if (wl->bv)
            for (int i = 0; i < kv_dim; ++i) v_cache[i] += wl->bv[i];

        orc_rope(m->q, k_cache, head_size, dim, kv_dim, pos, c->rope_base_freq, c->rope_variant);

        /* models/llama2/cpu.rs:486-541 */
        orc_attn_params ap = {(uint32_t)c->seq_len,   (uint32_t)kv_dim,    (uint32_t)(c->n_q_heads / c->n_kv_heads),
                              (uint32_t)c->n_q_heads, (uint32_t)head_size, (uint32_t)pos};
        orc_attention(&ap, m->q, m->key_cache[l], m->value_cache[l], m->att, m->xb);
        matmul(m->xb2, m->xb, &wl->attn_output, m->row_tmp);

        for (int i = 0; i < dim; ++i) m->x[i] += m->xb2[i];

        orc_rms_norm(m->xb, m->x, wl->ffn_norm, dim, c->rms_norm_eps);

        /* models/llama2/cpu.rs:543-562 */
        matmul(m->hb, m->xb, &wl->ffn_gate, m->row_tmp);
        matmul(m->hb2, m->xb, &wl->ffn_up, m->row_tmp);
        orc_silu(m->hb, m->hb2, c->hidden_dim);
        matmul(m->xb2, m->hb, &wl->ffn_down, m->row_tmp);

        for (int i = 0; i < dim; ++i) m->x[i] += m->xb2[i];
    }

    orc_rms_norm(m->xb, m->x, m->output_norm, dim, c->rms_norm_eps);
    matmul(m->logits, m->xb, &m->output, m->row_tmp);
}

typedef struct {
    const float *ln_1_g, *ln_1_b, *ln_2_g, *ln_2_b;
    omat attn_w, proj_w, fc_w, mlp_proj_w;
    const float *attn_b, *proj_b, *fc_b, *mlp_proj_b;
    float *key_cache, *value_cache;
} glayer;

struct orc_gpt2 {
    orc_gpt2_params p;
    glayer *layers;
    const float *wte, *wpe, *ln_f_g, *ln_f_b;
    omat lm_head;
    /* models/gpt2/cpu.rs:101-109 */
    float *memory_q, *memory_att, *layer_input, *curr_768, *curr_768_b, *curr_2304, *curr_3072,
        *curr_vocab, *row_tmp;
};

orc_gpt2 *orc_gpt2_new(const orc_gpt2_params *p, const orc_gpt2_layer *layers, const float *wte,
                       const float *wpe, const orc_matrix *lm_head, const float *ln_f_g,
                       const float *ln_f_b) {
    orc_gpt2 *m = (orc_gpt2 *)calloc(1, sizeof(*m));
    m->p = *p;
    m->layers = (glayer *)calloc((size_t)p->n_layer, sizeof(glayer));
    for (int l = 0; l < p->n_layer; ++l) {
        glayer *d = &m->layers[l];
        const orc_gpt2_layer *s = &layers[l];
        d->ln_1_g = s->ln_1_g;
        d->ln_1_b = s->ln_1_b;
        d->ln_2_g = s->ln_2_g;
        d->ln_2_b = s->ln_2_b;
        d->attn_w.m = s->c_attn_attn_w;
        d->attn_b = s->c_attn_attn_b;
        d->proj_w.m = s->c_attn_proj_w;
        d->proj_b = s->c_attn_proj_b;
        d->fc_w.m = s->c_mlp_fc_w;
        d->fc_b = s->c_mlp_fc_b;
        d->mlp_proj_w.m = s->c_mlp_proj_w;
        d->mlp_proj_b = s->c_mlp_proj_b;
        d->key_cache = (float *)calloc((size_t)p->n_embd * p->n_seq, 4);
        d->value_cache = (float *)calloc((size_t)p->n_embd * p->n_seq, 4);
    }
    m->wte = wte;
    m->wpe = wpe;
    m->lm_head.m = *lm_head;
    m->ln_f_g = ln_f_g;
    m->ln_f_b = ln_f_b;
    int maxc = p->ff_len > p->n_embd ? p->ff_len : p->n_embd;
    m->memory_q = (float *)calloc((size_t)p->n_embd, 4);
    m->memory_att = (float *)calloc((size_t)p->n_seq * p->n_head, 4);
    m->layer_input = (float *)calloc((size_t)p->n_embd, 4);
    m->curr_768 = (float *)calloc((size_t)p->n_embd, 4);
    m->curr_768_b = (float *)calloc((size_t)p->n_embd, 4);
    m->curr_2304 = (float *)calloc((size_t)p->attn_b, 4);
    m->curr_3072 = (float *)calloc((size_t)p->ff_len, 4);
    m->curr_vocab = (float *)calloc((size_t)p->n_vocab, 4);
    m->row_tmp = (float *)calloc((size_t)maxc, 4);
    return m;
}

void orc_gpt2_free(orc_gpt2 *m) {
    if (!m) return;
    for (int l = 0; l < m->p.n_layer; ++l) {
        glayer *d = &m->layers[l];
        free(d->attn_w.f32);
        free(d->proj_w.f32);
        free(d->fc_w.f32);
        free(d->mlp_proj_w.f32);
        free(d->key_cache);
        free(d->value_cache);
    }
    free(m->lm_head.f32);
    free(m->layers);
    free(m->memory_q);
    free(m->memory_att);
    free(m->layer_input);
    free(m->curr_768);
    free(m->curr_768_b);
    free(m->curr_2304);
    free(m->curr_3072);
    free(m->curr_vocab);
    free(m->row_tmp);
    free(m);
}

int orc_gpt2_predequantize(orc_gpt2 *m) {
    int rc = 0;
    for (int l = 0; l < m->p.n_layer; ++l) {
        glayer *d = &m->layers[l];
        rc |= omat_predequantize(&d->attn_w);
        rc |= omat_predequantize(&d->proj_w);
        rc |= omat_predequantize(&d->fc_w);
        rc |= omat_predequantize(&d->mlp_proj_w);
    }
    rc |= omat_predequantize(&m->lm_head);
    return rc;
}

float *orc_gpt2_logits(orc_gpt2 *m) { return m->curr_vocab; }

/* models/gpt2/cpu.rs:224-381 */
void orc_gpt2_forward(orc_gpt2 *m, int embd, int pos) {
    const orc_gpt2_params *p = &m->p;
    int n = p->n_embd;
    for (int i = 0; i < n; ++i) m->layer_input[i] = m->wte[(size_t)embd * n + i];
    for (int i = 0; i < n; ++i) m->layer_input[i] += m->wpe[(size_t)pos * n + i];

    for (int l = 0; l < p->n_layer; ++l) {
        glayer *layer = &m->layers[l];
        orc_layernorm(m->curr_768, m->layer_input, n);
        for (int i = 0; i < n; ++i) m->curr_768[i] *= layer->ln_1_g[i];
        for (int i = 0; i < n; ++i) m->curr_768[i] += layer->ln_1_b[i];

        matmul(m->curr_2304, m->curr_768, &layer->attn_w, m->row_tmp);
        for (int i = 0; i < p->attn_b; ++i) m->curr_2304[i] += layer->attn_b[i];

        float *k_cache = layer->key_cache + (size_t)pos * n;
        float *v_cache = layer->value_cache + (size_t)pos * n;
        memcpy(m->memory_q, m->curr_2304, (size_t)n * 4);
        memcpy(k_cache, m->curr_2304 + n, (size_t)n * 4);
        memcpy(v_cache, m->curr_2304 + 2 * n, (size_t)n * 4);

        orc_attn_params ap = {(uint32_t)p->n_seq,  (uint32_t)n, 1u, (uint32_t)p->n_head,
                              (uint32_t)(n / p->n_head), (uint32_t)pos};
        orc_attention(&ap, m->memory_q, layer->key_cache, layer->value_cache, m->memory_att,
                      m->curr_768);

        matmul(m->curr_768_b, m->curr_768, &layer->proj_w, m->row_tmp);
        for (int i = 0; i < n; ++i) m->curr_768_b[i] += layer->proj_b[i];
        for (int i = 0; i < n; ++i) m->curr_768_b[i] += m->layer_input[i];
        memcpy(m->layer_input, m->curr_768_b, (size_t)n * 4);

        orc_layernorm(m->curr_768, m->curr_768_b, n);
        for (int i = 0; i < n; ++i) m->curr_768[i] *= layer->ln_2_g[i];
        for (int i = 0; i < n; ++i) m->curr_768[i] += layer->ln_2_b[i];

        matmul(m->curr_3072, m->curr_768, &layer->fc_w, m->row_tmp);
        for (int i = 0; i < p->ff_len; ++i) m->curr_3072[i] += layer->fc_b[i];
        orc_gelu(m->curr_3072, p->ff_len);

        matmul(m->curr_768, m->curr_3072, &layer->mlp_proj_w, m->row_tmp);
        for (int i = 0; i < n; ++i) m->curr_768[i] += layer->mlp_proj_b[i];
        for (int i = 0; i < n; ++i) m->layer_input[i] += m->curr_768[i];
    }

    orc_layernorm(m->curr_768, m->layer_input, n);
    for (int i = 0; i < n; ++i) m->curr_768[i] *= m->ln_f_g[i];
    for (int i = 0; i < n; ++i) m->curr_768[i] += m->ln_f_b[i];
    matmul(m->curr_vocab, m->curr_768, &m->lm_head, m->row_tmp);
}
