// Per-token vector ops: RMSNorm, LayerNorm, RoPE, softmax, SiLU gate, unary ops,
// elementwise assign ops and arg-max.  Each replaces one WGSL kernel + Rust
// `dispatch` of the reference (ops/{rms_norm,layernorm,rope,softmax,silu,unary}.*)
// or a wgebra OpAssign.
#include "common.h"
#include "device_utils.h"

using namespace wgml;

namespace {

// ops/rms_norm.wgsl:36-67: out = (x * rsqrt(mean(x^2) + eps)) * w
__global__ __launch_bounds__(256) void rms_norm_kernel(const float *__restrict__ x,
                                                       const float *__restrict__ w,
                                                       float *__restrict__ out, uint32_t n,
                                                       float eps) {
    __shared__ float red[16];
    float ss = 0.f;
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = x[i];
        ss = fmaf(v, v, ss);
    }
    const float total = block_sum(ss, red);
    const float rms = 1.0f / sqrtf(total / (float)n + eps);
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) out[i] = (x[i] * rms) * w[i];
}

// ops/layernorm.wgsl:27-81: two-pass mean / variance, eps 1e-5, no affine.
// gamma/beta (optional) fold the caller's mul_assign + add_assign
// (models/gpt2/transformer.rs:295-302) into the same launch.
__global__ __launch_bounds__(256) void layernorm_kernel(const float *__restrict__ x,
                                                        float *__restrict__ out,
                                                        const float *__restrict__ gamma,
                                                        const float *__restrict__ beta,
                                                        uint32_t n) {
    __shared__ float red[16];
    float s = 0.f;
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) s += x[i];
    const float mean = block_sum(s, red) / (float)n;
    float ss = 0.f;
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
        const float d = x[i] - mean;
        ss = fmaf(d, d, ss);
    }
    const float var = block_sum(ss, red) / (float)n;
    const float scale = 1.0f / sqrtf(var + 1.0e-5f);
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
        float v = (x[i] - mean) * scale;
        if (gamma) v *= gamma[i];
        if (beta) v += beta[i];
        out[i] = v;
    }
}

// ops/rope.wgsl:35-78.  One thread per rotated pair.  Accurate powf/sincosf:
// at position 8k and base 5e5 the angle reaches thousands of radians.
__global__ void rope_kernel(float *__restrict__ q, float *__restrict__ k_base, uint32_t n_pairs,
                            uint32_t head_size, uint32_t kv_dim, DynPos pos, float base_freq,
                            int neox, uint64_t k_pos_stride) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_pairs) return;
    const uint32_t p = dyn_pos(pos);
    float *k = k_base + (size_t)p * k_pos_stride;
    const float head_dim = (float)((i * 2) % head_size);
    const float theta = powf(base_freq, -head_dim / (float)head_size);
    const float m_theta = (float)p * theta;
    float sn, cs;
    sincosf(m_theta, &sn, &cs);
    uint32_t a, b;
    if (!neox) {
        a = i * 2;
        b = a + 1;
    } else {
        const uint32_t head_id = (i * 2) / head_size;
        a = i + head_id * head_size / 2;
        b = a + head_size / 2;
    }
    {
        const float x = q[a], y = q[b];
        q[a] = cs * x - sn * y;
        q[b] = sn * x + cs * y;
    }
    if (i * 2 < kv_dim) {
        const float x = k[a], y = k[b];
        k[a] = cs * x - sn * y;
        k[b] = sn * x + cs * y;
    }
}

// ops/softmax.wgsl:30-92: one workgroup per column.
__global__ __launch_bounds__(256) void softmax_kernel(float *__restrict__ mat, uint32_t nrows,
                                                      uint32_t col_stride) {
    __shared__ float red[16];
    float *col = mat + (size_t)blockIdx.x * col_stride;
    float mx = -3.0e38f;
    for (uint32_t i = threadIdx.x; i < nrows; i += blockDim.x) mx = fmaxf(mx, col[i]);
    mx = block_max(mx, red);
    float s = 0.f;
    for (uint32_t i = threadIdx.x; i < nrows; i += blockDim.x) {
        const float e = expf(col[i] - mx);
        col[i] = e;
        s += e;
    }
    const float denom = block_sum(s, red);
    for (uint32_t i = threadIdx.x; i < nrows; i += blockDim.x) col[i] = col[i] / denom;
}

// ops/silu.wgsl:13-27
__global__ void silu_kernel(float *__restrict__ h1, const float *__restrict__ h2, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float x = h1[i];
    h1[i] = h2[i] * (x / (1.0f + expf(-x)));
}

// ops/unary.wgsl:18-122 / UnaryOp::eval (ops/unary.rs:87-129)
__device__ __forceinline__ float unary_eval(int op, float x, float4 a) {
    switch (op) {
    case WGML_UNARY_ABS: return fabsf(x);
    case WGML_UNARY_SGN: return x > 0.f ? 1.f : (x < 0.f ? -1.f : 0.f);
    case WGML_UNARY_NEG: return -x;
    case WGML_UNARY_STEP: return x > 0.f ? 1.f : 0.f;
    case WGML_UNARY_ELU: return x > 0.f ? x : expf(x) - 1.f;
    case WGML_UNARY_GELU: return gelu_tanh(x);
    case WGML_UNARY_GELU_QUICK: return x * (1.0f / (1.0f + expf(-1.702f * x)));
    case WGML_UNARY_SILU: return x / (1.0f + expf(-x));
    case WGML_UNARY_TANH: return tanhf(x);
    case WGML_UNARY_RELU: return fmaxf(x, 0.f);
    case WGML_UNARY_SIGMOID: return 1.0f / (1.0f + expf(-x));
    case WGML_UNARY_HARD_SIGMOID: return fminf(1.0f, fmaxf(0.0f, (x + 3.0f) / 6.0f));
    case WGML_UNARY_HARD_SWISH: return x * fminf(1.0f, fmaxf(0.0f, (x + 3.0f) / 6.0f));
    case WGML_UNARY_SQR: return x * x;
    case WGML_UNARY_SQRT: return sqrtf(x);
    case WGML_UNARY_LOG: return logf(x);
    case WGML_UNARY_LEAKY_RELU: return fmaxf(x, 0.f) + fminf(x, 0.f) * a.x;
    case WGML_UNARY_CLAMP: return fminf(fmaxf(x, a.x), a.y);
    case WGML_UNARY_SCALE: return x * a.x;
    case WGML_UNARY_ADD_SCALAR: return x + a.x;
    default: return x;
    }
}

__global__ void unary_kernel(float *__restrict__ x, uint32_t n, int op, float4 args) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = unary_eval(op, x[i], args);
}

__global__ void op_assign_kernel(float *__restrict__ a, const float *__restrict__ b, uint32_t n,
                                 int op) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float bv = b[i];
    if (op == WGML_ASSIGN_ADD) a[i] += bv;
    else if (op == WGML_ASSIGN_MUL) a[i] *= bv;
    else a[i] = bv;
}

// models/sampler.rs:54-56: first index of the maximum.  One workgroup; ties go
// to the lower index.  NaN never wins (comparisons with NaN are false), as with
// nalgebra's imax on well-formed logits.  The result is valid in thread 0.
__device__ __forceinline__ uint32_t block_argmax(const float *__restrict__ v, uint32_t n) {
    __shared__ float bv[16];
    __shared__ uint32_t bi[16];
    float best = -INFINITY;
    uint32_t idx = 0xffffffffu;
    // 16 independent loads per round: the scan of a thread is a chain of memory
    // round trips otherwise (125 of them for a 128k vocabulary)
    constexpr int U = 16;
    for (uint32_t i0 = threadIdx.x; i0 < n; i0 += U * blockDim.x) {
        float x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t i = i0 + u * blockDim.x;
            x[u] = i < n ? v[i] : -INFINITY;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t i = i0 + u * blockDim.x;
            if (i < n && (idx == 0xffffffffu || x[u] > best)) {
                best = x[u];
                idx = i;
            }
        }
    }
    // wave reduce (value, index) with xor-shuffles
    for (int off = 32; off >= 1; off >>= 1) {
        const float ob = __shfl_xor(best, off);
        const uint32_t oi = __shfl_xor(idx, off);
        if (ob > best || (ob == best && oi < idx)) {
            best = ob;
            idx = oi;
        }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    if (lane == 0) {
        bv[wave] = best;
        bi[wave] = idx;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < nw; ++w)
            if (bv[w] > best || (bv[w] == best && bi[w] < idx)) {
                best = bv[w];
                idx = bi[w];
            }
    }
    return idx;
}

__global__ __launch_bounds__(1024) void argmax_kernel(const float *__restrict__ v, uint32_t n,
                                                      uint32_t *__restrict__ out) {
    const uint32_t idx = block_argmax(v, n);
    if (threadIdx.x == 0) out[0] = idx;
}

// Greedy sampling + the token loop's bookkeeping on the device
// (ChatLlama2::forward / sample_next_token with temperature 0,
// wgml-chat/src/chat_llama2.rs:51-153, wgml-chat/src/sampler.rs:91-111): records
// the arg-max, picks the next input token (a forced prompt token wins over the
// sample) and advances the position, so that the next step can be enqueued
// without a host round trip.
__global__ __launch_bounds__(1024) void argmax_next_kernel(const float *__restrict__ v, uint32_t n,
                                                           DynState *dyn,
                                                           const uint32_t *__restrict__ prompt,
                                                           uint32_t *__restrict__ tokens_out) {
    const uint32_t idx = block_argmax(v, n);
    if (threadIdx.x == 0) {
        const uint32_t pos = dyn->pos, cnt = dyn->count;
        tokens_out[cnt] = idx;
        dyn->token = (pos + 1 < dyn->n_prompt) ? prompt[pos + 1] : idx;
        dyn->pos = pos + 1;
        dyn->count = cnt + 1;
    }
}

// argmax_next_kernel followed, in the same launch, by what embed_kernel does for the token and
// position just chosen (the same expressions, so the same bits): the next step of the loop needs
// no launch of its own for the embedding.
__global__ __launch_bounds__(1024) void argmax_next_embed_kernel(const float *__restrict__ v, uint32_t n,
                                                                 DynState *dyn,
                                                                 const uint32_t *__restrict__ prompt,
                                                                 uint32_t *__restrict__ tokens_out,
                                                                 const NextEmbed e) {
    __shared__ uint32_t next[2];
    const uint32_t idx = block_argmax(v, n);
    if (threadIdx.x == 0) {
        const uint32_t pos = dyn->pos, cnt = dyn->count;
        tokens_out[cnt] = idx;
        const uint32_t tok = (pos + 1 < dyn->n_prompt) ? prompt[pos + 1] : idx;
        dyn->token = tok;
        dyn->pos = pos + 1;
        dyn->count = cnt + 1;
        next[0] = tok;
        next[1] = pos + 1;
    }
    __syncthreads();
    const uint32_t tok = next[0], pos = next[1];
    for (uint32_t i = threadIdx.x; i < e.dim; i += blockDim.x) {
        float x = e.table[(size_t)tok * e.dim + i];
        if (e.pos_table && pos < e.n_pos) x += e.pos_table[(size_t)pos * e.dim + i];
        e.x[i] = x;
    }
    if (e.rope_cs && threadIdx.x < e.head_size / 2) {
        const float head_dim = (float)(2 * threadIdx.x);
        const float theta = powf(e.rope_base, -head_dim / (float)e.head_size);
        float sn, cs;
        sincosf((float)pos * theta, &sn, &cs);
        reinterpret_cast<float2 *>(e.rope_cs)[threadIdx.x] = make_float2(cs, sn);
    }
}

// state.x.copy_from_view(token_embd.column(token)) (wgml-chat/src/chat_llama2.rs:185-187)
// Also fills the step's RoPE table (if given): (cos, sin) of pos * theta_i for the
// head_size/2 pairs of a head, with the angle formed exactly as ops/rope.wgsl:38-41.
// With `pos_table` (GPT-2's learned positions) the row of the current position is added:
// layer_input = wte[:, token] + wpe[:, pos] (models/gpt2/transformer.rs:277-290).
__global__ void embed_kernel(float *__restrict__ x, const float *__restrict__ table, uint32_t dim,
                             DynPos token, float2 *__restrict__ rope_cs, uint32_t head_size,
                             float rope_base, DynPos pos, const float *__restrict__ pos_table) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < dim) {
        float v = table[(size_t)dyn_pos(token) * dim + i];
        if (pos_table) v += pos_table[(size_t)dyn_pos(pos) * dim + i];
        x[i] = v;
    }
    if (rope_cs && i < head_size / 2) {
        const float head_dim = (float)(2 * i);
        const float theta = powf(rope_base, -head_dim / (float)head_size);
        float sn, cs;
        sincosf((float)dyn_pos(pos) * theta, &sn, &cs);
        rope_cs[i] = make_float2(cs, sn);
    }
}

inline dim3 grid1(uint32_t n, uint32_t t = 256) { return dim3((n + t - 1) / t); }

}  // namespace

namespace wgml {

int launch_rms_norm(wgml_ctx *ctx, float eps, float *out, const float *x, const float *w,
                    uint32_t n) {
    rms_norm_kernel<<<dim3(1), dim3(256), 0, ctx->stream>>>(x, w, out, n, eps);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int launch_layernorm(wgml_ctx *ctx, float *out, const float *x, const float *gamma,
                     const float *beta, uint32_t n) {
    layernorm_kernel<<<dim3(1), dim3(256), 0, ctx->stream>>>(x, out, gamma, beta, n);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int launch_rope(wgml_ctx *ctx, int variant, uint32_t head_size, uint32_t kv_dim, DynPos pos,
                float base_freq, float *q, uint32_t q_len, float *k, uint64_t k_pos_stride) {
    const uint32_t n_pairs = q_len / 2;
    rope_kernel<<<grid1(n_pairs, 64), dim3(64), 0, ctx->stream>>>(
        q, k, n_pairs, head_size, kv_dim, pos, base_freq, variant == WGML_ROPE_NEOX, k_pos_stride);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int launch_softmax(wgml_ctx *ctx, float *mat, uint32_t nrows, uint32_t ncols,
                   uint32_t col_stride) {
    softmax_kernel<<<dim3(ncols), dim3(256), 0, ctx->stream>>>(mat, nrows, col_stride);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int launch_silu(wgml_ctx *ctx, float *h1, const float *h2, uint32_t n) {
    silu_kernel<<<grid1(n), dim3(256), 0, ctx->stream>>>(h1, h2, n);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int launch_unary(wgml_ctx *ctx, int op, float *x, uint32_t n, const float *args4) {
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
    if (args4) a = make_float4(args4[0], args4[1], args4[2], args4[3]);
    unary_kernel<<<grid1(n), dim3(256), 0, ctx->stream>>>(x, n, op, a);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int launch_op_assign(wgml_ctx *ctx, int op, float *a, const float *b, uint32_t n) {
    op_assign_kernel<<<grid1(n), dim3(256), 0, ctx->stream>>>(a, b, n, op);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int launch_argmax(wgml_ctx *ctx, const float *v, uint32_t n, uint32_t *d_out) {
    argmax_kernel<<<dim3(1), dim3(1024), 0, ctx->stream>>>(v, n, d_out);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int launch_embed(wgml_ctx *ctx, float *x, const float *table, uint32_t dim, DynPos token,
                 float *rope_cs, uint32_t head_size, float rope_base, DynPos pos,
                 const float *pos_table) {
    embed_kernel<<<grid1(dim), dim3(256), 0, ctx->stream>>>(
        x, table, dim, token, reinterpret_cast<float2 *>(rope_cs), head_size, rope_base, pos,
        pos_table);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int launch_argmax_next(wgml_ctx *ctx, const float *v, uint32_t n, DynState *dyn,
                       const uint32_t *prompt, uint32_t *tokens_out, const NextEmbed *embed) {
    if (embed) {
        if (embed->rope_cs && embed->head_size / 2 > 1024)
            return set_error(WGML_E_UNSUPPORTED, "argmax_next: head_size %u too large", embed->head_size);
        argmax_next_embed_kernel<<<dim3(1), dim3(1024), 0, ctx->stream>>>(v, n, dyn, prompt, tokens_out,
                                                                         *embed);
    } else {
        argmax_next_kernel<<<dim3(1), dim3(1024), 0, ctx->stream>>>(v, n, dyn, prompt, tokens_out);
    }
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

}  // namespace wgml

extern "C" {

int wgml_rms_norm(wgml_ctx *ctx, float eps, wgml_view out, wgml_view x, wgml_view w) {
    WGML_REQUIRE(ctx != nullptr, "wgml_rms_norm: null context");
    WGML_TRY(check_view(out, "wgml_rms_norm: out"));
    WGML_TRY(check_view(x, "wgml_rms_norm: x"));
    WGML_TRY(check_view(w, "wgml_rms_norm: w"));
    WGML_REQUIRE(x.len > 0 && out.len == x.len && w.len == x.len,
                 "RmsNorm: dimension mismatch (out %u, x %u, w %u)", out.len, x.len, w.len);
    return launch_rms_norm(ctx, eps, view_ptr(out), view_ptr(x), view_ptr(w), x.len);
}

int wgml_layernorm(wgml_ctx *ctx, wgml_view out, wgml_view x) {
    WGML_REQUIRE(ctx != nullptr, "wgml_layernorm: null context");
    WGML_TRY(check_view(out, "wgml_layernorm: out"));
    WGML_TRY(check_view(x, "wgml_layernorm: x"));
    WGML_REQUIRE(x.len > 0 && out.len == x.len, "LayerNorm: dimension mismatch.");
    return launch_layernorm(ctx, view_ptr(out), view_ptr(x), nullptr, nullptr, x.len);
}

int wgml_rope(wgml_ctx *ctx, int variant, const wgml_rope_config *cfg, wgml_view q, wgml_view k) {
    WGML_REQUIRE(ctx && cfg, "wgml_rope: null argument");
    WGML_TRY(check_view(q, "wgml_rope: q"));
    WGML_TRY(check_view(k, "wgml_rope: k"));
    WGML_REQUIRE(variant == WGML_ROPE_ORIGINAL || variant == WGML_ROPE_NEOX,
                 "wgml_rope: unknown variant %d", variant);
    WGML_REQUIRE(q.len % 2 == 0 && k.len % 2 == 0, "RoPE: vector lengths must be even");
    WGML_REQUIRE(q.len >= k.len,
                 "The Query vector must be larger than, or as large as, the Key vector.");
    WGML_REQUIRE(cfg->head_size > 0 && cfg->head_size % 2 == 0 && q.len % cfg->head_size == 0,
                 "RoPE: head_size %u does not divide the query length %u", cfg->head_size, q.len);
    WGML_REQUIRE(cfg->kv_dim <= k.len, "RoPE: kv_dim %u exceeds the key length %u", cfg->kv_dim,
                 k.len);
    DynPos pos{nullptr, cfg->pos};
    return launch_rope(ctx, variant, cfg->head_size, cfg->kv_dim, pos, cfg->base_freq, view_ptr(q),
                       q.len, view_ptr(k), 0);
}

int wgml_softmax(wgml_ctx *ctx, wgml_view mat, uint32_t nrows, uint32_t ncols,
                 uint32_t col_stride) {
    WGML_REQUIRE(ctx != nullptr, "wgml_softmax: null context");
    WGML_TRY(check_view(mat, "wgml_softmax: mat"));
    WGML_REQUIRE(nrows > 0 && ncols > 0 && col_stride >= nrows,
                 "wgml_softmax: bad shape %ux%u stride %u", nrows, ncols, col_stride);
    WGML_REQUIRE((uint64_t)(ncols - 1) * col_stride + nrows <= mat.len,
                 "wgml_softmax: shape exceeds the view");
    return launch_softmax(ctx, view_ptr(mat), nrows, ncols, col_stride);
}

int wgml_silu(wgml_ctx *ctx, wgml_view h1, wgml_view h2) {
    WGML_REQUIRE(ctx != nullptr, "wgml_silu: null context");
    WGML_TRY(check_view(h1, "wgml_silu: h1"));
    WGML_TRY(check_view(h2, "wgml_silu: h2"));
    WGML_REQUIRE(h1.len == h2.len, "Silu: dimension mismatch (%u vs %u)", h1.len, h2.len);
    if (h1.len == 0) return WGML_OK;
    return launch_silu(ctx, view_ptr(h1), view_ptr(h2), h1.len);
}

int wgml_unary_inplace(wgml_ctx *ctx, int op, wgml_view x, const float *args4) {
    WGML_REQUIRE(ctx != nullptr, "wgml_unary_inplace: null context");
    WGML_TRY(check_view(x, "wgml_unary_inplace: x"));
    WGML_REQUIRE(op >= WGML_UNARY_ABS && op <= WGML_UNARY_ADD_SCALAR,
                 "wgml_unary_inplace: unknown op %d", op);
    // ops/unary.rs:173-176: ops with arguments panic when none are given.
    WGML_REQUIRE(op < WGML_UNARY_LEAKY_RELU || args4 != nullptr,
                 "wgml_unary_inplace: op %d needs arguments", op);
    if (x.len == 0) return WGML_OK;
    return launch_unary(ctx, op, view_ptr(x), x.len, args4);
}

int wgml_op_assign(wgml_ctx *ctx, int op, wgml_view a, wgml_view b) {
    WGML_REQUIRE(ctx != nullptr, "wgml_op_assign: null context");
    WGML_TRY(check_view(a, "wgml_op_assign: a"));
    WGML_TRY(check_view(b, "wgml_op_assign: b"));
    WGML_REQUIRE(op >= WGML_ASSIGN_ADD && op <= WGML_ASSIGN_COPY, "wgml_op_assign: unknown op %d",
                 op);
    WGML_REQUIRE(a.len == b.len, "OpAssign: dimension mismatch (%u vs %u)", a.len, b.len);
    if (a.len == 0) return WGML_OK;
    return launch_op_assign(ctx, op, view_ptr(a), view_ptr(b), a.len);
}

int wgml_argmax(wgml_ctx *ctx, wgml_view logits, uint32_t *out_index) {
    WGML_REQUIRE(ctx && out_index, "wgml_argmax: null argument");
    WGML_TRY(check_view(logits, "wgml_argmax: logits"));
    WGML_REQUIRE(logits.len > 0, "wgml_argmax: empty vector");
    WGML_TRY(launch_argmax(ctx, view_ptr(logits), logits.len, ctx->d_scalar));
    WGML_CHECK_HIP(hipMemcpyAsync(ctx->h_scalar, ctx->d_scalar, 4, hipMemcpyDeviceToHost,
                                  ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    *out_index = ctx->h_scalar[0];
    return WGML_OK;
}

}  // extern "C"
