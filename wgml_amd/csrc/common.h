// Internal declarations shared by the library's translation units.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/wgml_hip.h"

namespace wgml {

// ---- errors ---------------------------------------------------------------
int set_error(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define WGML_CHECK_HIP(expr)                                                              \
    do {                                                                                  \
        hipError_t e__ = (expr);                                                          \
        if (e__ != hipSuccess)                                                            \
            return ::wgml::set_error(WGML_E_HIP, "%s failed: %s (%s:%d)", #expr,          \
                                     hipGetErrorString(e__), __FILE__, __LINE__);         \
    } while (0)

#define WGML_REQUIRE(cond, ...)                                                           \
    do {                                                                                  \
        if (!(cond)) return ::wgml::set_error(WGML_E_INVALID, __VA_ARGS__);               \
    } while (0)

#define WGML_TRY(expr)                                                                    \
    do {                                                                                  \
        int rc__ = (expr);                                                                \
        if (rc__ != WGML_OK) return rc__;                                                 \
    } while (0)

// Reports a launch-configuration error of the kernel just launched.
#define WGML_CHECK_LAUNCH() WGML_CHECK_HIP(hipGetLastError())

}  // namespace wgml

// ---- handles ----------------------------------------------------------------
// What a context remembers about a kernel it launches with dynamic LDS: whether it has opted
// in to more than 64 KB, and how many workgroups fit a CU at the LDS size last used.
struct wgml_kernel_info {
    bool opted_in = false;
    size_t lds = ~size_t(0);
    int blocks_per_cu = 0;
};

struct wgml_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    int n_cu = 0;
    char name[128] = {0};
    // scratch for device-side arg-max results (2 x u32) + pinned mirror
    uint32_t *d_scalar = nullptr;
    uint32_t *h_scalar = nullptr;
    // scratch for split attention partials, grown on demand
    float *attn_ws = nullptr;
    size_t attn_ws_bytes = 0;
    std::vector<void *> retired;  // outgrown workspaces, freed with the context
    // device address of the library's fixed scratch array on this context's device
    // (wgml_attention_noalloc), looked up when the context is created
    float *noalloc_scratch = nullptr;
    // f16 copy of the activations of a batched matrix product (+ one scale per token),
    // grown on demand
    void *prefill_xh = nullptr;
    void *prefill_xl = nullptr;  // low parts of the same activations (inside the same allocation)
    size_t prefill_xh_bytes = 0;
    int gemm_precise = 1;  // batched products: 1 = split-f16 operands (fp32-grade), 0 = f16
    float *prefill_xscale = nullptr;
    // partial sums of batched products whose K range is split between workgroups
    float *gemm_part = nullptr;
    size_t gemm_part_bytes = 0;
    // > 0: the last batched product left this many partial sums per element in gemm_part
    // for the next kernel to add to its output (launch_prefill_prep or launch_gemm_flush)
    uint32_t gemm_pending_ks = 0;
    uint32_t gemm_pending_pair = 0;  // those sums are a gate / up pair for a gated launch_prefill_prep
    uint64_t launches = 0;  // kernels enqueued so far (diagnostics)
    // launch-shape overrides for sweeps and tests (wgml_ctx_set_tuning), 0 = heuristic
    int tuning[WGML_TUNE_COUNT] = {0};
    uint64_t tuning_generation = 0;  // counts changes of `tuning` (recorded launches go stale)
    std::unordered_map<const void *, wgml_kernel_info> kernel_info;
    // Buffers, matrices and models keep their context alive: the device objects
    // are torn down when the last reference goes, whatever order handles are
    // destroyed in.
    int refs = 1;
};

struct wgml_buf {
    wgml_ctx *ctx = nullptr;
    void *ptr = nullptr;
    uint64_t bytes = 0;
};

// Device layout of a quantized matrix.
//   F32 : row-major f32.
//   Q4_K: the GGUF bytes unchanged (144-byte super-blocks, 16-byte aligned).
//   Q8_0: two planes: `qs` (nrows*ncols int8, row-major) then `d`
//         (nrows*ncols/32 f16), so that quants load as aligned 128-bit words.
//   Q6_K: four planes: ql (128 B/block), qh (64 B/block), scales (16 B/block),
//         d (2 B/block), each row-major in block order.
// Plane offsets are multiples of 256 bytes; the byte total equals the GGUF size
// up to that padding.
struct wgml_qmat {
    wgml_ctx *ctx = nullptr;
    int type = 0;
    uint32_t nrows = 0, ncols = 0;
    uint64_t gguf_bytes = 0;
    uint8_t *base = nullptr;  // device allocation
    uint64_t alloc_bytes = 0;
    uint8_t *p0 = nullptr, *p1 = nullptr, *p2 = nullptr, *p3 = nullptr;  // planes
    // upper bound on |w| over the dequantized matrix (Q8_0 / Q4_K / Q6_K; inf for NaN / inf
    // scales): the batched products need it below kGemmMaxWeight
    float max_abs = 0.f;
};

// The batched products (prefill.hip) expand weights into f16 times 2^8: a dequantized weight
// beyond 65504 / 2^8 (the largest finite f16) would round to infinity there, so a matrix whose
// bound exceeds this goes through the per-token kernels, which take any f32 value.
constexpr float kGemmMaxWeight = 65504.f / 256.f;  // 255.875

namespace wgml {

inline float *view_ptr(const wgml_view &v) {
    return reinterpret_cast<float *>(v.buf->ptr) + v.offset;
}

// True when the environment variable WGML_DISABLE_GRAPHS is set to a non-zero
// value: recorded launch sequences are then enqueued launch by launch instead of
// being replayed as HIP graphs (same kernels, same order; useful under profilers
// that cannot trace graph launches).
bool graphs_disabled();
int resolve_noalloc_scratch(wgml_ctx *ctx);  // attention.hip, where the array lives
void ctx_retain(wgml_ctx *ctx);
void ctx_release(wgml_ctx *ctx);

// Validates that a view lies inside its buffer.
int check_view(const wgml_view &v, const char *what);

// Dynamic per-token scalars read by kernels from device memory so that one
// captured launch sequence can be replayed for every position.
struct DynPos {
    const uint32_t *ptr;  // if non-null, *ptr is used
    uint32_t val;
};
// The value was written by an earlier launch and does not change while a kernel that reads
// it runs, so it is read through the constant address space: a scalar load, which takes no
// vector-memory slot and leaves the waits on the vector loads around it exact (behind a load
// through a generic pointer the compiler waits for every outstanding vector load).
__device__ __forceinline__ uint32_t dyn_pos(const DynPos &p) {
    typedef const __attribute__((address_space(4))) uint32_t *const_u32_ptr;
    return p.ptr ? *(const_u32_ptr)(uintptr_t)p.ptr : p.val;
}

// ---- internal launchers (async on ctx->stream, raw device pointers) --------
// Unmerged output of a decode-attention launch: for every head, n partial results of the
// flash-decoding scheme: weighted sums of V rows o[head][y][hsp] (hsp floats per row, the
// first head_size used) and (running maximum, sum of weights) ml[head][y][2].  A partial with
// maximum -inf is neutral and its o row is undefined.  The merged output is
//   xb[head][d] = sum_y o[y][d] e^(m_y - M) / sum_y l_y e^(m_y - M),   M = max_y m_y.
struct AttnPartials {
    const float *o = nullptr, *ml = nullptr;
    uint32_t n = 0, hsp = 0, head_size = 0;
};

struct GemvEpilogue {
    // out[r] = acc (+ bias[r]) (+ out[r] if accumulate)
    const float *bias = nullptr;
    int accumulate = 0;
    // out is displaced by (*dyn_pos) * out_pos_stride floats: lets a recorded launch
    // write "the KV-cache column of the current position"
    const uint32_t *dyn_pos = nullptr;
    uint32_t out_pos_stride = 0;
    // if norm_w != null the input is RMS-normalised first: v <- (v * rsqrt(mean(v^2) + eps)) * norm_w
    const float *norm_w = nullptr;
    float norm_eps = 0.f;
    // if ln_gamma != null the input goes through LayerNorm first (eps 1e-5, as
    // ops/layernorm.rs:46-53): v <- (v - mean) / sqrt(var + 1e-5) * ln_gamma + ln_beta
    const float *ln_gamma = nullptr, *ln_beta = nullptr;
    // activation applied to acc + bias before it is stored: 0 none, 1 GELU (tanh form,
    // ops/unary.rs:106-110)
    int act = 0;
    // partials.n > 0: the input vector is the merged attention output of these partial results
    // (the `v` argument is ignored); integer-dot kernels of Q8_0 / Q4_K / Q6_K only, up to 16
    // partial results per head
    AttnPartials partials;
};

// One launch for up to three quantized matrices that consume the same vector
// (Q8_0 / Q4_K / Q6_K, formats may differ between the matrices).
enum { FUSED_PLAIN = 0, FUSED_ROPE = 1, FUSED_SILU = 2 };
struct FusedGemvJob {
    const wgml_qmat *a = nullptr;  // the matrix (SILU: the gate matrix)
    const wgml_qmat *b = nullptr;  // SILU only: the up matrix
    float *out = nullptr;
    const float *bias = nullptr;
    int mode = FUSED_PLAIN;  // ROPE: adjacent-pair rotation of the output rows by pos
    int accumulate = 0;
    uint32_t out_pos_stride = 0;  // out += pos * out_pos_stride
    // the job covers rows [row0, row0 + nrows) of `a` (nrows 0: all of them); `bias`
    // and `out` are indexed from the job's first row
    uint32_t row0 = 0, nrows = 0;
};
struct FusedGemv {
    FusedGemvJob jobs[3];
    int njobs = 0;
    const float *x = nullptr;
    const float *norm_w = nullptr;  // optional fused RMSNorm of x
    float norm_eps = 0.f;
    const float *ln_gamma = nullptr, *ln_beta = nullptr;  // optional fused LayerNorm of x
    DynPos pos{nullptr, 0};
    uint32_t head_size = 0;
    float rope_base = 10000.f;
    // optional table of (cos, sin) pairs for the current position, one per rotated
    // pair of a head (head_size / 2 entries); computed in-kernel when null
    const float *rope_cs = nullptr;
};
bool gemv_fused_supported(const wgml_qmat *m);
// the matrices can share one launch_gemv_fused (with the context's settings): one format, or a
// mix of Q4_K / Q6_K / Q8_0
bool gemv_fused_set_supported(const wgml_ctx *ctx, const wgml_qmat *const *mats, int n);
// launch_gemv_quant takes GemvEpilogue::partials for this matrix (with the context's settings)
bool gemv_partials_supported(const wgml_ctx *ctx, const wgml_qmat *m);
int launch_gemv_fused(wgml_ctx *ctx, const FusedGemv &f);

int launch_gemv_quant(wgml_ctx *ctx, float *out, const wgml_qmat *m, const float *v,
                      const GemvEpilogue &ep);
int launch_gemv_f32(wgml_ctx *ctx, float *out, const float *a, uint32_t nrows, uint32_t ncols,
                    int transposed, const float *v);
int launch_rms_norm(wgml_ctx *ctx, float eps, float *out, const float *x, const float *w,
                    uint32_t n);
int launch_layernorm(wgml_ctx *ctx, float *out, const float *x, const float *gamma,
                     const float *beta, uint32_t n);
int launch_rope(wgml_ctx *ctx, int variant, uint32_t head_size, uint32_t kv_dim, DynPos pos,
                float base_freq, float *q, uint32_t q_len, float *k, uint64_t k_pos_stride);
int launch_softmax(wgml_ctx *ctx, float *mat, uint32_t nrows, uint32_t ncols, uint32_t col_stride);
int launch_attention(wgml_ctx *ctx, const wgml_attn_params &p, DynPos pos, uint32_t cache_rows,
                     const float *q, const float *kc, const float *vc, float *att, float *xb);
// The same with the grid planned for `plan_positions` positions (seq_len when the launch is
// recorded and replayed at growing positions).  `ext_ws`: optional caller-supplied workspace
// for the partial results (ext_ws_bytes bytes) instead of the context's own.
// A recorded decode step is captured once per range of positions ("bucket"): the attention
// launch of a step is planned for the bucket's upper limit rather than for seq_len, so that
// short contexts run the grid that suits them (one workgroup per head group and no partial
// results up to 256 positions, few partials per head after that).  Limits: 256, 512, 1024, ...
// doubling, the last one seq_len.
constexpr int kMaxPlanBuckets = 24;
inline uint32_t plan_bucket(uint32_t pos, uint32_t seq_len, int *index) {
    uint32_t limit = 256;
    int i = 0;
    while (pos >= limit && limit < seq_len && i + 1 < kMaxPlanBuckets) {
        limit <<= 1;
        ++i;
    }
    if (index) *index = i;
    return limit < seq_len ? limit : seq_len;
}
int reserve_attention_workspace(wgml_ctx *ctx, const wgml_attn_params &p, uint32_t plan_positions);
// `keep` (optional): the launch may leave the attention output unmerged, as per-workgroup
// partial results that the caller's next launch merges while it stages its input
// (GemvEpilogue::partials); keep->n > 0 then, and xb has NOT been written.  keep->n == 0: xb
// holds the result as usual.
int launch_attention_planned(wgml_ctx *ctx, const wgml_attn_params &p, DynPos pos,
                             uint32_t plan_positions, uint32_t cache_rows, const float *q,
                             const float *kc, const float *vc, float *att, float *xb,
                             float *ext_ws = nullptr, size_t ext_ws_bytes = 0,
                             AttnPartials *keep = nullptr);
int launch_silu(wgml_ctx *ctx, float *h1, const float *h2, uint32_t n);
int launch_unary(wgml_ctx *ctx, int op, float *x, uint32_t n, const float *args4);
int launch_op_assign(wgml_ctx *ctx, int op, float *a, const float *b, uint32_t n);
int launch_argmax(wgml_ctx *ctx, const float *v, uint32_t n, uint32_t *d_out);
// Token-loop state on the device: {pos, token, n_generated, n_prompt}.
struct DynState {
    uint32_t pos, token, count, n_prompt;
};
int launch_embed(wgml_ctx *ctx, float *x, const float *table, uint32_t dim, DynPos token,
                 float *rope_cs, uint32_t head_size, float rope_base, DynPos pos,
                 const float *pos_table = nullptr);
// What launch_embed does for the token and position that launch_argmax_next has just chosen,
// done by that same launch: the next step of a token loop then starts with its first layer.
struct NextEmbed {
    float *x;
    const float *table;
    uint32_t dim;
    float *rope_cs;  // optional
    uint32_t head_size;
    float rope_base;
    const float *pos_table;  // optional (GPT-2's learned positions)
    uint32_t n_pos;          // rows of pos_table: no row is read for a position beyond them
};
int launch_argmax_next(wgml_ctx *ctx, const float *v, uint32_t n, DynState *dyn,
                       const uint32_t *prompt, uint32_t *tokens_out,
                       const NextEmbed *embed = nullptr);
int launch_dequantize(wgml_ctx *ctx, float *out, const wgml_qmat *m);

// ---- batched products for prompt processing (prefill.hip) ---------------------
constexpr uint32_t kPrefillMaxTokens = 128;
uint32_t prefill_tpad(uint32_t T);  // tokens rounded up to 16, 32, 64 or 128
uint32_t prefill_kpad(uint32_t K);  // columns rounded up to a multiple of 128
int ensure_prefill_scratch(wgml_ctx *ctx, size_t xh_bytes);
// xh[tpad][kpad] (f16) <- x[T][K] (f32, rows x_stride apart): RMS-normalised with
// norm_w first when that is non-null; replaced by up[t][k] * silu(x[t][k]) when `up`
// is non-null.  xscale[tpad] receives what a token's products must be multiplied with.
// If the product before left partial sums for x (defer_reduce), they are added to x first.
int launch_prefill_prep(wgml_ctx *ctx, float *x, uint32_t x_stride, const float *up,
                        const float *norm_w, float eps, void *xh, float *xscale, uint32_t K,
                        uint32_t T);
// Adds partial sums left for x by a product with defer_reduce (no-op if there are none).
int launch_gemm_flush(wgml_ctx *ctx, float *x, uint32_t x_stride, const float *xscale, uint32_t K,
                      uint32_t T);
// xb[t] = attention of q[t] (position pos0 + t) over cache rows 0 .. pos0 + t
int launch_attention_rows(wgml_ctx *ctx, const wgml_attn_params &p, uint32_t pos0, uint32_t T,
                          const float *q, uint32_t q_stride, const float *kc, const float *vc,
                          float *xb, uint32_t xb_stride);
// out[t][r] (rows out_stride apart) = (or +=) sum_k M[r][k] x[t][k] + bias[r]
// defer_reduce: when the product's K range is split between workgroups and it is a plain
// `out += ` of one matrix, the partial sums are left for the caller's next kernel on out
// (launch_prefill_prep or launch_gemm_flush), which must come before anything else reads out
// or writes xscale.  The same for a gate / up pair (two matrices of equal height, `out =`)
// whose next kernel is the gated launch_prefill_prep(gate out, up out): the outputs are then
// never written.
int launch_gemm_quant(wgml_ctx *ctx, float *out, uint32_t out_stride, const wgml_qmat *m,
                      const void *xh, const float *xscale, uint32_t T, const float *bias,
                      int accumulate, bool defer_reduce = false);
// The same for up to three matrices of one format and width that multiply the same
// activations, in one launch.
struct GemmTarget {
    const wgml_qmat *m;
    float *out;
    uint32_t out_stride;
    const float *bias;
    bool rope = false;  // rotate the rows of this product (see GemmRope)
};
// Rotary position encoding of the targets marked `rope`, applied by the kernel that adds up the
// partial sums of a K-split product (the rows of a pair meet there anyway): token t sits at
// position pos0 + t.  `applied` tells the caller whether it happened (not when K was not split
// or a target has an odd number of rows: launch_rope_rows then).
struct GemmRope {
    int variant;  // WGML_ROPE_ORIGINAL or WGML_ROPE_NEOX
    uint32_t head_size, pos0;
    float base_freq;
    bool applied;
};
int launch_gemm_quant_multi(wgml_ctx *ctx, const GemmTarget *targets, int n, const void *xh,
                            const float *xscale, uint32_t T, int accumulate,
                            bool defer_reduce = false, GemmRope *rope = nullptr);
int launch_embed_rows(wgml_ctx *ctx, float *x, const float *table, const uint32_t *d_tokens,
                      uint32_t dim, uint32_t T);
// q (q_len wide) and k (kv_dim wide) of T tokens rotated in place; either may be null
int launch_rope_rows(wgml_ctx *ctx, int variant, uint32_t head_size, uint32_t kv_dim, uint32_t pos0,
                     float base_freq, float *q, uint32_t q_len, uint32_t q_stride, float *k,
                     uint32_t k_stride, uint32_t T);

}  // namespace wgml
