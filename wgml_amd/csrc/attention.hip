// KV-cache softmax attention for one query token.  Replaces
// BatchedMultiqueryAttention::{dispatch, dispatch_multi} and the attention WGSL
// kernels of the reference (ops/batched_multiquery_attention.rs:55-139,
// ops/batched_multiquery_attention.wgsl:26-100), with the softmax
// (ops/softmax.wgsl) fused in.
//
// One launch covers all heads.  The positions 0..pos are cut into chunks; each
// *wave* streams one chunk of K and V rows for one KV head and keeps a running
// (max, sum, weighted-V) triple per query head of the group ("online softmax"),
// so K and V are read exactly once per KV head even with grouped queries.  The
// four waves of a workgroup merge through LDS; workgroups merge through a small
// workspace and a second, tiny kernel.  With few positions a single workgroup
// per head group writes the result directly.
//
// Lane layout: lane L holds dimensions L, L+64, L+128, ... of a head
// (coalesced 256-byte loads per K/V row segment).
#include "common.h"
#include "device_utils.h"

using namespace wgml;

namespace {

struct AttnArgs {
    const float *q, *kc, *vc;
    float *att;  // optional: raw scores here, normalised by the merge kernel
    float *xb;
    float *ws;  // partials: [head][wg_y][2 + HSP]
    uint32_t seq_len, kv_dim, kv_mul, n_heads, head_size;
    DynPos pos;
    uint32_t chunk;  // positions per wave
    uint32_t n_wg_y;
    int direct;  // 1: grid.y == 1 and the workgroup writes xb itself
};

constexpr int WAVES = 4;
constexpr int UNROLL = 4;

template <int NV, int KM>
__global__ __launch_bounds__(WAVES * 64) void attn_split_kernel(const AttnArgs a) {
    constexpr int HSP = NV * 64;
    __shared__ float sm_m[WAVES][KM], sm_l[WAVES][KM];
    __shared__ float sm_acc[WAVES][KM][HSP];

    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t hs = a.head_size;
    const uint32_t pos = dyn_pos(a.pos);
    const uint32_t h0 = blockIdx.x * KM;
    const uint32_t kvh = h0 / a.kv_mul;
    const uint32_t c = blockIdx.y * WAVES + wave;
    const uint32_t t0 = c * a.chunk;
    const uint32_t t1 = min(t0 + a.chunk, pos + 1);
    const float sqrt_hs = sqrtf((float)hs);

    float q[KM][NV], acc[KM][NV], mx[KM], l[KM];
#pragma unroll
    for (int m = 0; m < KM; ++m) {
        mx[m] = -INFINITY;
        l[m] = 0.f;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const uint32_t d = lane + 64 * v;
            q[m][v] = d < hs ? a.q[(size_t)(h0 + m) * hs + d] : 0.f;
            acc[m][v] = 0.f;
        }
    }

    const float *kb = a.kc + (size_t)kvh * hs;
    const float *vb = a.vc + (size_t)kvh * hs;
    for (uint32_t t = t0; t < t1; t += UNROLL) {
        float kr[UNROLL][NV], vr[UNROLL][NV];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const uint32_t tt = min(t + u, t1 - 1);
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const uint32_t d = lane + 64 * v;
                kr[u][v] = d < hs ? kb[(size_t)tt * a.kv_dim + d] : 0.f;
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const uint32_t tt = min(t + u, t1 - 1);
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const uint32_t d = lane + 64 * v;
                vr[u][v] = d < hs ? vb[(size_t)tt * a.kv_dim + d] : 0.f;
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if (t + u < t1) {
#pragma unroll
                for (int m = 0; m < KM; ++m) {
                    float part = 0.f;
#pragma unroll
                    for (int v = 0; v < NV; ++v) part = fmaf(q[m][v], kr[u][v], part);
                    const float s = wave_sum(part) / sqrt_hs;
                    if (a.att && lane == 0) a.att[(size_t)(h0 + m) * a.seq_len + t + u] = s;
                    const float mn = fmaxf(mx[m], s);
                    const float sc = __expf(mx[m] - mn);
                    const float p = __expf(s - mn);
                    l[m] = fmaf(l[m], sc, p);
#pragma unroll
                    for (int v = 0; v < NV; ++v) acc[m][v] = fmaf(acc[m][v], sc, p * vr[u][v]);
                    mx[m] = mn;
                }
            }
        }
    }

    // merge the waves of this workgroup
#pragma unroll
    for (int m = 0; m < KM; ++m) {
        if (lane == 0) {
            sm_m[wave][m] = mx[m];
            sm_l[wave][m] = l[m];
        }
#pragma unroll
        for (int v = 0; v < NV; ++v) sm_acc[wave][m][lane + 64 * v] = acc[m][v];
    }
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < KM * HSP; i += blockDim.x) {
        const uint32_t m = i / HSP, d = i % HSP;
        float M = sm_m[0][m];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) M = fmaxf(M, sm_m[w][m]);
        float L = 0.f, o = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float mw = sm_m[w][m];
            const float wgt = mw == -INFINITY ? 0.f : __expf(mw - M);
            L = fmaf(sm_l[w][m], wgt, L);
            o = fmaf(sm_acc[w][m][d], wgt, o);
        }
        if (a.direct) {
            if (d < hs) a.xb[(size_t)(h0 + m) * hs + d] = o / L;
        } else {
            float *p = a.ws + ((size_t)(h0 + m) * a.n_wg_y + blockIdx.y) * (2 + HSP);
            if (d == 0) {
                p[0] = M;
                p[1] = L;
            }
            p[2 + d] = o;
        }
    }
}

// Merges the per-workgroup partials of one head; optionally normalises `att`.
__global__ __launch_bounds__(256) void attn_merge_kernel(const AttnArgs a, uint32_t hsp) {
    const uint32_t h = blockIdx.x;
    const uint32_t pos = dyn_pos(a.pos);
    const uint32_t stride = 2 + hsp;
    const float *base = a.ws + (size_t)h * a.n_wg_y * stride;
    // workgroups whose chunks start beyond pos hold empty partials
    const uint32_t per_wg = a.chunk * WAVES;
    const uint32_t n_used = min(a.n_wg_y, pos / per_wg + 1);
    float M = -INFINITY;
    for (uint32_t y = 0; y < n_used; ++y) M = fmaxf(M, base[(size_t)y * stride]);
    float L = 0.f;
    for (uint32_t y = 0; y < n_used; ++y) {
        const float my = base[(size_t)y * stride];
        const float wgt = my == -INFINITY ? 0.f : __expf(my - M);
        L = fmaf(base[(size_t)y * stride + 1], wgt, L);
    }
    for (uint32_t d = threadIdx.x; d < a.head_size; d += blockDim.x) {
        float o = 0.f;
        for (uint32_t y = 0; y < n_used; ++y) {
            const float my = base[(size_t)y * stride];
            const float wgt = my == -INFINITY ? 0.f : __expf(my - M);
            o = fmaf(base[(size_t)y * stride + 2 + d], wgt, o);
        }
        a.xb[(size_t)h * a.head_size + d] = o / L;
    }
    if (a.att) {
        float *att = a.att + (size_t)h * a.seq_len;
        for (uint32_t t = threadIdx.x; t <= pos; t += blockDim.x) att[t] = expf(att[t] - M) / L;
    }
}

int ensure_ws(wgml_ctx *ctx, size_t bytes) {
    if (bytes <= ctx->attn_ws_bytes) return WGML_OK;
    // The old buffer is kept until the context goes: recorded launches (HIP graphs)
    // may still point at it, and it is large enough for the plans they were made for.
    if (ctx->attn_ws) ctx->retired.push_back(ctx->attn_ws);
    ctx->attn_ws = nullptr;
    ctx->attn_ws_bytes = 0;
    hipError_t e = hipMalloc((void **)&ctx->attn_ws, bytes);
    if (e != hipSuccess)
        return set_error(WGML_E_OOM, "attention workspace hipMalloc(%zu) failed: %s", bytes,
                         hipGetErrorString(e));
    ctx->attn_ws_bytes = bytes;
    return WGML_OK;
}

template <int NV>
int launch_nv(wgml_ctx *ctx, const AttnArgs &a, int km, dim3 grid) {
    const dim3 block(WAVES * 64);
    switch (km) {
    case 8: attn_split_kernel<NV, 8><<<grid, block, 0, ctx->stream>>>(a); break;
    case 4: attn_split_kernel<NV, 4><<<grid, block, 0, ctx->stream>>>(a); break;
    case 2: attn_split_kernel<NV, 2><<<grid, block, 0, ctx->stream>>>(a); break;
    default: attn_split_kernel<NV, 1><<<grid, block, 0, ctx->stream>>>(a); break;
    }
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

}  // namespace

namespace wgml {

// `plan_positions`: the number of positions the grid is sized for (pos+1 for a
// one-off launch, seq_len when the launch is replayed for growing positions).
struct AttnPlan {
    int nv, km;
    uint32_t groups, chunk, n_wg_y, hsp;
};

static int make_plan(wgml_ctx *ctx, const wgml_attn_params &p, uint32_t plan_positions,
                     AttnPlan &pl) {
    const uint32_t hs = p.head_size;
    if (hs == 0 || hs > 256)
        return set_error(WGML_E_UNSUPPORTED, "attention: head_size %u not in 1..256", hs);
    pl.nv = (int)((hs + 63) / 64);
    pl.km = 1;
    if (p.kv_mul == 2 || p.kv_mul == 4 || p.kv_mul == 8) pl.km = (int)p.kv_mul;
    // LDS: WAVES*km*(nv*64+2) floats; keep it modest for large heads
    while (pl.km > 1 && (size_t)WAVES * pl.km * (pl.nv * 64 + 2) * 4 > 48 * 1024) pl.km >>= 1;
    pl.groups = p.n_heads / pl.km;
    const uint32_t target_waves = 8u * (ctx->n_cu > 0 ? (uint32_t)ctx->n_cu : 256u);
    uint32_t chunk =
        (uint32_t)(((uint64_t)plan_positions * pl.groups + target_waves - 1) / target_waves);
    chunk = ((chunk + 7) / 8) * 8;
    if (chunk < 16) chunk = 16;
    pl.chunk = chunk;
    const uint32_t n_chunks = (plan_positions + chunk - 1) / chunk;
    pl.n_wg_y = (n_chunks + WAVES - 1) / WAVES;
    pl.hsp = (uint32_t)pl.nv * 64;
    return WGML_OK;
}

// Sizes the partials workspace for a launch planned for `plan_positions`
// (so that no allocation happens while launches are being recorded).
int reserve_attention_workspace(wgml_ctx *ctx, const wgml_attn_params &p, uint32_t plan_positions) {
    AttnPlan pl;
    WGML_TRY(make_plan(ctx, p, plan_positions, pl));
    return ensure_ws(ctx, (size_t)p.n_heads * pl.n_wg_y * (2 + pl.hsp) * 4);
}

int launch_attention_planned(wgml_ctx *ctx, const wgml_attn_params &p, DynPos pos,
                             uint32_t plan_positions, const float *q, const float *kc,
                             const float *vc, float *att, float *xb) {
    AttnPlan pl;
    WGML_TRY(make_plan(ctx, p, plan_positions, pl));
    const uint32_t hs = p.head_size;
    const int nv = pl.nv, km = pl.km;
    const uint32_t groups = pl.groups, chunk = pl.chunk, n_wg_y = pl.n_wg_y;

    AttnArgs a;
    a.q = q;
    a.kc = kc;
    a.vc = vc;
    a.att = att;
    a.xb = xb;
    a.seq_len = p.seq_len;
    a.kv_dim = p.kv_dim;
    a.kv_mul = p.kv_mul;
    a.n_heads = p.n_heads;
    a.head_size = hs;
    a.pos = pos;
    a.chunk = chunk;
    a.n_wg_y = n_wg_y;
    a.direct = (n_wg_y == 1 && att == nullptr) ? 1 : 0;
    a.ws = nullptr;
    const uint32_t hsp = pl.hsp;
    if (!a.direct) {
        WGML_TRY(ensure_ws(ctx, (size_t)p.n_heads * n_wg_y * (2 + hsp) * 4));
        a.ws = ctx->attn_ws;
    }
    const dim3 grid(groups, n_wg_y);
    switch (nv) {
    case 1: WGML_TRY(launch_nv<1>(ctx, a, km, grid)); break;
    case 2: WGML_TRY(launch_nv<2>(ctx, a, km, grid)); break;
    case 3: WGML_TRY(launch_nv<3>(ctx, a, km, grid)); break;
    default: WGML_TRY(launch_nv<4>(ctx, a, km, grid)); break;
    }
    if (!a.direct) {
        attn_merge_kernel<<<dim3(p.n_heads), dim3(256), 0, ctx->stream>>>(a, hsp);
        WGML_CHECK_LAUNCH();
        ctx->launches++;
    }
    return WGML_OK;
}

int launch_attention(wgml_ctx *ctx, const wgml_attn_params &p, DynPos pos, const float *q,
                     const float *kc, const float *vc, float *att, float *xb) {
    return launch_attention_planned(ctx, p, pos, pos.ptr ? p.seq_len : pos.val + 1, q, kc, vc, att,
                                    xb);
}

}  // namespace wgml

extern "C" {

int wgml_attention(wgml_ctx *ctx, const wgml_attn_params *p, wgml_view q, wgml_view key_cache,
                   wgml_view value_cache, wgml_view att, wgml_view xb) {
    WGML_REQUIRE(ctx && p, "wgml_attention: null argument");
    WGML_TRY(check_view(q, "wgml_attention: q"));
    WGML_TRY(check_view(key_cache, "wgml_attention: key_cache"));
    WGML_TRY(check_view(value_cache, "wgml_attention: value_cache"));
    WGML_TRY(check_view(xb, "wgml_attention: xb"));
    WGML_REQUIRE(p->n_heads > 0 && p->head_size > 0 && p->kv_mul > 0 &&
                     p->n_heads % p->kv_mul == 0,
                 "wgml_attention: bad head configuration (%u heads, kv_mul %u)", p->n_heads,
                 p->kv_mul);
    WGML_REQUIRE(p->kv_dim == p->n_heads / p->kv_mul * p->head_size,
                 "wgml_attention: kv_dim %u != n_kv_heads * head_size", p->kv_dim);
    WGML_REQUIRE(p->pos < p->seq_len, "wgml_attention: pos %u outside seq_len %u", p->pos,
                 p->seq_len);
    const uint64_t dim = (uint64_t)p->n_heads * p->head_size;
    WGML_REQUIRE(q.len == dim && xb.len == dim, "wgml_attention: q/xb must have %llu elements",
                 (unsigned long long)dim);
    const uint64_t need = (uint64_t)(p->pos + 1) * p->kv_dim;
    WGML_REQUIRE(key_cache.len >= need && value_cache.len >= need,
                 "wgml_attention: KV cache views shorter than (pos+1)*kv_dim");
    float *att_ptr = nullptr;
    if (att.buf) {
        WGML_TRY(check_view(att, "wgml_attention: att"));
        WGML_REQUIRE((uint64_t)att.len >= (uint64_t)p->n_heads * p->seq_len,
                     "wgml_attention: att needs seq_len*n_heads elements");
        att_ptr = view_ptr(att);
    }
    DynPos pos{nullptr, p->pos};
    return launch_attention(ctx, *p, pos, view_ptr(q), view_ptr(key_cache),
                            view_ptr(value_cache), att_ptr, view_ptr(xb));
}

}  // extern "C"
