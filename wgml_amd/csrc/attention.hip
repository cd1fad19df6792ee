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
// Lane layout of the general kernel: lane L holds dimensions L, L+64, L+128, ...
// of a head (coalesced 256-byte loads per K/V row segment).
//
// Fast kernel (no score output wanted, head size a multiple of 4, 16-byte aligned
// operands): 16 lanes share a position (float4 loads, 16-lane DPP reductions), a
// wave works on 4 positions at a time (and has those four in flight, no more); the chunk
// per wave is derived from the current position on the device, so every wave of
// a recorded launch has work at any position.  Up to 256 positions one 16-wave
// workgroup per head group does everything and writes the result (one launch, no
// workspace); beyond that 4-wave workgroups write partials for the merge kernel.
// (Merging in the workgroup that arrives last was tried twice and dropped.  With
// device-scope fences every fence is an L2 write-back here, 20 us per launch.  Without
// fences -- partial results stored and loaded at device scope, a relaxed arrival counter
// per head group, every thread waiting for its own stores before the workgroup is counted
// in -- the results equal the merge launch's bit for bit, but the three dependent trips to
// memory (store acknowledgement, counter, loads) cost what the launch costs: +0.6 % on 32
// heads of 128 beyond position 256, -1.2 % on 12 heads of 64, -16 % at 8192 positions of
// 8 KV heads, where one workgroup merges the four heads of its group in turn.)
#include <algorithm>

#include "common.h"
#include "device_utils.h"

using namespace wgml;

namespace {

struct AttnArgs {
    const float *q, *kc, *vc;
    float *att;  // optional: raw scores here, normalised by the merge kernel
    float *xb;
    // partial results of the workgroups that share a head's positions: the weighted sums of V
    // as ws[head][wg_y][HSP] (rows of HSP floats, 16-byte aligned), and (max, sum) as
    // ws_ml[head][wg_y][2]
    float *ws, *ws_ml;
    uint32_t seq_len, kv_dim, kv_mul, n_heads, head_size;
    DynPos pos;
    uint32_t chunk;  // positions per wave
    uint32_t spec_rows;  // rows of the caches that exist (may be read before pos is known)
    uint32_t spec_sets;  // register sets whose quads are requested before pos is known (>= 1)
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
            const size_t slot = (size_t)(h0 + m) * a.n_wg_y + blockIdx.y;
            if (d == 0) {
                a.ws_ml[slot * 2] = M;
                a.ws_ml[slot * 2 + 1] = L;
            }
            a.ws[slot * HSP + d] = o;
        }
    }
}

// Fast kernel: positions are dealt out in quads (4 consecutive positions, one per
// 16-lane row of a wave); quad Q belongs to wave Q % (n_wg_y * nw) of the head
// group, counted over the workgroups.  The assignment does not depend on the
// current position, so the loads for a wave's first quads can be requested before
// the position is known.
__device__ __forceinline__ uint32_t fast_n_used(uint32_t pos, uint32_t n_wg_y, uint32_t nw) {
    const uint32_t nq = pos / 4 + 1;  // quads that hold a position <= pos
    return min(n_wg_y, (nq + nw - 1) / nw);
}

// Merges the per-workgroup partials of one head; optionally normalises `att`.
// All partials are requested at once (a loop of dependent loads would cost one
// memory round trip per partial).
constexpr int MERGE_MAX_Y = 64;
__global__ __launch_bounds__(256) void attn_merge_kernel(const AttnArgs a, uint32_t hsp) {
    __shared__ float sm_w[MERGE_MAX_Y];
    __shared__ float sm_ML[2];
    const uint32_t h = blockIdx.x;
    const uint32_t pos = dyn_pos(a.pos);
    const uint32_t stride = hsp;
    const float *base = a.ws + (size_t)h * a.n_wg_y * stride;
    const float *ml = a.ws_ml + (size_t)h * a.n_wg_y * 2;
    // workgroups whose positions start beyond pos hold no partial
    // (chunk == 0: partials of the fast kernel)
    const uint32_t n_used = a.chunk ? min(a.n_wg_y, pos / (a.chunk * WAVES) + 1)
                                    : fast_n_used(pos, a.n_wg_y, WAVES);
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    float M, L;
    if (n_used <= MERGE_MAX_Y) {
        if (tid < 64) {  // wave 0: one partial per lane
            const float my = lane < n_used ? ml[lane * 2] : -INFINITY;
            const float ly = lane < n_used ? ml[lane * 2 + 1] : 0.f;
            const float mm = wave_max(my);
            const float wgt = my == -INFINITY ? 0.f : __expf(my - mm);
            const float ll = wave_sum(ly * wgt);
            sm_w[lane] = wgt;
            if (lane == 0) {
                sm_ML[0] = mm;
                sm_ML[1] = ll;
            }
        }
        __syncthreads();
        M = sm_ML[0];
        L = sm_ML[1];
        for (uint32_t d = tid; d < a.head_size; d += blockDim.x) {
            float o = 0.f;
            for (uint32_t y0 = 0; y0 < n_used; y0 += 8) {
                float v[8];
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    v[k] = y0 + k < n_used ? base[(size_t)(y0 + k) * stride + d] : 0.f;
#pragma unroll
                for (int k = 0; k < 8; ++k) o = fmaf(v[k], y0 + k < n_used ? sm_w[y0 + k] : 0.f, o);
            }
            a.xb[(size_t)h * a.head_size + d] = o / L;
        }
    } else {
        M = -INFINITY;
        for (uint32_t y = 0; y < n_used; ++y) M = fmaxf(M, ml[y * 2]);
        L = 0.f;
        for (uint32_t y = 0; y < n_used; ++y) {
            const float my = ml[y * 2];
            const float wgt = my == -INFINITY ? 0.f : __expf(my - M);
            L = fmaf(ml[y * 2 + 1], wgt, L);
        }
        for (uint32_t d = tid; d < a.head_size; d += blockDim.x) {
            float o = 0.f;
            for (uint32_t y = 0; y < n_used; ++y) {
                const float my = ml[y * 2];
                const float wgt = my == -INFINITY ? 0.f : __expf(my - M);
                o = fmaf(base[(size_t)y * stride + d], wgt, o);
            }
            a.xb[(size_t)h * a.head_size + d] = o / L;
        }
    }
    if (a.att) {
        float *att = a.att + (size_t)h * a.seq_len;
        for (uint32_t t = tid; t <= pos; t += blockDim.x) att[t] = expf(att[t] - M) / L;
    }
}

// Merge of the fast kernel's partials: every workgroup of the grid has written one
// (a neutral one if it had no position), so nothing depends on the current position
// and all loads go out at once: lane y of every wave fetches (max, sum) of partial y,
// thread d the d-th value of every partial; the weights are formed in registers.
// B: partials fetched per round of loads (16 for short grids; 64 = all in one round for the
// long-context grids, where every extra round is another trip to memory).
template <int B>
__global__ __launch_bounds__(256) void attn_merge_fast_kernel(const AttnArgs a, uint32_t hsp) {
    const uint32_t h = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
    const uint32_t stride = hsp, ny = a.n_wg_y;  // ny <= MERGE_MAX_Y = 64
    const float *base = a.ws + (size_t)h * ny * stride;
    const float *ml = a.ws_ml + (size_t)h * ny * 2;
    const float my = lane < ny ? ml[lane * 2] : -INFINITY;
    const float ly = lane < ny ? ml[lane * 2 + 1] : 0.f;
    float v[B];
    const bool has_d = tid < a.head_size;  // head sizes up to 256: one dimension per thread
    // Loads without conditions (a thread beyond the head reads the head's last dimension, a
    // partial beyond ny the last one: their weights are zero or their results not stored), so
    // that they leave back to back instead of one branch each.
    const uint32_t td = has_d ? tid : a.head_size - 1;
#pragma unroll
    for (int k = 0; k < B; ++k) v[k] = base[(size_t)min((uint32_t)k, ny - 1) * stride + td];
    const float M = wave_max(my);
    const float wgt = my == -INFINITY ? 0.f : __expf(my - M);
    const float L = wave_sum(ly * wgt);
    float o = 0.f;
#pragma unroll
    for (int k = 0; k < B; ++k) {
        const float wk = readlane_f32(wgt, k);
        o = fmaf(wk > 0.f ? v[k] : 0.f, wk, o);  // values of neutral partials were never written
    }
    for (uint32_t y0 = B; y0 < ny; y0 += B) {
#pragma unroll
        for (int k = 0; k < B; ++k) v[k] = base[(size_t)min(y0 + k, ny - 1) * stride + td];
#pragma unroll
        for (int k = 0; k < B; ++k) {
            const float wk = __shfl(wgt, (int)(y0 + k), 64);
            o = fmaf(wk > 0.f ? v[k] : 0.f, wk, o);
        }
    }
    if (has_d) a.xb[(size_t)h * a.head_size + tid] = o / L;
}

// ---------------------------------------------------------------- fast kernel
__device__ __forceinline__ float dot4(const float4 a, const float4 b, float acc) {
    acc = fmaf(a.x, b.x, acc);
    acc = fmaf(a.y, b.y, acc);
    acc = fmaf(a.z, b.z, acc);
    return fmaf(a.w, b.w, acc);
}
__device__ __forceinline__ float4 axpby4(const float4 a, float sa, const float4 b, float sb) {
    return make_float4(fmaf(a.x, sa, b.x * sb), fmaf(a.y, sa, b.y * sb), fmaf(a.z, sa, b.z * sb),
                       fmaf(a.w, sa, b.w * sb));
}
__device__ __forceinline__ float shfl_xor_f32(float v, int mask) { return __shfl_xor(v, mask, 64); }

// NS register sets of QS quads each take turns (NS * QS quads of a wave in flight).  Less is
// more here: one set of one quad -- a wave requests the K and V rows of four positions, waits,
// consumes them and requests the next four; the other waves of the CU cover the wait -- is the
// fastest at every length measured (per layer, attention + merge, us; sets x quads 1x1 / 2x1 /
// 1x2 / 2x2 / 1x4: 32 heads of 128 at position 150: 4.38 / 4.62 / 4.54 / 4.84 / 5.94, at 1000:
// 9.41 / 9.61 / 9.57 / 10.26 / 10.41; 8 KV heads x 4 at 8192: 20.2 / 20.6 / 21.3 / 21.8 / 21.5;
// four sets of two were slower still), as with the GEMV's weight tiles: requests beyond what
// keeps the memory system busy only queue.
template <int NV4, int KM, int NW, int NS = 1, int QS = 1>
__global__ __launch_bounds__(NW * 64) void attn_fast_kernel(const AttnArgs a) {
    constexpr int HSP = NV4 * 64;  // dimension capacity: 16 lanes x 4 x NV4
    __shared__ float sm_m[NW][KM], sm_l[NW][KM];
    __shared__ float sm_acc[NW][KM][HSP];

    const uint32_t lane = threadIdx.x & 63;
    // readfirstlane: tells the compiler that the wave index is uniform (scalar loop control)
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t sub = lane & 15, quarter = lane >> 4;
    const uint32_t hs = a.head_size;
    const uint32_t h0 = blockIdx.x * KM;
    const uint32_t kvh = h0 / a.kv_mul;
    const uint32_t gid = blockIdx.y * NW + wave, total = a.n_wg_y * NW;
    const float inv_sqrt_hs = 1.0f / sqrtf((float)hs);
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
    const float *kb = a.kc + (size_t)kvh * hs;
    const float *vb = a.vc + (size_t)kvh * hs;
    // this lane's float4 number v lies inside the head; if not, it re-reads the head's
    // last float4 (loads stay unconditional 16-byte loads) and q is zero there, so
    // that it adds nothing to a score; its slots of the output are never stored
    bool dv[NV4];
    uint32_t cv[NV4];
#pragma unroll
    for (int v = 0; v < NV4; ++v) {
        dv[v] = (sub + 16 * v) * 4 < hs;
        cv[v] = min(sub + 16 * v, hs / 4 - 1);
    }

    // This wave's quads are gid, gid + total, ...  NS register sets of QS quads
    // each take turns: while one is consumed the others' loads (if NS > 1) are in flight.
    // The quads of the first set are requested before the position is known (`spec_rows` rows
    // of the caches may be read; rows beyond the position are masked out below),
    // the others once it is, and only those that hold a position <= pos.
    float4 kS[NS][QS][NV4], vS[NS][QS][NV4];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
#pragma unroll
        for (int u = 0; u < QS; ++u) {
#pragma unroll
            for (int v = 0; v < NV4; ++v) kS[s][u][v] = vS[s][u][v] = zero4;
        }
    }
    // requests quads number i0 + u (u_begin <= u < QS) of this wave into a set
    auto request = [&](float4(&kk)[QS][NV4], float4(&vv)[QS][NV4], uint32_t i0, uint32_t last,
                       int u_begin, uint32_t nq_limit) {
#pragma unroll
        for (int u = 0; u < QS; ++u) {
            const uint32_t quad = (i0 + u) * total + gid;
            if (u >= u_begin && quad < nq_limit) {  // uniform over the wave
                const uint32_t tt = min(quad * 4 + quarter, last);
                const float4 *kp = reinterpret_cast<const float4 *>(kb + (size_t)tt * a.kv_dim);
                const float4 *vp = reinterpret_cast<const float4 *>(vb + (size_t)tt * a.kv_dim);
#pragma unroll
                for (int v = 0; v < NV4; ++v) kk[u][v] = kp[cv[v]];
#pragma unroll
                for (int v = 0; v < NV4; ++v) vv[u][v] = vp[cv[v]];
            }
        }
    };
    // Quads that lie inside the caches whatever the position are requested right away: those
    // of the first `spec_sets` register sets (one: a recorded step is planned for a range of
    // positions whose lower end lies beyond what the first sets of all waves cover, so nothing
    // is read in vain).
    const uint32_t spec_quads = a.spec_rows / 4;  // whole quads below spec_rows
    int n_spec[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        // the set's leading quads that lie below spec_rows (a wave's quads ascend)
        n_spec[s] = 0;
        if ((uint32_t)s < a.spec_sets) {
#pragma unroll
            for (int u = 0; u < QS; ++u) n_spec[s] += ((uint32_t)(QS * s + u) * total + gid < spec_quads) ? 1 : 0;
        }
        if (n_spec[s]) request(kS[s], vS[s], QS * s, a.spec_rows - 1, 0, spec_quads);
    }

    float4 q[KM][NV4], acc[KM][NV4];
    float mx[KM], l[KM];
#pragma unroll
    for (int m = 0; m < KM; ++m) {
        mx[m] = -INFINITY;
        l[m] = 0.f;
#pragma unroll
        for (int v = 0; v < NV4; ++v) {
            const float4 qv = reinterpret_cast<const float4 *>(a.q + (size_t)(h0 + m) * hs)[cv[v]];
            q[m][v] = make_float4(dv[v] ? qv.x : 0.f, dv[v] ? qv.y : 0.f, dv[v] ? qv.z : 0.f,
                                  dv[v] ? qv.w : 0.f);
            acc[m][v] = zero4;
        }
    }

    const uint32_t pos = dyn_pos(a.pos);
    const uint32_t n_used = fast_n_used(pos, a.n_wg_y, NW);  // workgroups with work
    if (blockIdx.y >= n_used) {
        // no position for this workgroup: a neutral partial (max -inf, sum 0), so that the
        // merge need not know the position to tell which partials count
        if (threadIdx.x < KM) {
            float *p = a.ws_ml + ((size_t)(h0 + threadIdx.x) * a.n_wg_y + blockIdx.y) * 2;
            p[0] = -INFINITY;
            p[1] = 0.f;
        }
        return;
    }
    const uint32_t nq = pos / 4 + 1;
    // online-softmax update with the quads of a set
    auto consume = [&](const float4(&kk)[QS][NV4], const float4(&vv)[QS][NV4], uint32_t i0) {
#pragma unroll
        for (int u = 0; u < QS; ++u) {
            // uniform within each 16-lane row, so the row reductions below see whole rows
            if (((i0 + u) * total + gid) * 4 + quarter <= pos) {
#pragma unroll
                for (int m = 0; m < KM; ++m) {
                    float part = 0.f;
#pragma unroll
                    for (int v = 0; v < NV4; ++v) part = dot4(q[m][v], kk[u][v], part);
                    const float s = row16_sum(part) * inv_sqrt_hs;
                    const float mn = fmaxf(mx[m], s);
                    const float sc = __expf(mx[m] - mn);
                    const float p = __expf(s - mn);
                    l[m] = fmaf(l[m], sc, p);
#pragma unroll
                    for (int v = 0; v < NV4; ++v) acc[m][v] = axpby4(acc[m][v], sc, vv[u][v], p);
                    mx[m] = mn;
                }
            }
        }
    };
#pragma unroll
    for (int s = 0; s < NS; ++s) request(kS[s], vS[s], QS * s, pos, n_spec[s], nq);
    for (uint32_t i0 = 0; i0 * total + gid < nq; i0 += QS * NS) {
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            consume(kS[s], vS[s], i0 + QS * s);
            request(kS[s], vS[s], i0 + QS * s + QS * NS, pos, 0, nq);
        }
    }

    // merge the four quarters of the wave (every lane ends up with the merged state)
#pragma unroll
    for (int step = 16; step <= 32; step <<= 1) {
#pragma unroll
        for (int m = 0; m < KM; ++m) {
            const float om = shfl_xor_f32(mx[m], step), ol = shfl_xor_f32(l[m], step);
            const float M = fmaxf(mx[m], om);
            const float sa = mx[m] == -INFINITY ? 0.f : __expf(mx[m] - M);
            const float sb = om == -INFINITY ? 0.f : __expf(om - M);
            l[m] = fmaf(l[m], sa, ol * sb);
#pragma unroll
            for (int v = 0; v < NV4; ++v) {
                float4 o;
                o.x = shfl_xor_f32(acc[m][v].x, step);
                o.y = shfl_xor_f32(acc[m][v].y, step);
                o.z = shfl_xor_f32(acc[m][v].z, step);
                o.w = shfl_xor_f32(acc[m][v].w, step);
                acc[m][v] = axpby4(acc[m][v], sa, o, sb);
            }
            mx[m] = M;
        }
    }
    // merge the waves of this workgroup
#pragma unroll
    for (int m = 0; m < KM; ++m) {
        if (lane == 0) {
            sm_m[wave][m] = mx[m];
            sm_l[wave][m] = l[m];
        }
        if (quarter == 0) {
#pragma unroll
            for (int v = 0; v < NV4; ++v)
                reinterpret_cast<float4 *>(&sm_acc[wave][m][0])[sub + 16 * v] = acc[m][v];
        }
    }
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < KM * HSP; i += blockDim.x) {
        const uint32_t m = i / HSP, d = i % HSP;
        float M = sm_m[0][m];
#pragma unroll
        for (int w = 1; w < NW; ++w) M = fmaxf(M, sm_m[w][m]);
        float L = 0.f, o = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float mw = sm_m[w][m];
            const float wgt = mw == -INFINITY ? 0.f : __expf(mw - M);
            L = fmaf(sm_l[w][m], wgt, L);
            o = fmaf(sm_acc[w][m][d], wgt, o);
        }
        if (a.n_wg_y == 1) {
            if (d < hs) a.xb[(size_t)(h0 + m) * hs + d] = o / L;
        } else {
            const size_t slot = (size_t)(h0 + m) * a.n_wg_y + blockIdx.y;
            if (d == 0) {
                a.ws_ml[slot * 2] = M;
                a.ws_ml[slot * 2 + 1] = L;
            }
            a.ws[slot * HSP + d] = o;
        }
    }
}

// Scratch of the entry point that allocates nothing (wgml_attention_noalloc): the partial
// results (max, sum, weighted V per workgroup and head) live in this fixed array instead of a
// workspace from hipMalloc.  Every GPU the library runs on holds its own copy for the life of
// the process.  In host code the array's name is only a handle for hipGetSymbolAddress: the
// device address it returns, kept in every context of that device, is what kernels and copies
// are given.
constexpr size_t kNoAllocScratchBytes = 2u << 20;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

}  // namespace

namespace wgml {

// Looks up the device address of `scratch` on the context's device and keeps it in the
// context.  Called by wgml_ctx_create with that device current, so that the entry point itself
// neither switches devices nor touches the symbol table (it may run under stream capture).
int resolve_noalloc_scratch(wgml_ctx *ctx) {
    void *p = nullptr;
    WGML_CHECK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return set_error(WGML_E_HIP, "wgml_ctx_create: null address for the fixed scratch array");
    ctx->noalloc_scratch = reinterpret_cast<float *>(p);
    return WGML_OK;
}

}  // namespace wgml

namespace {

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

template <int NV4, int NW>
int launch_fast_nv(wgml_ctx *ctx, const AttnArgs &a, int km, dim3 grid) {
    const dim3 block(NW * 64);
    // the planner keeps km * NV4 within the register budget of the variant
    constexpr int kMaxKmNv = NW == 16 ? 4 : 8;
    if (km * NV4 > kMaxKmNv)
        return set_error(WGML_E_INVALID, "attention: no kernel for km %d, %d float4 per lane", km,
                         NV4);
    if constexpr (4 * NV4 <= kMaxKmNv) {
        if (km == 4) attn_fast_kernel<NV4, 4, NW><<<grid, block, 0, ctx->stream>>>(a);
    }
    if constexpr (2 * NV4 <= kMaxKmNv) {
        if (km == 2) attn_fast_kernel<NV4, 2, NW><<<grid, block, 0, ctx->stream>>>(a);
    }
    if (km == 1) attn_fast_kernel<NV4, 1, NW><<<grid, block, 0, ctx->stream>>>(a);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

template <int NW>
int launch_fast(wgml_ctx *ctx, const AttnArgs &a, int nv, int km, dim3 grid) {
    switch (nv) {
    case 1: return launch_fast_nv<1, NW>(ctx, a, km, grid);
    case 2: return launch_fast_nv<2, NW>(ctx, a, km, grid);
    default: break;
    }
    if constexpr (NW != 16) {  // large heads: only the 4-wave variant has the registers
        if (nv == 3) return launch_fast_nv<3, NW>(ctx, a, km, grid);
        return launch_fast_nv<4, NW>(ctx, a, km, grid);
    }
    return set_error(WGML_E_INVALID, "attention: no 16-wave kernel for %d float4 per lane", nv);
}

}  // namespace

namespace wgml {

// `plan_positions`: the number of positions the grid is sized for (pos+1 for a
// one-off launch, seq_len when the launch is replayed for growing positions).
struct AttnPlan {
    int nv, km;
    uint32_t groups, chunk, n_wg_y, hsp;
    int wide;  // fast plan: one 16-wave workgroup per head group, no partials
};

// The fast kernel needs float4-addressable heads; `aligned` says that q and the
// cache views start on 16-byte boundaries.
static bool fast_ok(const wgml_attn_params &p, bool aligned, bool wants_scores) {
    return !wants_scores && aligned && p.head_size % 4 == 0 && p.kv_dim % 4 == 0 &&
           p.head_size <= 256;
}

constexpr uint32_t kWidePositions = 256;  // up to here one workgroup per head group
// the most partial results per head that a consumer merges while it stages its input
// (launch_gemv_quant with GemvEpilogue::partials)
constexpr uint32_t kMaxFoldedPartials = 16;

static int make_fast_plan(wgml_ctx *ctx, const wgml_attn_params &p, uint32_t plan_positions,
                          AttnPlan &pl, bool folded = false) {
    const uint32_t hs = p.head_size;
    pl.nv = (int)((hs + 63) / 64);  // float4 per lane: 16 lanes x 4 floats x nv
    const int wide_tune = ctx->tuning[WGML_TUNE_ATTN_WIDE_POSITIONS];
    const uint32_t wide_limit = wide_tune > 0 ? (uint32_t)wide_tune : kWidePositions;
    // (a caller that merges the partial results in its own next launch gets the split grid at
    // every length: the merge launch is what made one workgroup per head the better plan)
    pl.wide = (plan_positions <= wide_limit && pl.nv <= 2 && !(folded && wide_tune <= 0)) ? 1 : 0;
    pl.km = 1;
    if (p.kv_mul == 2 || p.kv_mul == 4) pl.km = (int)p.kv_mul;
    if (p.kv_mul == 8) pl.km = 4;
    // register budget (q and acc are km * nv float4 each): 128 VGPRs for the
    // 16-wave variant, 256 for the 4-wave one
    const int max_kmnv = pl.wide ? 4 : 8;
    while (pl.km > 1 && pl.km * pl.nv > max_kmnv) pl.km >>= 1;
    pl.groups = p.n_heads / pl.km;
    pl.chunk = 0;  // derived from the position on the device
    pl.hsp = (uint32_t)pl.nv * 64;
    if (pl.wide) {
        pl.n_wg_y = 1;
        return WGML_OK;
    }
    const uint32_t cu = ctx->n_cu > 0 ? (uint32_t)ctx->n_cu : 256u;
    // about two workgroups per CU, each with at least 64 positions at full length (four
    // quads per wave; measured on 32 x 128 and 12 x 64 heads, shorter shares only add
    // partial results for the merge to read) -- or 32 positions while that keeps the partial
    // results within the 16 that the merge takes in one round of loads (512 planned positions:
    // 6.9 against 7.3 us per layer with 16 instead of 8 workgroups per head of 128, 4.95 against
    // 5.17 with heads of 64; beyond 16 the merge costs 2 us more)
    uint32_t n_wg_y = (2 * cu + pl.groups - 1) / pl.groups;
    uint32_t max_y = (plan_positions + 16 * WAVES - 1) / (16 * WAVES);
    const uint32_t short_y = std::min<uint32_t>(16u, (plan_positions + 8 * WAVES - 1) / (8 * WAVES));
    if (max_y < short_y && !folded) max_y = short_y;
    // short contexts of a folded plan: up to one workgroup per CU
    if (folded && plan_positions <= kWidePositions) {
        max_y = (cu + pl.groups - 1) / pl.groups;
        // four quads per wave: both register sets, all of them requested before the position
        // is known; and few partial results, which every workgroup of the consumer merges
        const uint32_t enough = (plan_positions + 16 * WAVES - 1) / (16 * WAVES);
        if (max_y > enough) max_y = enough;
        if (max_y > kMaxFoldedPartials) max_y = kMaxFoldedPartials;
    }
    if (n_wg_y > max_y) n_wg_y = max_y;
    if (n_wg_y > (uint32_t)MERGE_MAX_Y) n_wg_y = MERGE_MAX_Y;  // what the merge takes in one go
    if (ctx->tuning[WGML_TUNE_ATTN_SPLITS] > 0) n_wg_y = (uint32_t)ctx->tuning[WGML_TUNE_ATTN_SPLITS];
    if (n_wg_y < 2) n_wg_y = 2;
    pl.n_wg_y = n_wg_y;
    return WGML_OK;
}

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
    size_t bytes = (size_t)p.n_heads * pl.n_wg_y * (2 + pl.hsp) * 4;
    if (fast_ok(p, true, false)) {
        for (int folded = 0; folded < 2; ++folded) {
            WGML_TRY(make_fast_plan(ctx, p, plan_positions, pl, folded != 0));
            const size_t fast = (size_t)p.n_heads * pl.n_wg_y * (2 + pl.hsp) * 4;
            if (fast > bytes) bytes = fast;
        }
    }
    return ensure_ws(ctx, bytes);
}

// `ext_ws` (optional): a caller-supplied partials workspace of `ext_ws_bytes` bytes that is
// used instead of the context's own (which is grown with hipMalloc when it is too small);
// a plan that needs more than it holds is refused.
int launch_attention_planned(wgml_ctx *ctx, const wgml_attn_params &p, DynPos pos,
                             uint32_t plan_positions, uint32_t cache_rows, const float *q,
                             const float *kc, const float *vc, float *att, float *xb,
                             float *ext_ws, size_t ext_ws_bytes, AttnPartials *keep) {
    AttnPlan pl;
    if (keep) *keep = AttnPartials{};
    // A caller that merges the partial results itself gets the plan with partial results also
    // where one workgroup per head would do, as long as there are few enough of them.  Only on
    // request (WGML_TUNE_ATTN_MERGE): every workgroup of the consumer then reads all
    // partial results through the L2s, which was measured to cost more than the merge launch it
    // saves (7B shape: the 4096-wide output projection grows from 3.9 to 8.4 us with eight
    // partial results per head, 7.4 with four, against 3.0 us for the merge launch; GPT-2 124M
    // over 1024 positions 3199 against 3273 tok/s).
    const bool want_partials = keep != nullptr && att == nullptr && ctx->tuning[WGML_TUNE_ATTN_MERGE] == 1;
    if (!want_partials) keep = nullptr;
    auto workspace = [&](size_t bytes, float **ws) -> int {
        if (ext_ws) {
            if (bytes > ext_ws_bytes)
                return set_error(WGML_E_UNSUPPORTED,
                                 "attention: this shape needs %zu bytes of partial results, the "
                                 "fixed scratch array holds %zu", bytes, ext_ws_bytes);
            *ws = ext_ws;
            return WGML_OK;
        }
        WGML_TRY(ensure_ws(ctx, bytes));
        *ws = ctx->attn_ws;
        return WGML_OK;
    };
    const bool aligned = (((uintptr_t)q | (uintptr_t)kc | (uintptr_t)vc) & 15u) == 0;
    if (fast_ok(p, aligned, att != nullptr)) {
        WGML_TRY(make_fast_plan(ctx, p, plan_positions, pl, want_partials));
        if (want_partials && (pl.wide || pl.n_wg_y > kMaxFoldedPartials)) {
            // more partial results than a consumer merges: the plan with a merge launch
            keep = nullptr;
            WGML_TRY(make_fast_plan(ctx, p, plan_positions, pl, false));
        }
        AttnArgs a{};
        a.q = q;
        a.kc = kc;
        a.vc = vc;
        a.xb = xb;
        a.seq_len = p.seq_len;
        a.kv_dim = p.kv_dim;
        a.kv_mul = p.kv_mul;
        a.n_heads = p.n_heads;
        a.head_size = p.head_size;
        a.pos = pos;
        a.n_wg_y = pl.n_wg_y;
        a.spec_rows = cache_rows;
        // (all sets at short planned lengths was measured: the launch reads up to twice the
        // rows it needs and gets slower, 5.1 against 4.7 us with four workgroups per head)
        a.spec_sets = 1u;
        const dim3 grid(pl.groups, pl.n_wg_y);
        if (pl.wide) return launch_fast<16>(ctx, a, pl.nv, pl.km, grid);
        WGML_TRY(workspace((size_t)p.n_heads * pl.n_wg_y * (2 + pl.hsp) * 4, &a.ws));
        a.ws_ml = a.ws + (size_t)p.n_heads * pl.n_wg_y * pl.hsp;
        WGML_TRY(launch_fast<WAVES>(ctx, a, pl.nv, pl.km, grid));
        if (keep) {
            // the caller's next launch merges the partial results while it stages its input
            keep->o = a.ws;
            keep->ml = a.ws_ml;
            keep->n = pl.n_wg_y;
            keep->hsp = pl.hsp;
            keep->head_size = p.head_size;
            return WGML_OK;
        }
        if (pl.n_wg_y > 16)
            attn_merge_fast_kernel<64><<<dim3(p.n_heads), dim3(256), 0, ctx->stream>>>(a, pl.hsp);
        else
            attn_merge_fast_kernel<16><<<dim3(p.n_heads), dim3(256), 0, ctx->stream>>>(a, pl.hsp);
        WGML_CHECK_LAUNCH();
        ctx->launches++;
        return WGML_OK;
    }
    WGML_TRY(make_plan(ctx, p, plan_positions, pl));
    const uint32_t hs = p.head_size;
    const int nv = pl.nv, km = pl.km;
    const uint32_t groups = pl.groups, chunk = pl.chunk, n_wg_y = pl.n_wg_y;

    AttnArgs a{};
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
        WGML_TRY(workspace((size_t)p.n_heads * n_wg_y * (2 + hsp) * 4, &a.ws));
        a.ws_ml = a.ws + (size_t)p.n_heads * n_wg_y * hsp;
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

// `cache_rows`: positions the cache views hold (at least pos + 1).
int launch_attention(wgml_ctx *ctx, const wgml_attn_params &p, DynPos pos, uint32_t cache_rows,
                     const float *q, const float *kc, const float *vc, float *att, float *xb) {
    return launch_attention_planned(ctx, p, pos, pos.ptr ? p.seq_len : pos.val + 1, cache_rows, q,
                                    kc, vc, att, xb, nullptr, 0, nullptr);
}

}  // namespace wgml

extern "C" {

static int attention_entry(const char *name, wgml_ctx *ctx, const wgml_attn_params *p, wgml_view q,
                           wgml_view key_cache, wgml_view value_cache, wgml_view att, wgml_view xb,
                           float *ext_ws, size_t ext_ws_bytes, AttnPartials *keep = nullptr) {
    WGML_REQUIRE(ctx && p, "%s: null argument", name);
    WGML_TRY(check_view(q, "attention: q"));
    WGML_TRY(check_view(key_cache, "attention: key_cache"));
    WGML_TRY(check_view(value_cache, "attention: value_cache"));
    WGML_TRY(check_view(xb, "attention: xb"));
    WGML_REQUIRE(p->n_heads > 0 && p->head_size > 0 && p->kv_mul > 0 &&
                     p->n_heads % p->kv_mul == 0,
                 "%s: bad head configuration (%u heads, kv_mul %u)", name, p->n_heads, p->kv_mul);
    WGML_REQUIRE(p->kv_dim == p->n_heads / p->kv_mul * p->head_size,
                 "%s: kv_dim %u != n_kv_heads * head_size", name, p->kv_dim);
    WGML_REQUIRE(p->pos < p->seq_len, "%s: pos %u outside seq_len %u", name, p->pos, p->seq_len);
    const uint64_t dim = (uint64_t)p->n_heads * p->head_size;
    WGML_REQUIRE(q.len == dim && xb.len == dim, "%s: q/xb must have %llu elements", name,
                 (unsigned long long)dim);
    const uint64_t need = (uint64_t)(p->pos + 1) * p->kv_dim;
    WGML_REQUIRE(key_cache.len >= need && value_cache.len >= need,
                 "%s: KV cache views shorter than (pos+1)*kv_dim", name);
    float *att_ptr = nullptr;
    if (att.buf) {
        WGML_TRY(check_view(att, "attention: att"));
        WGML_REQUIRE((uint64_t)att.len >= (uint64_t)p->n_heads * p->seq_len,
                     "%s: att needs seq_len*n_heads elements", name);
        att_ptr = view_ptr(att);
    }
    DynPos pos{nullptr, p->pos};
    const uint64_t rows = (key_cache.len < value_cache.len ? key_cache.len : value_cache.len) /
                          p->kv_dim;
    return launch_attention_planned(ctx, *p, pos, p->pos + 1,
                                    (uint32_t)(rows < p->seq_len ? rows : p->seq_len), view_ptr(q),
                                    view_ptr(key_cache), view_ptr(value_cache), att_ptr,
                                    view_ptr(xb), ext_ws, ext_ws_bytes, keep);
}

int wgml_attention(wgml_ctx *ctx, const wgml_attn_params *p, wgml_view q, wgml_view key_cache,
                   wgml_view value_cache, wgml_view att, wgml_view xb) {
    return attention_entry("wgml_attention", ctx, p, q, key_cache, value_cache, att, xb, nullptr, 0);
}

int wgml_attention_gemv_quant(wgml_ctx *ctx, const wgml_attn_params *p, wgml_view q,
                              wgml_view key_cache, wgml_view value_cache, wgml_view xb,
                              const wgml_qmat *m, wgml_view out, int accumulate) {
    WGML_REQUIRE(ctx && p && m, "wgml_attention_gemv_quant: null argument");
    WGML_TRY(check_view(out, "wgml_attention_gemv_quant: out"));
    WGML_REQUIRE((uint64_t)m->ncols == (uint64_t)p->n_heads * p->head_size && out.len == m->nrows,
                 "wgml_attention_gemv_quant: the matrix is %ux%u, attention gives %llu values and "
                 "out holds %u", m->nrows, m->ncols, (unsigned long long)p->n_heads * p->head_size,
                 out.len);
    const wgml_view no_att{nullptr, 0, 0};
    AttnPartials parts;
    WGML_TRY(attention_entry("wgml_attention_gemv_quant", ctx, p, q, key_cache, value_cache, no_att,
                             xb, nullptr, 0, gemv_partials_supported(ctx, m) ? &parts : nullptr));
    GemvEpilogue e;
    e.accumulate = accumulate ? 1 : 0;
    e.partials = parts;
    return launch_gemv_quant(ctx, view_ptr(out), m, view_ptr(xb), e);
}

// The same launches as wgml_attention with no `att` output, partial results in the library's
// fixed scratch array: no hipMalloc / hipFree, no memset (every partial a merge reads is
// written by the launch before it).  Calls that overlap on one GPU share the array and race.
int wgml_attention_noalloc(wgml_ctx *ctx, const wgml_attn_params *p, wgml_view q,
                           wgml_view key_cache, wgml_view value_cache, wgml_view xb) {
    WGML_REQUIRE(ctx != nullptr, "wgml_attention_noalloc: null context");
    float *ws = ctx->noalloc_scratch;  // resolved when the context was created
    WGML_REQUIRE(ws != nullptr, "wgml_attention_noalloc: the context holds no scratch address");
    const wgml_view no_att{nullptr, 0, 0};
    return attention_entry("wgml_attention_noalloc", ctx, p, q, key_cache, value_cache, no_att, xb,
                           ws, kNoAllocScratchBytes);
}

}  // extern "C"
