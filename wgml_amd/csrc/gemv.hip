// Dequantize-and-GEMV kernels for Q8_0 / Q4_K / Q6_K and the dense f32 GEMV.
// Replaces GemvQuant::dispatch and its WGSL kernels (ops/gemv_quant.rs:243-348,
// ops/gemv_quant_{q8_0x2,q4_k,q6_kx2}.wgsl of the reference) and wgebra's f32
// Gemv/GemvTr.
//
// Scheme (wavefront-64, HBM-bound, no MFMA):
//   * the activation vector x is staged once per workgroup into LDS in a
//     lane-transposed order, so that lane L of a wave reads its k-th float4 at
//     LDS slot [k][L]: consecutive lanes hit consecutive 16-byte slots (no bank
//     conflicts);
//   * a wave owns R consecutive rows.  Per 64-tile step every lane loads one
//     tile of x from LDS into registers and reuses it for the R rows, so LDS
//     traffic is 1/R of the naive rate;
//   * weights stream from HBM as aligned 128-bit loads; a wave touches one
//     contiguous run of bytes per row and plane;
//   * sub-block minima / offsets are folded in through per-tile sums of x that
//     are computed once per workgroup (not once per row);
//   * the 64 partial sums of a row are reduced with DPP + v_readlane in a fixed
//     order (deterministic results).
//
// A "tile" is the span one lane covers per step:
//   Q4_K: one 64-element group of a super-block (32 bytes of qs) + the 16-byte
//         header {d, dmin, scales[12]};
//   Q6_K: 64 elements {e, e+32, e+64, e+96 : e in 16-run} of one 128-half: 16
//         bytes of ql, 16 of ql+32, 16 of qh, 8 scale bytes, d;
//   Q8_0: one 32-element block: 32 bytes of qs + d.
#include "common.h"
#include "device_utils.h"

using namespace wgml;

namespace {

struct GemvParams {
    const uint8_t *p0, *p1, *p2, *p3;  // matrix planes
    const float *x;
    float *out;
    const float *bias;
    uint32_t nrows, ncols;
    int accumulate;
};

// ------------------------------------------------------------------ Q4_K ----
struct FmtQ4K {
    static constexpr int TILE = 64;    // elements per lane tile
    static constexpr int CHUNKS = 16;  // float4 of x per tile
    static constexpr int NSUM = 2;     // x sums per tile (low-nibble half, high-nibble half)
    struct Row {
        uint4 hdr, qa, qb;
    };
    struct RowBase {
        const uint8_t *blocks;
    };
    __device__ static RowBase row_base(const GemvParams &p, uint32_t row) {
        return {p.p0 + (size_t)row * (p.ncols / 256) * 144};
    }
    // float4 index g of x -> (tile, chunk)
    __device__ static void map(uint32_t g, uint32_t &tile, uint32_t &chunk) {
        tile = g >> 4;
        chunk = g & 15;
    }
    // which sum a chunk contributes to
    __device__ static uint32_t sum_of_chunk(uint32_t chunk) { return chunk >> 3; }
    __device__ static void load(Row &w, const RowBase &rb, uint32_t tile) {
        const uint8_t *blk = rb.blocks + (size_t)(tile >> 2) * 144;
        w.hdr = *reinterpret_cast<const uint4 *>(blk);
        const uint4 *q = reinterpret_cast<const uint4 *>(blk + 16 + (tile & 3) * 32);
        w.qa = q[0];
        w.qb = q[1];
    }
    __device__ static float dot(const Row &w, const float4 (&x)[CHUNKS], const float (&s)[NSUM],
                                uint32_t tile) {
        const uint32_t j = tile & 3;
        const float d = f16_bits_to_f32((uint16_t)(w.hdr.x & 0xffffu));
        const float dmin = f16_bits_to_f32((uint16_t)(w.hdr.x >> 16));
        // 6-bit scale/min pairs of sub-blocks 2j and 2j+1 (get_scale_min_k4).
        const uint32_t sh = (j & 1u) * 16u;
        const uint32_t a = (w.hdr.y >> sh) & 0xffffu, b = (w.hdr.z >> sh) & 0xffffu,
                       c = (w.hdr.w >> sh) & 0xffffu;
        uint32_t sc2, m2;
        if (j < 2) {
            sc2 = a & 0x3f3fu;
            m2 = b & 0x3f3fu;
        } else {
            sc2 = (c & 0x0f0fu) | ((a >> 2) & 0x3030u);
            m2 = ((c >> 4) & 0x0f0fu) | ((b >> 2) & 0x3030u);
        }
        const float sc_lo = ub0(sc2), sc_hi = ub1(sc2), m_lo = ub0(m2), m_hi = ub1(m2);
        const uint32_t q[8] = {w.qa.x, w.qa.y, w.qa.z, w.qa.w, w.qb.x, w.qb.y, w.qb.z, w.qb.w};
        float dlo = 0.f, dhi = 0.f;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint32_t lo = q[k] & 0x0f0f0f0fu;
            const uint32_t hi = q[k] & 0xf0f0f0f0u;  // 16 * nibble per byte
            const float4 xl = x[k], xh = x[8 + k];
            dlo = fmaf(ub0(lo), xl.x, dlo);
            dlo = fmaf(ub1(lo), xl.y, dlo);
            dlo = fmaf(ub2(lo), xl.z, dlo);
            dlo = fmaf(ub3(lo), xl.w, dlo);
            dhi = fmaf(ub0(hi), xh.x, dhi);
            dhi = fmaf(ub1(hi), xh.y, dhi);
            dhi = fmaf(ub2(hi), xh.z, dhi);
            dhi = fmaf(ub3(hi), xh.w, dhi);
        }
        float r = (d * sc_lo) * dlo;
        r = fmaf((d * sc_hi) * 0.0625f, dhi, r);
        r = fmaf(-dmin, fmaf(m_lo, s[0], m_hi * s[1]), r);
        return r;
    }
};

// ------------------------------------------------------------------ Q6_K ----
struct FmtQ6K {
    static constexpr int TILE = 64;
    static constexpr int CHUNKS = 16;
    static constexpr int NSUM = 4;  // one per 16-element sub-block
    struct Row {
        uint4 l0, l1, h;
        uint2 sc;
        uint16_t d;
    };
    struct RowBase {
        const uint8_t *ql, *qh, *sc, *d;
    };
    __device__ static RowBase row_base(const GemvParams &p, uint32_t row) {
        const size_t nb = (size_t)row * (p.ncols / 256);
        return {p.p0 + nb * 128, p.p1 + nb * 64, p.p2 + nb * 16, p.p3 + nb * 2};
    }
    __device__ static void map(uint32_t g, uint32_t &tile, uint32_t &chunk) {
        const uint32_t e = g * 4;
        const uint32_t blk = e >> 8, i = (e >> 7) & 1, quarter = (e >> 5) & 3, s = (e >> 4) & 1,
                       k4 = (e & 15) >> 2;
        tile = blk * 4 + i * 2 + s;
        chunk = quarter * 4 + k4;
    }
    __device__ static uint32_t sum_of_chunk(uint32_t chunk) { return chunk >> 2; }
    __device__ static void load(Row &w, const RowBase &rb, uint32_t tile) {
        const size_t blk = tile >> 2;
        const uint32_t i = (tile >> 1) & 1, s = tile & 1;
        const uint8_t *ql = rb.ql + blk * 128 + i * 64 + s * 16;
        w.l0 = *reinterpret_cast<const uint4 *>(ql);
        w.l1 = *reinterpret_cast<const uint4 *>(ql + 32);
        w.h = *reinterpret_cast<const uint4 *>(rb.qh + blk * 64 + i * 32 + s * 16);
        w.sc = *reinterpret_cast<const uint2 *>(rb.sc + blk * 16 + i * 8);
        w.d = *reinterpret_cast<const uint16_t *>(rb.d + blk * 2);
    }
    __device__ static float dot(const Row &w, const float4 (&x)[CHUNKS], const float (&s)[NSUM],
                                uint32_t tile) {
        const uint32_t sb = (tile & 1u) * 8u;  // bit offset of scales[is], is = tile & 1
        const float sc1 = sb0(w.sc.x >> sb), sc2 = sb0(w.sc.x >> (sb + 16)),
                    sc3 = sb0(w.sc.y >> sb), sc4 = sb0(w.sc.y >> (sb + 16));
        const uint32_t l0[4] = {w.l0.x, w.l0.y, w.l0.z, w.l0.w};
        const uint32_t l1[4] = {w.l1.x, w.l1.y, w.l1.z, w.l1.w};
        const uint32_t hh[4] = {w.h.x, w.h.y, w.h.z, w.h.w};
        float d1 = 0.f, d2 = 0.f, d3 = 0.f, d4 = 0.f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t H = hh[k];
            const uint32_t q1 = (l0[k] & 0x0f0f0f0fu) | ((H << 4) & 0x30303030u);
            const uint32_t q2 = (l1[k] & 0x0f0f0f0fu) | ((H << 2) & 0x30303030u);
            const uint32_t q3 = ((l0[k] >> 4) & 0x0f0f0f0fu) | (H & 0x30303030u);
            const uint32_t q4 = ((l1[k] >> 4) & 0x0f0f0f0fu) | ((H >> 2) & 0x30303030u);
            const float4 x1 = x[k], x2 = x[4 + k], x3 = x[8 + k], x4 = x[12 + k];
            d1 = fmaf(ub0(q1), x1.x, d1);
            d1 = fmaf(ub1(q1), x1.y, d1);
            d1 = fmaf(ub2(q1), x1.z, d1);
            d1 = fmaf(ub3(q1), x1.w, d1);
            d2 = fmaf(ub0(q2), x2.x, d2);
            d2 = fmaf(ub1(q2), x2.y, d2);
            d2 = fmaf(ub2(q2), x2.z, d2);
            d2 = fmaf(ub3(q2), x2.w, d2);
            d3 = fmaf(ub0(q3), x3.x, d3);
            d3 = fmaf(ub1(q3), x3.y, d3);
            d3 = fmaf(ub2(q3), x3.z, d3);
            d3 = fmaf(ub3(q3), x3.w, d3);
            d4 = fmaf(ub0(q4), x4.x, d4);
            d4 = fmaf(ub1(q4), x4.y, d4);
            d4 = fmaf(ub2(q4), x4.z, d4);
            d4 = fmaf(ub3(q4), x4.w, d4);
        }
        // q - 32 folded in through the sub-block sums of x.
        float r = sc1 * fmaf(-32.f, s[0], d1);
        r = fmaf(sc2, fmaf(-32.f, s[1], d2), r);
        r = fmaf(sc3, fmaf(-32.f, s[2], d3), r);
        r = fmaf(sc4, fmaf(-32.f, s[3], d4), r);
        return f16_bits_to_f32(w.d) * r;
    }
};

// ------------------------------------------------------------------ Q8_0 ----
struct FmtQ8_0 {
    static constexpr int TILE = 32;
    static constexpr int CHUNKS = 8;
    static constexpr int NSUM = 0;
    struct Row {
        uint4 a, b;
        uint16_t d;
    };
    struct RowBase {
        const uint8_t *qs, *d;
    };
    __device__ static RowBase row_base(const GemvParams &p, uint32_t row) {
        return {p.p0 + (size_t)row * p.ncols, p.p1 + (size_t)row * (p.ncols / 32) * 2};
    }
    __device__ static void map(uint32_t g, uint32_t &tile, uint32_t &chunk) {
        tile = g >> 3;
        chunk = g & 7;
    }
    __device__ static uint32_t sum_of_chunk(uint32_t) { return 0; }
    __device__ static void load(Row &w, const RowBase &rb, uint32_t tile) {
        const uint4 *q = reinterpret_cast<const uint4 *>(rb.qs + (size_t)tile * 32);
        w.a = q[0];
        w.b = q[1];
        w.d = *reinterpret_cast<const uint16_t *>(rb.d + (size_t)tile * 2);
    }
    __device__ static float dot(const Row &w, const float4 (&x)[CHUNKS], const float (&)[1],
                                uint32_t) {
        const uint32_t q[8] = {w.a.x, w.a.y, w.a.z, w.a.w, w.b.x, w.b.y, w.b.z, w.b.w};
        float acc = 0.f;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float4 xv = x[k];
            acc = fmaf(sb0(q[k]), xv.x, acc);
            acc = fmaf(sb1(q[k]), xv.y, acc);
            acc = fmaf(sb2(q[k]), xv.z, acc);
            acc = fmaf(sb3(q[k]), xv.w, acc);
        }
        return f16_bits_to_f32(w.d) * acc;
    }
};

// LDS layout: x as float4 xs[step][chunk][lane]; then sums[sum][tile_padded].
template <class F>
__device__ __forceinline__ uint32_t lds_slot(uint32_t tile, uint32_t chunk) {
    return ((tile >> 6) * F::CHUNKS + chunk) * 64 + (tile & 63);
}

template <class F, int R>
__global__ __launch_bounds__(256) void gemv_quant_kernel(const GemvParams p) {
    extern __shared__ float4 smem[];
    constexpr int NS = F::NSUM > 0 ? F::NSUM : 1;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t nwaves = blockDim.x >> 6;
    const uint32_t ntiles = p.ncols / F::TILE;
    const uint32_t nsteps = (ntiles + 63) >> 6;
    const uint32_t ntiles_pad = nsteps << 6;
    float *sums = reinterpret_cast<float *>(smem + (size_t)ntiles_pad * F::CHUNKS);

    const uint32_t row0 = (blockIdx.x * nwaves + wave) * R;

    // First step's weights are requested before x is staged: they do not depend on it.
    typename F::RowBase rb[R];
    typename F::Row w[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint32_t row = min(row0 + r, p.nrows - 1);
        rb[r] = F::row_base(p, row);
    }
    if (lane < ntiles) {
#pragma unroll
        for (int r = 0; r < R; ++r) F::load(w[r], rb[r], lane);
    }

    // Stage x.
    const float4 *x4 = reinterpret_cast<const float4 *>(p.x);
    const uint32_t n4 = p.ncols >> 2;
    for (uint32_t g = tid; g < n4; g += blockDim.x) {
        uint32_t tile, chunk;
        F::map(g, tile, chunk);
        smem[lds_slot<F>(tile, chunk)] = x4[g];
    }
    __syncthreads();
    if (F::NSUM > 0) {
        constexpr int CPS = F::CHUNKS / NS;  // chunks per sum
        for (uint32_t t = tid; t < ntiles * NS; t += blockDim.x) {
            const uint32_t tile = t % ntiles, si = t / ntiles;
            float acc = 0.f;
#pragma unroll
            for (int c = 0; c < CPS; ++c) {
                const float4 v = smem[lds_slot<F>(tile, si * CPS + c)];
                acc += (v.x + v.y) + (v.z + v.w);
            }
            sums[si * ntiles_pad + tile] = acc;
        }
        __syncthreads();
    }

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;

    for (uint32_t step = 0; step < nsteps; ++step) {
        const uint32_t tile = step * 64 + lane;
        const bool active = tile < ntiles;
        // Prefetch the next step's weights while this step is computed.
        typename F::Row wn[R];
        const uint32_t tile_n = tile + 64;
        const bool active_n = (step + 1 < nsteps) && tile_n < ntiles;
        if (active_n) {
#pragma unroll
            for (int r = 0; r < R; ++r) F::load(wn[r], rb[r], tile_n);
        }
        if (active) {
            float4 xr[F::CHUNKS];
#pragma unroll
            for (int c = 0; c < F::CHUNKS; ++c) xr[c] = smem[(step * F::CHUNKS + c) * 64 + lane];
            float s[NS];
#pragma unroll
            for (int k = 0; k < NS; ++k) s[k] = F::NSUM > 0 ? sums[k * ntiles_pad + tile] : 0.f;
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] += F::dot(w[r], xr, s, tile);
        }
        if (active_n) {
#pragma unroll
            for (int r = 0; r < R; ++r) w[r] = wn[r];
        }
    }

#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float total = wave_sum(acc[r]);
        const uint32_t row = row0 + r;
        if (lane == 0 && row < p.nrows) {
            float v = total;
            if (p.bias) v += p.bias[row];
            if (p.accumulate) v += p.out[row];
            p.out[row] = v;
        }
    }
}

// ------------------------------------------------------------- dense f32 ----
// out = A v, A row-major.  One wave per row, float4 loads, x from LDS.
__global__ __launch_bounds__(256) void gemv_f32_kernel(const float *__restrict__ a,
                                                       const float *__restrict__ x,
                                                       float *__restrict__ out,
                                                       const float *__restrict__ bias,
                                                       uint32_t nrows, uint32_t ncols,
                                                       int accumulate, int vec4) {
    extern __shared__ float4 smem[];
    float *xs = reinterpret_cast<float *>(smem);
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    for (uint32_t i = tid; i < ncols; i += blockDim.x) xs[i] = x[i];
    __syncthreads();
    const uint32_t row = blockIdx.x * nwaves + wave;
    if (row >= nrows) return;
    const float *ar = a + (size_t)row * ncols;
    float acc = 0.f;
    if (vec4) {
        const float4 *a4 = reinterpret_cast<const float4 *>(ar);
        const uint32_t n4 = ncols >> 2;
        for (uint32_t g = lane; g < n4; g += 64) {
            const float4 av = a4[g];
            const float4 xv = smem[g];
            acc = fmaf(av.x, xv.x, acc);
            acc = fmaf(av.y, xv.y, acc);
            acc = fmaf(av.z, xv.z, acc);
            acc = fmaf(av.w, xv.w, acc);
        }
    } else {
        for (uint32_t j = lane; j < ncols; j += 64) acc = fmaf(ar[j], xs[j], acc);
    }
    const float total = wave_sum(acc);
    if (lane == 0) {
        float v = total;
        if (bias) v += bias[row];
        if (accumulate) v += out[row];
        out[row] = v;
    }
}

// out = A^T v: thread per output column, coalesced across columns.
__global__ __launch_bounds__(256) void gemv_tr_f32_kernel(const float *__restrict__ a,
                                                          const float *__restrict__ v,
                                                          float *__restrict__ out, uint32_t nrows,
                                                          uint32_t ncols) {
    const uint32_t j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= ncols) return;
    float acc = 0.f;
    for (uint32_t i = 0; i < nrows; ++i) acc = fmaf(a[(size_t)i * ncols + j], v[i], acc);
    out[j] = acc;
}

int g_force_r = 0;  // 0 = heuristic
constexpr size_t kMaxLds = 128 * 1024;

template <class F>
int launch_fmt(wgml_ctx *ctx, const GemvParams &p) {
    constexpr int NS = F::NSUM;
    const uint32_t ntiles = p.ncols / F::TILE;
    const uint32_t ntiles_pad = ((ntiles + 63) / 64) * 64;
    const size_t lds = (size_t)ntiles_pad * F::CHUNKS * 16 + (size_t)ntiles_pad * NS * 4;
    if (lds > kMaxLds)
        return set_error(WGML_E_UNSUPPORTED,
                         "gemv_quant: %u columns need %zu bytes of LDS (limit %zu)", p.ncols, lds,
                         kMaxLds);
    if (lds > 64 * 1024) {
        // gfx950 has 160 KB of LDS per CU; above 64 KB a kernel must opt in once.
        static bool opted_in = false;
        if (!opted_in) {
            WGML_CHECK_HIP(hipFuncSetAttribute((const void *)gemv_quant_kernel<F, 1>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize,
                                               (int)kMaxLds));
            WGML_CHECK_HIP(hipFuncSetAttribute((const void *)gemv_quant_kernel<F, 2>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize,
                                               (int)kMaxLds));
            WGML_CHECK_HIP(hipFuncSetAttribute((const void *)gemv_quant_kernel<F, 4>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize,
                                               (int)kMaxLds));
            opted_in = true;
        }
    }
    const int waves = 4;
    // Rows per wave: more rows amortise the LDS reads of x, fewer rows give more
    // waves to hide HBM latency when the matrix has few rows.
    int R = g_force_r;
    if (!R) {
        const uint32_t cu = ctx->n_cu > 0 ? (uint32_t)ctx->n_cu : 256u;
        if (p.nrows >= cu * 8 * 4) R = 4;
        else if (p.nrows >= cu * 8 * 2) R = 2;
        else R = 1;
    }
    const uint32_t rows_per_wg = waves * R;
    const dim3 grid((p.nrows + rows_per_wg - 1) / rows_per_wg), block(waves * 64);
    switch (R) {
    case 4: gemv_quant_kernel<F, 4><<<grid, block, lds, ctx->stream>>>(p); break;
    case 2: gemv_quant_kernel<F, 2><<<grid, block, lds, ctx->stream>>>(p); break;
    default: gemv_quant_kernel<F, 1><<<grid, block, lds, ctx->stream>>>(p); break;
    }
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

}  // namespace

namespace wgml {

int launch_gemv_f32(wgml_ctx *ctx, float *out, const float *a, uint32_t nrows, uint32_t ncols,
                    int transposed, const float *v) {
    if (transposed) {
        gemv_tr_f32_kernel<<<dim3((ncols + 255) / 256), dim3(256), 0, ctx->stream>>>(a, v, out,
                                                                                     nrows, ncols);
    } else {
        const size_t lds = (((size_t)ncols + 3) / 4) * 16;
        if (lds > 64 * 1024)
            return set_error(WGML_E_UNSUPPORTED, "gemv_f32: %u columns exceed the LDS limit", ncols);
        const int vec4 = (ncols % 4 == 0) && ((uintptr_t)a % 16 == 0);
        gemv_f32_kernel<<<dim3((nrows + 3) / 4), dim3(256), lds, ctx->stream>>>(
            a, v, out, nullptr, nrows, ncols, 0, vec4);
    }
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int launch_gemv_quant(wgml_ctx *ctx, float *out, const wgml_qmat *m, const float *v,
                      const GemvEpilogue &ep) {
    if ((uintptr_t)v % 16 != 0)
        return set_error(WGML_E_INVALID, "gemv_quant: the input vector must be 16-byte aligned");
    if (m->type == WGML_F32) {
        const size_t lds = (size_t)m->ncols * 4;
        if (lds > 64 * 1024)
            return set_error(WGML_E_UNSUPPORTED, "gemv_f32: %u columns exceed the LDS limit",
                             m->ncols);
        gemv_f32_kernel<<<dim3((m->nrows + 3) / 4), dim3(256), lds, ctx->stream>>>(
            (const float *)m->p0, v, out, ep.bias, m->nrows, m->ncols, ep.accumulate, 1);
        WGML_CHECK_LAUNCH();
        ctx->launches++;
        return WGML_OK;
    }
    GemvParams p;
    p.p0 = m->p0;
    p.p1 = m->p1;
    p.p2 = m->p2;
    p.p3 = m->p3;
    p.x = v;
    p.out = out;
    p.bias = ep.bias;
    p.nrows = m->nrows;
    p.ncols = m->ncols;
    p.accumulate = ep.accumulate;
    switch (m->type) {
    case WGML_Q4_K: return launch_fmt<FmtQ4K>(ctx, p);
    case WGML_Q6_K: return launch_fmt<FmtQ6K>(ctx, p);
    case WGML_Q8_0: return launch_fmt<FmtQ8_0>(ctx, p);
    default: return set_error(WGML_E_UNSUPPORTED, "gemv_quant: unsupported type %d", m->type);
    }
}

}  // namespace wgml

extern "C" {

// Debug knob for kernel sweeps: rows per wave of the quantized GEMV (0 = heuristic).
WGML_API int wgml_debug_set_gemv_rows_per_wave(int r) {
    WGML_REQUIRE(r == 0 || r == 1 || r == 2 || r == 4,
                 "wgml_debug_set_gemv_rows_per_wave: %d not in {0,1,2,4}", r);
    g_force_r = r;
    return WGML_OK;
}

int wgml_gemv_quant(wgml_ctx *ctx, wgml_view out, const wgml_qmat *m, wgml_view v) {
    WGML_REQUIRE(ctx && m, "wgml_gemv_quant: null argument");
    WGML_TRY(check_view(out, "wgml_gemv_quant: out"));
    WGML_TRY(check_view(v, "wgml_gemv_quant: v"));
    WGML_REQUIRE(v.len == m->ncols, "Gemv: dimension mismatch (v has %u, matrix has %u columns)",
                 v.len, m->ncols);
    WGML_REQUIRE(out.len == m->nrows, "Gemv: dimension mismatch (out has %u, matrix has %u rows)",
                 out.len, m->nrows);
    return launch_gemv_quant(ctx, view_ptr(out), m, view_ptr(v), GemvEpilogue{});
}

int wgml_gemv_f32(wgml_ctx *ctx, wgml_view out, wgml_view a, uint32_t nrows, uint32_t ncols,
                  int transposed, wgml_view v) {
    WGML_REQUIRE(ctx != nullptr, "wgml_gemv_f32: null context");
    WGML_TRY(check_view(out, "wgml_gemv_f32: out"));
    WGML_TRY(check_view(a, "wgml_gemv_f32: a"));
    WGML_TRY(check_view(v, "wgml_gemv_f32: v"));
    WGML_REQUIRE((uint64_t)a.len == (uint64_t)nrows * ncols,
                 "wgml_gemv_f32: matrix view has %u elements, expected %llu", a.len,
                 (unsigned long long)nrows * ncols);
    if (transposed) {
        WGML_REQUIRE(v.len == nrows && out.len == ncols, "GemvTr: dimension mismatch");
    } else {
        WGML_REQUIRE(v.len == ncols && out.len == nrows, "Gemv: dimension mismatch");
    }
    return launch_gemv_f32(ctx, view_ptr(out), view_ptr(a), nrows, ncols, transposed, view_ptr(v));
}

}  // extern "C"
