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
#include <type_traits>

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
    const uint32_t *dyn_pos;  // out += *dyn_pos * out_pos_stride
    uint32_t out_pos_stride;
    const float *norm_w;  // optional fused RMSNorm of x
    float norm_eps;
    const float *ln_g, *ln_b;  // optional fused LayerNorm of x (integer-dot kernels)
    int act;                   // 1: GELU on acc + bias before the store
    // integer-dot kernels: the first `active_waves` waves of every workgroup walk
    // the row-groups with stride gridDim.x * active_waves
    uint32_t active_waves;
    // part_n > 0: x is the merged output of a decode-attention launch that left part_n partial
    // results per head (AttnPartials in common.h); x itself is then not read
    const float *part_o, *part_ml;
    uint32_t part_n, part_hsp, part_hs, part_hs_inv;  // part_hs_inv = ceil(2^32 / part_hs)
};

// Merging attention partial results (see AttnPartials) for float4 number g4 of the merged
// output: the partial results of its head are taken in eight at a time, the way an online
// softmax takes in new scores.  PartialChunk holds one round of loads, so that a caller can
// request it early and merge it later.
struct PartialChunk {
    float2 s[8];  // (maximum, sum of weights)
    float4 v[8];  // weighted sums of V
};
__device__ __forceinline__ void load_partials(PartialChunk &c, const GemvParams &p, uint32_t g4,
                                              uint32_t y0) {
    // h = e / head_size by multiplication with ceil(2^32 / head_size): exact for the e < 2^20
    // and head sizes up to 256 that occur here
    const uint32_t e = g4 * 4, h = __umulhi(e, p.part_hs_inv), d = e - h * p.part_hs, P = p.part_n;
    const float *o = p.part_o + (size_t)h * P * p.part_hsp + d;
    const float2 *ml = reinterpret_cast<const float2 *>(p.part_ml) + (size_t)h * P;
    // The loads are unconditional (a partial result beyond the last one re-reads the last one
    // and is masked out when it is merged): with a load under a condition the compiler cannot
    // count the loads in flight, and the wait for these would also wait for the weight tiles
    // requested after them.
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const uint32_t y = min(y0 + (uint32_t)k, P - 1);
        c.s[k] = ml[y];
        c.v[k] = *reinterpret_cast<const float4 *>(o + (size_t)y * p.part_hsp);
    }
}
struct PartialState {
    float M = -INFINITY, L = 0.f;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
};
// `n`: how many of the chunk's eight partial results exist.
__device__ __forceinline__ void merge_partials(PartialState &st, const PartialChunk &c, uint32_t n) {
    float Mc = st.M;
#pragma unroll
    for (int k = 0; k < 8; ++k) Mc = fmaxf(Mc, (uint32_t)k < n ? c.s[k].x : -INFINITY);
    // the running state is rescaled to the new maximum (M = -inf only while nothing has been
    // taken in, and then L and acc are zero)
    const float r = st.M == -INFINITY ? 0.f : __expf(st.M - Mc);
    st.L *= r;
    st.acc.x *= r;
    st.acc.y *= r;
    st.acc.z *= r;
    st.acc.w *= r;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        // a neutral partial (maximum -inf) has undefined values: they must not be touched
        const bool live = (uint32_t)k < n && c.s[k].x != -INFINITY;
        const float wk = live ? __expf(c.s[k].x - Mc) : 0.f;
        st.L = fmaf(c.s[k].y, wk, st.L);
        st.acc.x = fmaf(live ? c.v[k].x : 0.f, wk, st.acc.x);
        st.acc.y = fmaf(live ? c.v[k].y : 0.f, wk, st.acc.y);
        st.acc.z = fmaf(live ? c.v[k].z : 0.f, wk, st.acc.z);
        st.acc.w = fmaf(live ? c.v[k].w : 0.f, wk, st.acc.w);
    }
    st.M = Mc;
}
// `first`: the partial results 0..7, already requested; the others are fetched here.
__device__ __forceinline__ float4 merged_partials(const GemvParams &p, uint32_t g4,
                                                  const PartialChunk &first) {
    PartialState st;
    merge_partials(st, first, p.part_n);
    for (uint32_t y0 = 8; y0 < p.part_n; y0 += 8) {
        PartialChunk c;
        load_partials(c, p, g4, y0);
        merge_partials(st, c, p.part_n - y0);
    }
    return make_float4(st.acc.x / st.L, st.acc.y / st.L, st.acc.z / st.L, st.acc.w / st.L);
}
__device__ __forceinline__ float4 merged_partials(const GemvParams &p, uint32_t g4) {
    PartialChunk c;
    load_partials(c, p, g4, 0);
    return merged_partials(p, g4, c);
}

// Hides a value from the optimizer (no instruction is emitted).  Used on masked
// 32-bit words so that the four bytes are converted with v_cvt_f32_ubyte0..3 of
// the *shared* masked word instead of one bit-field extract per element.
__device__ __forceinline__ uint32_t opaque(uint32_t v) {
    asm("" : "+v"(v));
    return v;
}

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
    __device__ static void load(Row &w, const RowBase &rb, uint32_t tile) {
        const uint8_t *blk = rb.blocks + (size_t)(tile >> 2) * 144;
        w.hdr = *reinterpret_cast<const uint4 *>(blk);
        const uint4 *q = reinterpret_cast<const uint4 *>(blk + 16 + (tile & 3) * 32);
        w.qa = q[0];
        w.qb = q[1];
    }
    // acc[r] += dot(row r tile, x tile).  xl points at this lane's slot of chunk 0
    // (chunk c is xl[c * 64]); s = the two half-tile sums of x.
    template <int R>
    __device__ static void accumulate(const Row (&w)[R], const float4 *xl, const float *s,
                                      uint32_t tile, float (&acc)[R]) {
        const uint32_t j = tile & 3;
        const uint32_t sh = (j & 1u) * 16u;
        float dlo[R], dhi[R];
#pragma unroll
        for (int r = 0; r < R; ++r) dlo[r] = dhi[r] = 0.f;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float4 xa = xl[k * 64], xb = xl[(8 + k) * 64];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t q = k < 4 ? (&w[r].qa.x)[k] : (&w[r].qb.x)[k - 4];
                const uint32_t lo = opaque(q & 0x0f0f0f0fu);
                const uint32_t hi = opaque(q & 0xf0f0f0f0u);  // 16 * nibble per byte
                dlo[r] = fmaf(ub0(lo), xa.x, dlo[r]);
                dlo[r] = fmaf(ub1(lo), xa.y, dlo[r]);
                dlo[r] = fmaf(ub2(lo), xa.z, dlo[r]);
                dlo[r] = fmaf(ub3(lo), xa.w, dlo[r]);
                dhi[r] = fmaf(ub0(hi), xb.x, dhi[r]);
                dhi[r] = fmaf(ub1(hi), xb.y, dhi[r]);
                dhi[r] = fmaf(ub2(hi), xb.z, dhi[r]);
                dhi[r] = fmaf(ub3(hi), xb.w, dhi[r]);
            }
        }
        const float s0 = s[0], s1 = s[1];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float d = f16_bits_to_f32((uint16_t)(w[r].hdr.x & 0xffffu));
            const float dmin = f16_bits_to_f32((uint16_t)(w[r].hdr.x >> 16));
            // 6-bit scale/min pairs of sub-blocks 2j and 2j+1 (get_scale_min_k4).
            const uint32_t a = (w[r].hdr.y >> sh) & 0xffffu, b = (w[r].hdr.z >> sh) & 0xffffu,
                           c = (w[r].hdr.w >> sh) & 0xffffu;
            uint32_t sc2, m2;
            if (j < 2) {
                sc2 = a & 0x3f3fu;
                m2 = b & 0x3f3fu;
            } else {
                sc2 = (c & 0x0f0fu) | ((a >> 2) & 0x3030u);
                m2 = ((c >> 4) & 0x0f0fu) | ((b >> 2) & 0x3030u);
            }
            const float sc_lo = ub0(sc2), sc_hi = ub1(sc2), m_lo = ub0(m2), m_hi = ub1(m2);
            float v = (d * sc_lo) * dlo[r];
            v = fmaf((d * sc_hi) * 0.0625f, dhi[r], v);
            v = fmaf(-dmin, fmaf(m_lo, s0, m_hi * s1), v);
            acc[r] += v;
        }
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
    template <int R>
    __device__ static void accumulate(const Row (&w)[R], const float4 *xl, const float *s,
                                      uint32_t tile, float (&acc)[R]) {
        float d1[R], d2[R], d3[R], d4[R];
#pragma unroll
        for (int r = 0; r < R; ++r) d1[r] = d2[r] = d3[r] = d4[r] = 0.f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float4 x1 = xl[k * 64], x2 = xl[(4 + k) * 64], x3 = xl[(8 + k) * 64],
                         x4 = xl[(12 + k) * 64];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t L0 = (&w[r].l0.x)[k], L1 = (&w[r].l1.x)[k], H = (&w[r].h.x)[k];
                const uint32_t q1 = opaque((L0 & 0x0f0f0f0fu) | ((H << 4) & 0x30303030u));
                const uint32_t q2 = opaque((L1 & 0x0f0f0f0fu) | ((H << 2) & 0x30303030u));
                const uint32_t q3 = opaque(((L0 >> 4) & 0x0f0f0f0fu) | (H & 0x30303030u));
                const uint32_t q4 = opaque(((L1 >> 4) & 0x0f0f0f0fu) | ((H >> 2) & 0x30303030u));
                d1[r] = fmaf(ub0(q1), x1.x, d1[r]);
                d1[r] = fmaf(ub1(q1), x1.y, d1[r]);
                d1[r] = fmaf(ub2(q1), x1.z, d1[r]);
                d1[r] = fmaf(ub3(q1), x1.w, d1[r]);
                d2[r] = fmaf(ub0(q2), x2.x, d2[r]);
                d2[r] = fmaf(ub1(q2), x2.y, d2[r]);
                d2[r] = fmaf(ub2(q2), x2.z, d2[r]);
                d2[r] = fmaf(ub3(q2), x2.w, d2[r]);
                d3[r] = fmaf(ub0(q3), x3.x, d3[r]);
                d3[r] = fmaf(ub1(q3), x3.y, d3[r]);
                d3[r] = fmaf(ub2(q3), x3.z, d3[r]);
                d3[r] = fmaf(ub3(q3), x3.w, d3[r]);
                d4[r] = fmaf(ub0(q4), x4.x, d4[r]);
                d4[r] = fmaf(ub1(q4), x4.y, d4[r]);
                d4[r] = fmaf(ub2(q4), x4.z, d4[r]);
                d4[r] = fmaf(ub3(q4), x4.w, d4[r]);
            }
        }
        const uint32_t sb = (tile & 1u) * 8u;  // bit offset of scales[is], is = tile & 1
        const float s0 = s[0], s1 = s[1], s2 = s[2], s3 = s[3];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float sc1 = sb0(w[r].sc.x >> sb), sc2 = sb0(w[r].sc.x >> (sb + 16)),
                        sc3 = sb0(w[r].sc.y >> sb), sc4 = sb0(w[r].sc.y >> (sb + 16));
            // q - 32 folded in through the sub-block sums of x.
            float v = sc1 * fmaf(-32.f, s0, d1[r]);
            v = fmaf(sc2, fmaf(-32.f, s1, d2[r]), v);
            v = fmaf(sc3, fmaf(-32.f, s2, d3[r]), v);
            v = fmaf(sc4, fmaf(-32.f, s3, d4[r]), v);
            acc[r] = fmaf(f16_bits_to_f32(w[r].d), v, acc[r]);
        }
    }
};

// ------------------------------------------------------------------ Q8_0 ----
struct FmtQ8_0 {
    static constexpr int TILE = 32;
    static constexpr int CHUNKS = 8;
    static constexpr int NSUM = 1;  // sum of the tile's x: quants are used as q + 128
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
    __device__ static void load(Row &w, const RowBase &rb, uint32_t tile) {
        const uint4 *q = reinterpret_cast<const uint4 *>(rb.qs + (size_t)tile * 32);
        w.a = q[0];
        w.b = q[1];
        w.d = *reinterpret_cast<const uint16_t *>(rb.d + (size_t)tile * 2);
    }
    template <int R>
    __device__ static void accumulate(const Row (&w)[R], const float4 *xl, const float *s,
                                      uint32_t, float (&acc)[R]) {
        float dt[R];
#pragma unroll
        for (int r = 0; r < R; ++r) dt[r] = 0.f;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float4 xv = xl[k * 64];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t q = k < 4 ? (&w[r].a.x)[k] : (&w[r].b.x)[k - 4];
                const uint32_t u = opaque(q ^ 0x80808080u);  // q + 128 per byte, unsigned
                dt[r] = fmaf(ub0(u), xv.x, dt[r]);
                dt[r] = fmaf(ub1(u), xv.y, dt[r]);
                dt[r] = fmaf(ub2(u), xv.z, dt[r]);
                dt[r] = fmaf(ub3(u), xv.w, dt[r]);
            }
        }
        const float s0 = s[0];
#pragma unroll
        for (int r = 0; r < R; ++r)
            acc[r] = fmaf(f16_bits_to_f32(w[r].d), fmaf(-128.f, s0, dt[r]), acc[r]);
    }
};

// ----------------------------------------- the 32-element GGUF blocks ----
// Q4_0 (18 B: d, 16 B of nibbles), Q4_1 (20 B: d, m, nibbles), Q5_0 (22 B: d, 32 fifth
// bits, nibbles), Q5_1 (24 B: d, m, fifth bits, nibbles); quantization.rs:47-162 of the
// reference.  The bytes stay as in the GGUF file (blocks are only 2-byte aligned: the loads
// below are unaligned 16-byte loads, which gfx950 serves).  A tile is one block: element k
// of a block is the low nibble of qs[k] for k < 16, the high nibble of qs[k-16] otherwise,
// plus bit k of qh as its fifth bit.  Integer-dot kernels only.
template <int BYTES, bool HAS_M, bool HAS_QH>
struct FmtLegacy {
    struct Row {
        uint4 q;
        uint32_t qh;
        uint16_t d, m;
    };
    struct RowBase {
        const uint8_t *blocks;
    };
    __device__ static RowBase row_base(const GemvParams &p, uint32_t row) {
        return {p.p0 + (size_t)row * (p.ncols / 32) * BYTES};
    }
    __device__ static void load(Row &w, const RowBase &rb, uint32_t tile) {
        const uint8_t *b = rb.blocks + (size_t)tile * BYTES;
        __builtin_memcpy(&w.d, b, 2);
        w.m = 0;
        w.qh = 0;
        if (HAS_M) __builtin_memcpy(&w.m, b + 2, 2);
        if (HAS_QH) __builtin_memcpy(&w.qh, b + 2 + (HAS_M ? 2 : 0), 4);
        __builtin_memcpy(&w.q, b + 2 + (HAS_M ? 2 : 0) + (HAS_QH ? 4 : 0), 16);
    }
};
using FmtQ4_0 = FmtLegacy<18, false, false>;
using FmtQ4_1 = FmtLegacy<20, true, false>;
using FmtQ5_0 = FmtLegacy<22, false, true>;
using FmtQ5_1 = FmtLegacy<24, true, true>;

// Q8_K (292 B: f32 d, 256 int8, 16 block sums that dequantization does not use;
// quantization.rs:170-199).  A tile is 32 of the 256 quants.
struct FmtQ8K {
    struct Row {
        uint4 a, b;
        float d;
    };
    struct RowBase {
        const uint8_t *blocks;
    };
    __device__ static RowBase row_base(const GemvParams &p, uint32_t row) {
        return {p.p0 + (size_t)row * (p.ncols / 256) * 292};
    }
    __device__ static void load(Row &w, const RowBase &rb, uint32_t tile) {
        const uint8_t *b = rb.blocks + (size_t)(tile >> 3) * 292;
        __builtin_memcpy(&w.d, b, 4);
        __builtin_memcpy(&w.a, b + 4 + (tile & 7) * 32, 16);
        __builtin_memcpy(&w.b, b + 4 + (tile & 7) * 32 + 16, 16);
    }
};

// Q5_K (176 B: d, dmin, scales[12] as Q4_K, 32 bytes of fifth bits, 128 bytes of nibbles;
// quantization.rs:249-317).  A tile is a 64-element group as for Q4_K: sub-blocks 2j (low
// nibbles) and 2j+1 (high nibbles), whose fifth bits are bits 2j and 2j+1 of qh[l].
struct FmtQ5K {
    struct Row {
        uint4 hdr, qa, qb, ha, hb;
    };
    struct RowBase {
        const uint8_t *blocks;
    };
    __device__ static RowBase row_base(const GemvParams &p, uint32_t row) {
        return {p.p0 + (size_t)row * (p.ncols / 256) * 176};
    }
    __device__ static void load(Row &w, const RowBase &rb, uint32_t tile) {
        const uint8_t *blk = rb.blocks + (size_t)(tile >> 2) * 176;
        w.hdr = *reinterpret_cast<const uint4 *>(blk);
        w.ha = *reinterpret_cast<const uint4 *>(blk + 16);
        w.hb = *reinterpret_cast<const uint4 *>(blk + 32);
        const uint4 *q = reinterpret_cast<const uint4 *>(blk + 48 + (tile & 3) * 32);
        w.qa = q[0];
        w.qb = q[1];
    }
};

// LDS layout: x as float4 xs[step][chunk][lane]; then sums[sum][tile_padded].
template <class F>
__device__ __forceinline__ uint32_t lds_slot(uint32_t tile, uint32_t chunk) {
    return ((tile >> 6) * F::CHUNKS + chunk) * 64 + (tile & 63);
}

// rsqrt(mean(x^2) + eps) over the whole vector, computed by the workgroup
// (ops/rms_norm.wgsl:36-60 of the reference).  Contains barriers.
__device__ __forceinline__ float block_rms_scale(const GemvParams &p, float *red) {
    const float4 *x4 = reinterpret_cast<const float4 *>(p.x);
    const uint32_t n4 = p.ncols >> 2;
    float ss = 0.f;
    for (uint32_t g4 = threadIdx.x; g4 < n4; g4 += blockDim.x) {
        const float4 v = x4[g4];
        ss = fmaf(v.x, v.x, ss);
        ss = fmaf(v.y, v.y, ss);
        ss = fmaf(v.z, v.z, ss);
        ss = fmaf(v.w, v.w, ss);
    }
    const float total = block_sum(ss, red);
    return 1.0f / sqrtf(total / (float)p.ncols + p.norm_eps);
}

__device__ __forceinline__ float4 apply_norm(float4 v, float rms, const float4 w) {
    v.x = (v.x * rms) * w.x;
    v.y = (v.y * rms) * w.y;
    v.z = (v.z * rms) * w.z;
    v.w = (v.w * rms) * w.w;
    return v;
}

// Loads the tiles of the R rows of row-group `g` for tile index `tile`.
template <class F, int R>
__device__ __forceinline__ void load_group(typename F::Row (&w)[R], const GemvParams &p,
                                           uint32_t g, uint32_t tile) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint32_t row = min(g * R + r, p.nrows - 1);
        F::load(w[r], F::row_base(p, row), tile);
    }
}

// =========================================================================
// Integer-dot path (default).  The fp32 path above spends ~3 VALU operations
// per weight element (convert, multiply-add, unpack), which makes the 4-bit
// formats issue-bound on the four SIMD16 units of a CU well below HBM speed.
// Here the activation vector is staged once per workgroup as 16-bit block
// fixed point: per block of XB elements a scale s = max|x| / 32512 and
// X = round(x / s), stored as two int8 planes X = 256*hi + lo (hi in
// [-127,127], lo in [-128,127]).  Weights are unpacked to bytes and multiplied
// with v_dot4c_i32_i8 (four exact integer MACs per lane-operation); the two
// int32 partial sums are recombined as 256*hi + lo and scaled once per
// sub-block in fp32.  The rounding of x is at most 2^-16 of the block maximum
// per element (about 3e-5 of a block's RMS), i.e. ~30x inside the 1e-3
// tolerance of the GEMV.  The result is the product of the exactly dequantized
// weights with the rounded activation vector: the block sums used for the
// minima / offsets are sums of the rounded values too.  Everything after the
// sub-block dot product is fp32.
// =========================================================================

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ int sdot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

template <int CTRL>
__device__ __forceinline__ float dpp_max(float v) {
    return fmaxf(v, dpp_f32<CTRL>(v));
}

// --- formats: TILE elements per lane, XB elements per activation block ------
struct IFmtQ4K {
    using W = FmtQ4K;
    static constexpr bool F32X = false;
    static constexpr int TILE = 64, XB = 32, NXB = 2, NSUM = 2;
    // element index e of x -> tile, element within tile, block within tile
    __device__ static void locate(uint32_t e, uint32_t &tile, uint32_t &local, uint32_t &xb) {
        tile = e >> 6;
        local = e & 63;
        xb = local >> 5;
    }
    // A lane's tile of the staged activations.
    struct X {
        uint4 xh[4], xl[4];
        float4 mt;  // s0, s1, S0, S1
    };
    // xq: this lane's slot of chunk 0 of the hi plane; chunk c at xq[c*64], lo plane 4 chunks on
    __device__ static void load_x(X &x, const uint4 *xq, const float *meta) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            x.xh[c] = xq[c * 64];
            x.xl[c] = xq[(4 + c) * 64];
        }
        x.mt = *reinterpret_cast<const float4 *>(meta);
    }
    template <int R>
    __device__ static void accumulate(const W::Row (&w)[R], const X &x, uint32_t tile,
                                      float (&acc)[R]) {
        const uint4(&xh)[4] = x.xh;
        const uint4(&xl)[4] = x.xl;
        const float4 mt = x.mt;
        const uint32_t j = tile & 3;
        const uint32_t sh = (j & 1u) * 16u;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int hlo = 0, llo = 0, hhi = 0, lhi = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const uint32_t q = k < 4 ? (&w[r].qa.x)[k] : (&w[r].qb.x)[k - 4];
                const uint32_t lo = q & 0x0f0f0f0fu, hi = (q >> 4) & 0x0f0f0f0fu;
                hlo = sdot4(lo, (&xh[k >> 2].x)[k & 3], hlo);
                llo = sdot4(lo, (&xl[k >> 2].x)[k & 3], llo);
                hhi = sdot4(hi, (&xh[2 + (k >> 2)].x)[k & 3], hhi);
                lhi = sdot4(hi, (&xl[2 + (k >> 2)].x)[k & 3], lhi);
            }
            const float flo = (float)((hlo << 8) + llo) * mt.x;
            const float fhi = (float)((hhi << 8) + lhi) * mt.y;
            const float d = f16_bits_to_f32((uint16_t)(w[r].hdr.x & 0xffffu));
            const float dmin = f16_bits_to_f32((uint16_t)(w[r].hdr.x >> 16));
            const uint32_t a = (w[r].hdr.y >> sh) & 0xffffu, b = (w[r].hdr.z >> sh) & 0xffffu,
                           c = (w[r].hdr.w >> sh) & 0xffffu;
            uint32_t sc2, m2;
            if (j < 2) {
                sc2 = a & 0x3f3fu;
                m2 = b & 0x3f3fu;
            } else {
                sc2 = (c & 0x0f0fu) | ((a >> 2) & 0x3030u);
                m2 = ((c >> 4) & 0x0f0fu) | ((b >> 2) & 0x3030u);
            }
            float v = (d * ub0(sc2)) * flo;
            v = fmaf(d * ub1(sc2), fhi, v);
            v = fmaf(-dmin, fmaf(ub0(m2), mt.z, ub1(m2) * mt.w), v);
            acc[r] += v;
        }
    }
};

struct IFmtQ6K {
    using W = FmtQ6K;
    static constexpr bool F32X = false;
    static constexpr int TILE = 64, XB = 16, NXB = 4, NSUM = 4;
    __device__ static void locate(uint32_t e, uint32_t &tile, uint32_t &local, uint32_t &xb) {
        const uint32_t blk = e >> 8, i = (e >> 7) & 1, quarter = (e >> 5) & 3, s = (e >> 4) & 1;
        tile = blk * 4 + i * 2 + s;
        xb = quarter;
        local = quarter * 16 + (e & 15);
    }
    struct X {
        uint4 xh[4], xl[4];  // chunk = quarter
        float4 ms, mS;       // scales of the 4 quarters, sums of the rounded values
    };
    __device__ static void load_x(X &x, const uint4 *xq, const float *meta) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            x.xh[c] = xq[c * 64];
            x.xl[c] = xq[(4 + c) * 64];
        }
        x.ms = *reinterpret_cast<const float4 *>(meta);
        x.mS = *reinterpret_cast<const float4 *>(meta + 4);
    }
    template <int R>
    __device__ static void accumulate(const W::Row (&w)[R], const X &x, uint32_t tile,
                                      float (&acc)[R]) {
        const uint4(&xh)[4] = x.xh;
        const uint4(&xl)[4] = x.xl;
        const float4 ms = x.ms, mS = x.mS;
        const uint32_t sb = (tile & 1u) * 8u;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int h1 = 0, l1 = 0, h2 = 0, l2 = 0, h3 = 0, l3 = 0, h4 = 0, l4 = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t L0 = (&w[r].l0.x)[k], L1 = (&w[r].l1.x)[k], H = (&w[r].h.x)[k];
                const uint32_t q1 = (L0 & 0x0f0f0f0fu) | ((H << 4) & 0x30303030u);
                const uint32_t q2 = (L1 & 0x0f0f0f0fu) | ((H << 2) & 0x30303030u);
                const uint32_t q3 = ((L0 >> 4) & 0x0f0f0f0fu) | (H & 0x30303030u);
                const uint32_t q4 = ((L1 >> 4) & 0x0f0f0f0fu) | ((H >> 2) & 0x30303030u);
                h1 = sdot4(q1, (&xh[0].x)[k], h1);
                l1 = sdot4(q1, (&xl[0].x)[k], l1);
                h2 = sdot4(q2, (&xh[1].x)[k], h2);
                l2 = sdot4(q2, (&xl[1].x)[k], l2);
                h3 = sdot4(q3, (&xh[2].x)[k], h3);
                l3 = sdot4(q3, (&xl[2].x)[k], l3);
                h4 = sdot4(q4, (&xh[3].x)[k], h4);
                l4 = sdot4(q4, (&xl[3].x)[k], l4);
            }
            const float f1 = fmaf((float)((h1 << 8) + l1), ms.x, -32.f * mS.x);
            const float f2 = fmaf((float)((h2 << 8) + l2), ms.y, -32.f * mS.y);
            const float f3 = fmaf((float)((h3 << 8) + l3), ms.z, -32.f * mS.z);
            const float f4 = fmaf((float)((h4 << 8) + l4), ms.w, -32.f * mS.w);
            const float sc1 = sb0(w[r].sc.x >> sb), sc2 = sb0(w[r].sc.x >> (sb + 16)),
                        sc3 = sb0(w[r].sc.y >> sb), sc4 = sb0(w[r].sc.y >> (sb + 16));
            float v = sc1 * f1;
            v = fmaf(sc2, f2, v);
            v = fmaf(sc3, f3, v);
            v = fmaf(sc4, f4, v);
            acc[r] = fmaf(f16_bits_to_f32(w[r].d), v, acc[r]);
        }
    }
};

struct IFmtQ8_0 {
    using W = FmtQ8_0;
    static constexpr bool F32X = false;
    static constexpr int TILE = 32, XB = 32, NXB = 1, NSUM = 0;
    __device__ static void locate(uint32_t e, uint32_t &tile, uint32_t &local, uint32_t &xb) {
        tile = e >> 5;
        local = e & 31;
        xb = 0;
    }
    struct X {
        uint4 xh[2], xl[2];
        float s0;
    };
    __device__ static void load_x(X &x, const uint4 *xq, const float *meta) {
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            x.xh[c] = xq[c * 64];
            x.xl[c] = xq[(2 + c) * 64];
        }
        x.s0 = meta[0];
    }
    template <int R>
    __device__ static void accumulate(const W::Row (&w)[R], const X &x, uint32_t,
                                      float (&acc)[R]) {
        const uint4(&xh)[2] = x.xh;
        const uint4(&xl)[2] = x.xl;
        const float s0 = x.s0;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int h = 0, l = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const uint32_t q = k < 4 ? (&w[r].a.x)[k] : (&w[r].b.x)[k - 4];
                h = sdot4(q, (&xh[k >> 2].x)[k & 3], h);
                l = sdot4(q, (&xl[k >> 2].x)[k & 3], l);
            }
            acc[r] = fmaf(f16_bits_to_f32(w[r].d) * s0, (float)((h << 8) + l), acc[r]);
        }
    }
};

// Bits 0..3 of b moved to bit 4 of bytes 0..3 (the fifth bits of four 5-bit quants).
__device__ __forceinline__ uint32_t spread_bit4(uint32_t b) {
    return ((b * 0x00204081u) & 0x01010101u) << 4;
}

template <int BYTES, bool HAS_M, bool HAS_QH>
struct IFmtLegacy {
    using W = FmtLegacy<BYTES, HAS_M, HAS_QH>;
    static constexpr bool F32X = false;
    static constexpr int TILE = 32, XB = 32, NXB = 1, NSUM = 1;
    __device__ static void locate(uint32_t e, uint32_t &tile, uint32_t &local, uint32_t &xb) {
        tile = e >> 5;
        local = e & 31;
        xb = 0;
    }
    struct X {
        uint4 xh[2], xl[2];
        float s0, S0;  // scale of the block's fixed-point activations, sum of the rounded values
    };
    __device__ static void load_x(X &x, const uint4 *xq, const float *meta) {
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            x.xh[c] = xq[c * 64];
            x.xl[c] = xq[(2 + c) * 64];
        }
        x.s0 = meta[0];
        x.S0 = meta[1];
    }
    template <int R>
    __device__ static void accumulate(const typename W::Row (&w)[R], const X &x, uint32_t,
                                      float (&acc)[R]) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int h = 0, l = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t q = (&w[r].q.x)[k];
                uint32_t lo = q & 0x0f0f0f0fu, hi = (q >> 4) & 0x0f0f0f0fu;
                if (HAS_QH) {
                    lo |= spread_bit4((w[r].qh >> (4 * k)) & 15u);
                    hi |= spread_bit4((w[r].qh >> (16 + 4 * k)) & 15u);
                }
                h = sdot4(lo, (&x.xh[0].x)[k], h);
                l = sdot4(lo, (&x.xl[0].x)[k], l);
                h = sdot4(hi, (&x.xh[1].x)[k], h);
                l = sdot4(hi, (&x.xl[1].x)[k], l);
            }
            const float dot = (float)((h << 8) + l) * x.s0;  // sum of quant * x over the block
            const float d = f16_bits_to_f32(w[r].d);
            if (HAS_M)  // y = d q + m   (quantization.rs:93-96, 160-165)
                acc[r] += fmaf(d, dot, f16_bits_to_f32(w[r].m) * x.S0);
            else  // y = d (q - 8) or d (q - 16)   (quantization.rs:62-66, 123-129)
                acc[r] = fmaf(d, fmaf(HAS_QH ? -16.f : -8.f, x.S0, dot), acc[r]);
        }
    }
};
using IFmtQ4_0 = IFmtLegacy<18, false, false>;
using IFmtQ4_1 = IFmtLegacy<20, true, false>;
using IFmtQ5_0 = IFmtLegacy<22, false, true>;
using IFmtQ5_1 = IFmtLegacy<24, true, true>;

struct IFmtQ8K {
    using W = FmtQ8K;
    static constexpr bool F32X = false;
    static constexpr int TILE = 32, XB = 32, NXB = 1, NSUM = 0;
    __device__ static void locate(uint32_t e, uint32_t &tile, uint32_t &local, uint32_t &xb) {
        tile = e >> 5;
        local = e & 31;
        xb = 0;
    }
    using X = IFmtQ8_0::X;
    __device__ static void load_x(X &x, const uint4 *xq, const float *meta) {
        IFmtQ8_0::load_x(x, xq, meta);
    }
    template <int R>
    __device__ static void accumulate(const W::Row (&w)[R], const X &x, uint32_t,
                                      float (&acc)[R]) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int h = 0, l = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const uint32_t q = k < 4 ? (&w[r].a.x)[k] : (&w[r].b.x)[k - 4];
                h = sdot4(q, (&x.xh[k >> 2].x)[k & 3], h);
                l = sdot4(q, (&x.xl[k >> 2].x)[k & 3], l);
            }
            acc[r] = fmaf(w[r].d * x.s0, (float)((h << 8) + l), acc[r]);
        }
    }
};

struct IFmtQ5K {
    using W = FmtQ5K;
    static constexpr bool F32X = false;
    static constexpr int TILE = 64, XB = 32, NXB = 2, NSUM = 2;
    __device__ static void locate(uint32_t e, uint32_t &tile, uint32_t &local, uint32_t &xb) {
        IFmtQ4K::locate(e, tile, local, xb);
    }
    using X = IFmtQ4K::X;
    __device__ static void load_x(X &x, const uint4 *xq, const float *meta) {
        IFmtQ4K::load_x(x, xq, meta);
    }
    template <int R>
    __device__ static void accumulate(const W::Row (&w)[R], const X &x, uint32_t tile,
                                      float (&acc)[R]) {
        const uint4(&xh)[4] = x.xh;
        const uint4(&xl)[4] = x.xl;
        const float4 mt = x.mt;
        const uint32_t j = tile & 3;
        const uint32_t sh = (j & 1u) * 16u;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int hlo = 0, llo = 0, hhi = 0, lhi = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const uint32_t q = k < 4 ? (&w[r].qa.x)[k] : (&w[r].qb.x)[k - 4];
                const uint32_t H = (k < 4 ? (&w[r].ha.x)[k] : (&w[r].hb.x)[k - 4]) >> (2 * j);
                const uint32_t lo = (q & 0x0f0f0f0fu) | ((H & 0x01010101u) << 4);
                const uint32_t hi = ((q >> 4) & 0x0f0f0f0fu) | (((H >> 1) & 0x01010101u) << 4);
                hlo = sdot4(lo, (&xh[k >> 2].x)[k & 3], hlo);
                llo = sdot4(lo, (&xl[k >> 2].x)[k & 3], llo);
                hhi = sdot4(hi, (&xh[2 + (k >> 2)].x)[k & 3], hhi);
                lhi = sdot4(hi, (&xl[2 + (k >> 2)].x)[k & 3], lhi);
            }
            const float flo = (float)((hlo << 8) + llo) * mt.x;
            const float fhi = (float)((hhi << 8) + lhi) * mt.y;
            const float d = f16_bits_to_f32((uint16_t)(w[r].hdr.x & 0xffffu));
            const float dmin = f16_bits_to_f32((uint16_t)(w[r].hdr.x >> 16));
            // 6-bit scale / min pairs of sub-blocks 2j and 2j+1 (get_scale_min_k4)
            const uint32_t a = (w[r].hdr.y >> sh) & 0xffffu, b = (w[r].hdr.z >> sh) & 0xffffu,
                           c = (w[r].hdr.w >> sh) & 0xffffu;
            uint32_t sc2, m2;
            if (j < 2) {
                sc2 = a & 0x3f3fu;
                m2 = b & 0x3f3fu;
            } else {
                sc2 = (c & 0x0f0fu) | ((a >> 2) & 0x3030u);
                m2 = ((c >> 4) & 0x0f0fu) | ((b >> 2) & 0x3030u);
            }
            float v = (d * ub0(sc2)) * flo;
            v = fmaf(d * ub1(sc2), fhi, v);
            v = fmaf(-dmin, fmaf(ub0(m2), mt.z, ub1(m2) * mt.w), v);
            acc[r] += v;
        }
    }
};

// The fp32-activation twin of a format: x is staged in LDS as it is (RMSNorm / LayerNorm applied),
// float4 xs[step][chunk][lane] followed by the NSUM sums of x per tile, and the weights are
// expanded with one conversion and one multiply-add per element (FmtQ4K / FmtQ6K / FmtQ8_0
// ::accumulate).  The arithmetic the reference's shaders use (ops/gemv_quant.rs:243-348 multiply
// f32 vectors); about 3 VALU operations per weight against 1 on the integer-dot path.
template <class WFmt>
struct FFmt {
    using W = WFmt;
    static constexpr bool F32X = true;
    static constexpr int TILE = WFmt::TILE, CHUNKS = WFmt::CHUNKS, NSUM = WFmt::NSUM;
    static constexpr int XB = WFmt::TILE / WFmt::NSUM, NXB = 0;  // elements per sum of x
    struct X {};
};

// Row source / sink of a plain single-matrix GEMV: group g = rows g*R .. g*R+R-1.
struct PlainPolicy {
    static constexpr int S = 1;  // passes per group
    const GemvParams &p;
    // `ok` false: the load still happens, from row-group 0 (a wave's loads are never
    // skipped, see gemv_i8_body)
    template <class WF, int R>
    __device__ void load(typename WF::Row (&w)[R], uint32_t g, uint32_t, uint32_t tile,
                         bool ok) const {
        load_group<WF, R>(w, p, ok ? g : 0u, tile);
    }
    // Lane n holds finished result n of the wave, whose first group is g0: result n
    // belongs to row (g0 + (n / R) * GW) * R + n % R.  The operands the epilogue needs
    // are fetched by prefetch() at kernel start: fetched at the end they would add a
    // memory round trip to every wave's tail.
    float *out;
    float pre_bias, pre_out;
    uint32_t pos;
    __device__ const uint32_t *pos_ptr() const { return p.dyn_pos; }
    __device__ void set_pos(uint32_t fetched) { pos = fetched; }
    // `late` false: at kernel start, whatever does not need the position; true: behind the
    // first weight tiles, once the position is there, the rest.
    template <int R>
    __device__ void prefetch(bool late, uint32_t g0, uint32_t GW, uint32_t my_groups, uint32_t lane) {
        const uint32_t row = (g0 + (lane / R) * GW) * R + lane % R;
        const bool mine = lane < my_groups * R && row < p.nrows;
        if (!late) {
            out = p.out;
            pre_bias = pre_out = 0.f;
            if (mine && p.bias) pre_bias = p.bias[row];
            if (mine && p.accumulate && !p.dyn_pos) pre_out = out[row];
        } else if (p.dyn_pos) {
            out += (size_t)pos * p.out_pos_stride;
            if (mine && p.accumulate) pre_out = out[row];
        }
    }
    template <int R>
    __device__ void finish(float mine, uint32_t n, uint32_t g0, uint32_t GW, uint32_t lane) {
        const uint32_t row = (g0 + (lane / R) * GW) * R + lane % R;
        if (lane < n && row < p.nrows) {
            float v = mine + pre_bias;
            if (p.act == 1) v = gelu_tanh(v);
            out[row] = v + pre_out;
        }
    }
};

// The body shared by the single-matrix and the fused multi-matrix kernels.  `p`
// supplies x, ncols and the optional norm folding; `pol` the rows.
// The workgroup is number `wg` of the `nwg` that share the matrix; its waves
// w < nw take the row-groups (wg * nw + w) + i * (nwg * nw) < ngroups, so that at
// any time the machine reads one contiguous window of the matrix.  A group is
// Policy::S passes over R rows each (a fused pair is two single-row passes of
// the same wave).  The (group, pass, step) triples
// of a wave form one sequence that is software-pipelined D deep.
// LDS: uint4 xq[step][plane(2)][chunk(PCH)][lane(64)], then float meta[tile][MF].
// XREG: rows fit one step (ncols <= 64 tiles), so a lane's tile of x is the same
// for every row and is read from LDS once instead of once per row.
// XPART: x is not read from p.x but merged from attention partial results (merged_partials).
template <class F, int R, int D, bool XREG, class Policy, bool XPART = false>
__device__ __forceinline__ void gemv_i8_body(const GemvParams &p, Policy &pol, uint32_t wg,
                                             uint32_t nwg, uint32_t nw, uint32_t ngroups) {
    using WF = typename F::W;
    constexpr int S = Policy::S;
    constexpr int PCH = F::TILE / 16;         // 16-byte chunks per plane per tile
    constexpr int MF = F::NXB + F::NSUM;      // floats of meta per tile
    constexpr int LPB = F::XB / 4;            // lanes (float4) per activation block (fp32: per sum)
    static_assert(!(F::F32X && XREG), "fp32 activations are read from LDS tile by tile");
    extern __shared__ float4 smem4[];
    uint4 *xq = reinterpret_cast<uint4 *>(smem4);
    // the wave index is read through readfirstlane: the compiler then knows that it,
    // and the loop control derived from it, are the same in every lane (scalar registers
    // and branches instead of vector compares and masks)
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t nwaves = blockDim.x >> 6;
    const uint32_t ntiles = p.ncols / F::TILE;
    const uint32_t nsteps = (ntiles + 63) >> 6;
    const uint32_t ntiles_pad = nsteps << 6;
    float *meta = reinterpret_cast<float *>(xq + (size_t)ntiles_pad * 2 * PCH);
    // fp32 activations: the tile sums follow the ntiles_pad * CHUNKS float4 of x
    float *fsums = reinterpret_cast<float *>(smem4 + (size_t)ntiles_pad * (F::TILE / 4));

    const uint32_t first = wg * nw + wave, GW = nwg * nw;
    const uint32_t my_groups = (wave < nw && first < ngroups) ? (ngroups - first + GW - 1) / GW : 0;
    const uint32_t n_it = my_groups * S * nsteps;

    // the epilogue's operands that do not depend on the position (bias, RoPE table entry,
    // the value to accumulate into) are requested before anything else
    pol.template prefetch<R>(false, first, GW, my_groups, lane);

    // The requests for x go out first, the first D weight requests after them: a
    // wave's loads return in order, so x, a cache hit, is not held up behind the
    // weights and is staged while they are in flight.
    // The position (when it lives in device memory) is requested by a vector load ahead of
    // x: it returns in order with x, so it is there once x has been staged, and no scalar
    // round trip for it stands between the kernel's start and its first weight request.
    const uint32_t *pos_src = pol.pos_ptr();
    uint32_t pos_fetched = 0;
    if (pos_src) pos_fetched = pos_src[opaque(0u)];
    constexpr int XP = 3;  // float4 of x per thread requested up front
    const float4 *x4 = reinterpret_cast<const float4 *>(p.x);
    const float4 *nw4 = reinterpret_cast<const float4 *>(p.norm_w);
    const uint32_t n4 = p.ncols >> 2;
    // (The x loads stay under their conditions: clamping the out-of-range ones to a
    // valid address instead makes every idle thread of the machine hit the same
    // cache line, which cost 1 us on a 4096x4096 launch.)
    // nv: the RMSNorm weights, or gamma of a folded LayerNorm; bv: its beta.  They are
    // requested here, ahead of the weights, so that waiting for them later does not
    // mean waiting for a weight tile.
    // Only the first `ns` waves stage x (as few as cover it with their XP float4 per lane,
    // in fours so that every SIMD takes part): the waves of a 1024-thread workgroup start
    // up to a microsecond apart, and the staging would otherwise end a whole prologue after
    // the last of them has arrived.  The other waves request their weights and wait at the
    // barrier.  (The folded LayerNorm has barriers of its own, so there every wave stages.)
    // (Merging partial results is several loads per float4: every wave takes a share.)
    uint32_t ns = ((n4 + 64 * XP - 1) / (64 * XP) + 3) & ~3u;
    if (ns > nwaves || p.ln_g || XPART) ns = nwaves;
    const bool stager = wave < ns;
    // a wave with neither rows nor a share of x is done: the barrier below counts only the
    // waves that are still running, and it would be the last to reach it
    if (n_it == 0 && !stager) return;
    const uint32_t sthreads = ns * 64;
    float4 xv[XP], nv[XP], bv[XP];
    const float4 *gsrc = p.ln_g ? reinterpret_cast<const float4 *>(p.ln_g) : nw4;
    const float4 *bsrc = reinterpret_cast<const float4 *>(p.ln_b);
#pragma unroll
    for (int i = 0; i < XP; ++i) {
        const uint32_t g4 = stager ? tid + i * sthreads : n4;
        xv[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        nv[i] = make_float4(1.f, 1.f, 1.f, 1.f);
        bv[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (g4 < n4) {
            if constexpr (!XPART) xv[i] = x4[g4];
            if (gsrc) nv[i] = gsrc[g4];
            if (p.ln_g && bsrc) bv[i] = bsrc[g4];
        }
    }
    // XPART: the first eight partial results of each thread's first float4 are requested here,
    // ahead of the weights, and merged in stage_x once they are there (merging them here would
    // put a memory round trip in front of the first weight request)
    PartialChunk early;
    if constexpr (XPART) {
        load_partials(early, p, min(tid, n4 - 1), 0);  // unconditional, see there
        // the compiler must not move the weight requests below ahead of these (a wave's loads
        // return in the order they were issued)
        asm volatile("" ::: "memory");
    }

    // Stage x as 16-bit block fixed point (two int8 planes) + per-block scale and sum.
    // A fused RMSNorm costs no extra pass and no extra barrier: the normalisation
    // factor rsqrt(mean(x^2) + eps) is one scalar for the whole vector, so x * w is
    // staged, the sum of squares is gathered on the way and the factor multiplies
    // the finished dot products instead.
    __shared__ float red[16], red_a[16], red_b[16];
    auto stage_x = [&]() -> float {
        float out_scale = 1.f;
        uint32_t *xq32 = reinterpret_cast<uint32_t *>(xq);
        float ss = 0.f;
        if constexpr (XPART) {  // every wave stages (sthreads == blockDim.x)
            if (tid < n4) xv[0] = merged_partials(p, tid, early);
#pragma unroll
            for (int i = 1; i < XP; ++i)
                if (tid + i * sthreads < n4) xv[i] = merged_partials(p, tid + i * sthreads);
        }
        if (p.ln_g) {
            // LayerNorm folded in (host guarantees that the XP float4 per thread cover
            // x): mean, then variance about the mean (two exact passes over registers,
            // ops/layernorm.rs:46-53), then x <- (x - mean) * rstd * gamma + beta.
            auto block_total = [&](float v, float *buf) {
                v = wave_sum(v);
                if (lane == 0) buf[wave] = v;
                __syncthreads();
                const float part = lane < nwaves ? buf[lane] : 0.f;
                return readlane_f32(row16_sum(part), 0);
            };
            float s1 = 0.f;
#pragma unroll
            for (int i = 0; i < XP; ++i)
                if (tid + i * blockDim.x < n4) s1 += (xv[i].x + xv[i].y) + (xv[i].z + xv[i].w);
            const float mean = block_total(s1, red_a) / (float)p.ncols;
            float s2 = 0.f;
#pragma unroll
            for (int i = 0; i < XP; ++i) {
                if (tid + i * blockDim.x < n4) {
                    xv[i].x -= mean;
                    xv[i].y -= mean;
                    xv[i].z -= mean;
                    xv[i].w -= mean;
                    s2 = fmaf(xv[i].x, xv[i].x, s2);
                    s2 = fmaf(xv[i].y, xv[i].y, s2);
                    s2 = fmaf(xv[i].z, xv[i].z, s2);
                    s2 = fmaf(xv[i].w, xv[i].w, s2);
                }
            }
            const float rstd = 1.0f / sqrtf(block_total(s2, red_b) / (float)p.ncols + 1.0e-5f);
#pragma unroll
            for (int i = 0; i < XP; ++i) {
                const uint32_t g4 = tid + i * blockDim.x;
                if (g4 < n4) {
                    const float4 ga = nv[i], be = bv[i];
                    xv[i].x = (xv[i].x * rstd) * ga.x + be.x;
                    xv[i].y = (xv[i].y * rstd) * ga.y + be.y;
                    xv[i].z = (xv[i].z * rstd) * ga.z + be.z;
                    xv[i].w = (xv[i].w * rstd) * ga.w + be.w;
                }
            }
        }
        auto stage_one = [&](uint32_t g4, float4 v, const float4 nw) {
            if constexpr (F::F32X) {
                if (p.norm_w) {
                    ss = fmaf(v.x, v.x, ss);
                    ss = fmaf(v.y, v.y, ss);
                    ss = fmaf(v.z, v.z, ss);
                    ss = fmaf(v.w, v.w, ss);
                    v.x *= nw.x;
                    v.y *= nw.y;
                    v.z *= nw.z;
                    v.w *= nw.w;
                }
                uint32_t tile, chunk;
                WF::map(g4, tile, chunk);
                smem4[lds_slot<WF>(tile, chunk)] = v;
                if constexpr (F::NSUM > 0) {
                    // the sum of x over the LPB consecutive float4 that one sum covers
                    float sum = (v.x + v.y) + (v.z + v.w);
                    sum += dpp_f32<0xB1>(sum);
                    sum += dpp_f32<0x4E>(sum);
                    if (LPB == 8) sum += dpp_f32<0x141>(sum);
                    constexpr int CPS = F::CHUNKS / F::NSUM;  // chunks per sum
                    if ((g4 & (LPB - 1)) == 0) fsums[tile * F::NSUM + chunk / CPS] = sum;
                }
            } else {
            if (p.norm_w) {
                ss = fmaf(v.x, v.x, ss);
                ss = fmaf(v.y, v.y, ss);
                ss = fmaf(v.z, v.z, ss);
                ss = fmaf(v.w, v.w, ss);
                v.x *= nw.x;
                v.y *= nw.y;
                v.z *= nw.z;
                v.w *= nw.w;
            }
            float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
            float sum;
            amax = dpp_max<0xB1>(amax);
            amax = dpp_max<0x4E>(amax);
            if (LPB == 8) amax = dpp_max<0x141>(amax);
            const float inv = amax > 0.f ? 32512.f / amax : 0.f;
            const int X0 = __float2int_rn(v.x * inv), X1 = __float2int_rn(v.y * inv),
                      X2 = __float2int_rn(v.z * inv), X3 = __float2int_rn(v.w * inv);
            // block sum of the *rounded* activations, so that the minima / offset terms
            // see exactly the same vector as the dot products (exact in fp32: |sum| < 2^21)
            sum = (float)((X0 + X1) + (X2 + X3));
            sum += dpp_f32<0xB1>(sum);
            sum += dpp_f32<0x4E>(sum);
            if (LPB == 8) sum += dpp_f32<0x141>(sum);
            sum *= amax * (1.0f / 32512.f);
            // X = 256 hi + lo with lo the sign-extended low byte: lo is byte 0 of X as it stands
            // and hi = (X + 128) >> 8 is byte 1 of X + 128 (|X| <= 32512, so 16 bits hold both).
            // Two values per register as 16-bit halves, one packed add, and two byte
            // permutes gather the four lo bytes and the four hi bytes.
            const uint32_t p01 = __builtin_amdgcn_perm((uint32_t)X1, (uint32_t)X0, 0x05040100u);
            const uint32_t p23 = __builtin_amdgcn_perm((uint32_t)X3, (uint32_t)X2, 0x05040100u);
            const u16x2 bias128 = {128, 128};
            u16x2 y01, y23;
            __builtin_memcpy(&y01, &p01, 4);
            __builtin_memcpy(&y23, &p23, 4);
            y01 += bias128;
            y23 += bias128;
            uint32_t q01, q23;
            __builtin_memcpy(&q01, &y01, 4);
            __builtin_memcpy(&q23, &y23, 4);
            const uint32_t lo = __builtin_amdgcn_perm(p23, p01, 0x06040200u);
            const uint32_t hi = __builtin_amdgcn_perm(q23, q01, 0x07050301u);
            uint32_t tile, local, xb;
            F::locate(g4 * 4, tile, local, xb);
            const uint32_t dl = local >> 2, chunk = dl >> 2, sub = dl & 3;
            const uint32_t slot = ((tile >> 6) * 2 * PCH + chunk) * 64 + (tile & 63);
            xq32[(size_t)slot * 4 + sub] = hi;
            xq32[(size_t)(slot + PCH * 64) * 4 + sub] = lo;
            if ((g4 & (LPB - 1)) == 0) {
                meta[tile * MF + xb] = amax * (1.0f / 32512.f);
                if (F::NSUM > 0) meta[tile * MF + F::NXB + xb] = sum;
            }
            }  // integer-dot staging
        };
        // ncols is a multiple of the tile size, so the LPB lanes of a block are
        // active together in every one of these branches
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            const uint32_t g4 = stager ? tid + i * sthreads : n4;
            if (g4 < n4) stage_one(g4, xv[i], nv[i]);
        }
        for (uint32_t g4 = stager ? tid + XP * sthreads : n4; g4 < n4; g4 += sthreads)
            stage_one(g4, XPART ? merged_partials(p, g4) : x4[g4],
                      p.norm_w ? nw4[g4] : make_float4(1.f, 1.f, 1.f, 1.f));
        if (p.norm_w && stager) {
            ss = wave_sum(ss);
            if (lane == 0) red[wave] = ss;
        }
        __syncthreads();
        if (p.norm_w) {
            // one LDS read per lane and a 16-lane DPP sum instead of a chain of
            // dependent reads (a workgroup has at most 16 waves; only the staging ones
            // have written a partial sum)
            const float part = lane < ns ? red[lane] : 0.f;
            const float total = readlane_f32(row16_sum(part), 0);
            out_scale = 1.0f / sqrtf(total / (float)p.ncols + p.norm_eps);
        }
        return out_scale;
    };

    // The weight loads below and in the main loop are issued unconditionally (a lane
    // without a tile re-reads tile 0; a register set beyond the wave's last iteration
    // re-reads the wave's own first tile, a cache hit).  Only then can the compiler
    // count the loads in flight and wait for exactly the one it needs: with a load
    // under a condition it falls back to waiting for all of them, and the staging of
    // x, a cache hit, would wait for the first weight tile to arrive from HBM.
    // A wave without any row re-reads row-group 0: the host sizes the workgroups so that
    // only the last one can have such waves (thousands of idle waves asking for one and
    // the same tile would queue up on a single cache line).
    typename WF::Row w[D][R];
    uint32_t lg = first, lsub = 0, ls = 0;  // (group, pass, step) of the next load
    // A wave's finished row sums are parked one per lane (result n in lane n) until the
    // policy's epilogue at the end, so a wave takes at most 64 results: the host sizes
    // the grid accordingly (plan_groups).  The loads of the first D iterations go out
    // here; with fewer than D iterations the other register sets take a dummy load and
    // are never consumed.
    auto advance_load_cursor = [&]() {
        if (++ls == nsteps) {
            ls = 0;
            if (++lsub == S) {
                lsub = 0;
                lg += GW;
            }
        }
    };
#pragma unroll
    for (int d = 0; d < D; ++d) {
        const bool ok = (uint32_t)d < n_it;
        const uint32_t tile = ok ? ls * 64 + lane : lane;
        // no tile left: the wave's own first one again, or, for a wave without rows, the
        // first one of its workgroup (a hit in the CU's cache either way)
        const uint32_t spare = n_it ? first : (wg * nw < ngroups ? wg * nw : 0u);
        pol.template load<WF, R>(w[d], ok ? lg : spare, ok ? lsub : 0u, tile < ntiles ? tile : 0u, true);
        if (ok) advance_load_cursor();
    }

    const float out_scale = stage_x();
    if (n_it == 0) return;
    // The epilogue's operands whose addresses depend on the position are requested here,
    // behind the first weight tiles: the position is a second memory round trip away from
    // the kernel arguments, and nothing before this point waits for it.
    pol.set_pos((uint32_t)__builtin_amdgcn_readfirstlane((int)pos_fetched));
    pol.template prefetch<R>(true, first, GW, my_groups, lane);

    // XREG: a lane without a tile (rows shorter than 64 tiles) keeps an all-zero tile of
    // x, so that the row loop needs no condition on the lane
    typename F::X xr{};
    if constexpr (XREG) {
        if (lane < ntiles) F::load_x(xr, xq + lane, meta + (size_t)lane * MF);
    }
    uint32_t step = 0;  // step within the row being computed
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;
    uint32_t nres = 0;
    float mine = 0.f;
    // one iteration on a register set: the dot products of a tile, and the row
    // reduction when the row is complete (no memory operation, LDS aside)
    auto compute = [&](typename WF::Row(&wd)[R]) {
        const uint32_t tile = step * 64 + lane;
        if constexpr (F::F32X) {
            if (tile < ntiles)
                WF::template accumulate<R>(wd, smem4 + (size_t)step * F::CHUNKS * 64 + lane,
                                           fsums + (size_t)tile * F::NSUM, tile, acc);
        } else if constexpr (XREG) {
            F::template accumulate<R>(wd, xr, lane, acc);
        } else if (tile < ntiles) {
            typename F::X xt;
            F::load_x(xt, xq + (size_t)step * 2 * PCH * 64 + lane, meta + (size_t)tile * MF);
            F::template accumulate<R>(wd, xt, tile, acc);
        }
        if (XREG || ++step == nsteps) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const float t = wave_sum(acc[r]) * out_scale;
                mine = lane == nres ? t : mine;
                ++nres;
                acc[r] = 0.f;
            }
            step = 0;
        }
    };
    // refills a register set with the next triple of the load cursor
    auto refill = [&](typename WF::Row(&wd)[R]) {
        const uint32_t tile_n = ls * 64 + lane;
        pol.template load<WF, R>(wd, lg, lsub, tile_n < ntiles ? tile_n : 0u, true);
        advance_load_cursor();
    };
    // The last K < 2 D iterations as straight-line code: iteration i runs on
    // register set i mod D and refills it only if iteration i + D exists.  No load sits
    // under a run-time condition, so every wait is for exactly the tile that is needed.
    auto tail = [&](auto kc) {
        constexpr int K = decltype(kc)::value;
#pragma unroll
        for (int i = 0; i < K; ++i) {
            compute(w[i % D]);
            if (i + D < K) refill(w[i % D]);
        }
    };
    uint32_t left = n_it;
    // rounds of D iterations whose refills all exist
    for (; left >= 2u * D; left -= D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            compute(w[d]);
            refill(w[d]);
        }
    }
    switch (left) {  // 1 .. 2 D - 1
#define WGML_TAIL_CASE(K)                                                 \
    case K:                                                               \
        if constexpr (K < 2 * D) tail(std::integral_constant<int, K>{});  \
        break;
        WGML_TAIL_CASE(1)
        WGML_TAIL_CASE(2)
        WGML_TAIL_CASE(3)
        WGML_TAIL_CASE(4)
        WGML_TAIL_CASE(5)
        WGML_TAIL_CASE(6)
        WGML_TAIL_CASE(7)
#undef WGML_TAIL_CASE
    default: break;
    }
    // The policy's epilogue: its loads (bias, RoPE table, the value to accumulate into)
    // were requested at kernel start, its stores come after the last weight tile.
    pol.template finish<R>(mine, nres, first, GW, lane);
}

// MINW: waves per SIMD the register allocation must leave room for (MAXT / 256 = one
// workgroup per CU; twice that caps the kernel at 64 vector registers, so that two
// 1024-thread workgroups share a CU).
template <class F, int R, int D, int MAXT, int MINW = MAXT / 256, bool XPART = false>
__global__ __launch_bounds__(MAXT, MINW) void gemv_quant_i8_kernel(const GemvParams p) {
    PlainPolicy pol{p, nullptr, 0.f, 0.f, 0};
    const uint32_t ngroups = (p.nrows + R - 1) / R;
    if constexpr (!F::F32X) {
        if (p.ncols <= 64 * F::TILE) {
            gemv_i8_body<F, R, D, true, PlainPolicy, XPART>(p, pol, blockIdx.x, gridDim.x,
                                                            p.active_waves, ngroups);
            return;
        }
    }
    gemv_i8_body<F, R, D, false, PlainPolicy, XPART>(p, pol, blockIdx.x, gridDim.x, p.active_waves,
                                                     ngroups);
}

// ------------------------------------------------------------------------
// Fused multi-matrix launch.  Up to three matrices that consume the same input
// vector share one launch (Q, K and V; gate and up): each workgroup works on one
// of them (so mixed quantization formats are fine: the format decides the
// workgroup's staging layout and inner loop), and the row pairs of a wave get an
// epilogue:
//   PLAIN  out[row] = dot (+ bias) (+ out)
//   ROPE   the pair (2g, 2g+1) is rotated by the RoPE angle of pair g before it
//          is stored (ops/rope.wgsl:35-58, adjacent-pair variant)
//   SILU   the wave holds row g of the gate matrix and row g of the up matrix and
//          stores up * gate / (1 + exp(-gate))   (ops/silu.wgsl:13-27)
// Outputs may be displaced by pos * out_pos_stride (KV-cache column of the
// current position).
enum { JOB_PLAIN = 0, JOB_ROPE = 1, JOB_SILU = 2 };

struct GemvJob {
    const uint8_t *a0, *a1, *a2, *a3;  // matrix planes
    const uint8_t *b0, *b1, *b2, *b3;  // second matrix (SILU: a = gate, b = up)
    float *out;
    const float *bias;
    uint32_t nrows;
    int type, mode, accumulate;
    uint32_t out_pos_stride;
    uint32_t wg_begin, wg_count;  // workgroups assigned to this matrix
    uint32_t active_waves;        // waves of a workgroup that walk its row pairs
};

struct FusedParams {
    GemvJob jobs[3];
    const float *x;
    uint32_t ncols;
    const float *norm_w;
    float norm_eps;
    const float *ln_g, *ln_b;
    DynPos pos;
    uint32_t head_size;
    float rope_base;
    const float2 *rope_cs;  // optional: (cos, sin) of the current position per pair of a head
    // The first field a workgroup needs sits in the last cache line of the arguments, so that
    // the first batch of scalar loads touches every line (a line first touched by a later
    // batch is another round trip to memory).
    int njobs;
};

// A group is a pair of rows whose tiles a wave loads together and multiplies with one
// read of its tile of x:
//   PLAIN / ROPE  rows 2g and 2g+1 of the matrix
//   SILU          row g of the gate matrix and row g of the up matrix
struct JobPolicy {
    static constexpr int S = 1;
    const GemvJob &j;
    const GemvParams &pa, &pb;  // plane views of the two matrices
    DynPos dpos;
    uint32_t head_size;
    float rope_base;
    const float2 *rope_cs;
    template <class WF, int R>
    __device__ void load(typename WF::Row (&w)[R], uint32_t g, uint32_t, uint32_t tile,
                         bool ok) const {
        static_assert(R == 2, "fused launches work on row pairs");
        if (!ok) g = 0;
        const bool silu = j.mode == JOB_SILU;
        // plane pointers are picked one by one (wave-uniform selects): choosing between
        // the two parameter blocks by reference would force them into memory
        GemvParams q{};
        q.p0 = silu ? pb.p0 : pa.p0;
        q.p1 = silu ? pb.p1 : pa.p1;
        q.p2 = silu ? pb.p2 : pa.p2;
        q.p3 = silu ? pb.p3 : pa.p3;
        q.ncols = pa.ncols;
        WF::load(w[0], WF::row_base(pa, silu ? g : 2 * g), tile);
        WF::load(w[1], WF::row_base(q, silu ? g : min(2 * g + 1, j.nrows - 1)), tile);
    }
    // Lanes 2i and 2i+1 hold the two results of group g0 + i * GW.  prefetch()
    // fetches what the epilogue of the first segment needs at kernel start.
    float pre_bias, pre_out;
    float2 pre_cs;
    uint32_t pos;
    __device__ const uint32_t *pos_ptr() const { return dpos.ptr; }
    __device__ void set_pos(uint32_t fetched) { pos = dpos.ptr ? fetched : dpos.val; }
    __device__ float2 rope_entry(uint32_t row) const {
        if (rope_cs) return rope_cs[((row & ~1u) % head_size) >> 1];
        const float head_dim = (float)((row & ~1u) % head_size);
        const float theta = powf(rope_base, -head_dim / (float)head_size);
        float sn, cs;
        sincosf((float)pos * theta, &sn, &cs);
        return make_float2(cs, sn);
    }
    template <int R>
    __device__ void prefetch(bool late, uint32_t g0, uint32_t GW, uint32_t my_groups, uint32_t lane) {
        if (!late) {
            pre_bias = pre_out = 0.f;
            pre_cs = make_float2(1.f, 0.f);
        }
        if (j.mode == JOB_SILU) return;
        const uint32_t row = 2 * (g0 + (lane >> 1) * GW) + (lane & 1);
        if (!(lane < 2 * my_groups && row < j.nrows)) return;
        // what depends on the position waits for the late call: the output column of a
        // position-strided destination, and RoPE angles when there is no table of them
        const bool out_needs_pos = dpos.ptr && j.out_pos_stride;
        const bool cs_needs_pos = dpos.ptr && !rope_cs;
        if (!late) {
            if (j.bias) pre_bias = j.bias[row];
            if (j.accumulate && !out_needs_pos) pre_out = (j.out + (size_t)dpos.val * j.out_pos_stride)[row];
            if (j.mode == JOB_ROPE && !cs_needs_pos) {
                pos = dpos.val;
                pre_cs = rope_entry(row);
            }
        } else {
            if (j.accumulate && out_needs_pos) pre_out = (j.out + (size_t)pos * j.out_pos_stride)[row];
            if (j.mode == JOB_ROPE && cs_needs_pos) pre_cs = rope_entry(row);
        }
    }
    template <int R>
    __device__ void finish(float mine, uint32_t n, uint32_t g0, uint32_t GW, uint32_t lane) {
        const uint32_t g = g0 + (lane >> 1) * GW, sub = lane & 1;
        const bool valid = lane < n;
        float *out = j.out + (size_t)pos * j.out_pos_stride;
        if (j.mode == JOB_SILU) {
            const float up = dpp_f32<0xB1>(mine);  // the neighbouring lane's value
            if (valid && sub == 0) out[g] = up * (mine / (1.0f + expf(-mine)));
            return;
        }
        const uint32_t row = 2 * g + sub;
        float t = mine + pre_bias;
        if (j.mode == JOB_ROPE) {  // ROPE matrices have an even number of rows
            const float other = dpp_f32<0xB1>(t);
            // (x, y) = (even row, odd row):  x' = cs x - sn y,  y' = sn x + cs y
            t = sub ? pre_cs.y * other + pre_cs.x * t : pre_cs.x * t - pre_cs.y * other;
        }
        if (valid && row < j.nrows) out[row] = j.accumulate ? pre_out + t : t;
    }
};

template <class F, int D>
__device__ __forceinline__ void fused_job_body(const FusedParams &P, const GemvJob &j) {
    GemvParams xp{};
    xp.x = P.x;
    xp.ncols = P.ncols;
    xp.norm_w = P.norm_w;
    xp.norm_eps = P.norm_eps;
    xp.ln_g = P.ln_g;
    xp.ln_b = P.ln_b;
    xp.nrows = j.nrows;
    GemvParams pa = xp, pb = xp;
    pa.p0 = j.a0; pa.p1 = j.a1; pa.p2 = j.a2; pa.p3 = j.a3;
    pb.p0 = j.b0; pb.p1 = j.b1; pb.p2 = j.b2; pb.p3 = j.b3;
    JobPolicy pol{j, pa, pb, P.pos, P.head_size, P.rope_base, P.rope_cs, 0.f, 0.f, make_float2(1.f, 0.f), 0};
    const uint32_t ngroups = j.mode == JOB_SILU ? j.nrows : (j.nrows + 1) / 2;
    if constexpr (!F::F32X) {
        if (P.ncols <= 64 * F::TILE) {
            gemv_i8_body<F, 2, D, true>(xp, pol, blockIdx.x - j.wg_begin, j.wg_count, j.active_waves,
                                        ngroups);
            return;
        }
    }
    gemv_i8_body<F, 2, D, false>(xp, pol, blockIdx.x - j.wg_begin, j.wg_count, j.active_waves, ngroups);
}

// The format struct of a GGUF type: integer-dot (F32 false) or fp32-activation.
template <int TYPE, bool F32> struct FusedFmt;
template <> struct FusedFmt<WGML_Q4_K, false> { using T = IFmtQ4K; };
template <> struct FusedFmt<WGML_Q6_K, false> { using T = IFmtQ6K; };
template <> struct FusedFmt<WGML_Q8_0, false> { using T = IFmtQ8_0; };
template <> struct FusedFmt<WGML_Q4_K, true> { using T = FFmt<FmtQ4K>; };
template <> struct FusedFmt<WGML_Q6_K, true> { using T = FFmt<FmtQ6K>; };
template <> struct FusedFmt<WGML_Q8_0, true> { using T = FFmt<FmtQ8_0>; };
template <> struct FusedFmt<WGML_Q5_K, false> { using T = IFmtQ5K; };
template <> struct FusedFmt<WGML_Q8_K, false> { using T = IFmtQ8K; };
template <> struct FusedFmt<WGML_Q4_0, false> { using T = IFmtQ4_0; };
template <> struct FusedFmt<WGML_Q4_1, false> { using T = IFmtQ4_1; };
template <> struct FusedFmt<WGML_Q5_0, false> { using T = IFmtQ5_0; };
template <> struct FusedFmt<WGML_Q5_1, false> { using T = IFmtQ5_1; };

// MINW: waves per SIMD the register budget must allow.  FMT: 0 = the matrices of
// a launch may differ in format (Q4_K / Q6_K / Q8_0, decided per workgroup), else the one
// format all of them have (smaller code, registers of that format only).  F32: fp32
// activations (the three main formats only).
template <int D, int MAXT, int MINW, int FMT, bool F32 = false>
__global__ __launch_bounds__(MAXT, MINW) void gemv_fused_kernel(const FusedParams P) {
    // All three job records are fetched at once and the workgroup's own is picked field by
    // field afterwards: indexing the kernel arguments with the job number would put a second
    // scalar-memory round trip (a microsecond when the arguments come from HBM) in front of
    // the first weight request.
    const bool is1 = P.njobs > 1 && blockIdx.x >= P.jobs[1].wg_begin;
    const bool is2 = P.njobs > 2 && blockIdx.x >= P.jobs[2].wg_begin;
    const GemvJob &j0 = P.jobs[0], &j1 = P.jobs[1], &j2 = P.jobs[2];
#define WGML_PICK(f) (is2 ? j2.f : (is1 ? j1.f : j0.f))
    const GemvJob j{WGML_PICK(a0), WGML_PICK(a1), WGML_PICK(a2), WGML_PICK(a3),
                    WGML_PICK(b0), WGML_PICK(b1), WGML_PICK(b2), WGML_PICK(b3),
                    WGML_PICK(out), WGML_PICK(bias), WGML_PICK(nrows), WGML_PICK(type),
                    WGML_PICK(mode), WGML_PICK(accumulate), WGML_PICK(out_pos_stride),
                    WGML_PICK(wg_begin), WGML_PICK(wg_count), WGML_PICK(active_waves)};
#undef WGML_PICK
    if constexpr (FMT != 0) {
        fused_job_body<typename FusedFmt<FMT, F32>::T, D>(P, j);
    } else {
        switch (j.type) {
        case WGML_Q4_K: fused_job_body<typename FusedFmt<WGML_Q4_K, F32>::T, D>(P, j); break;
        case WGML_Q6_K: fused_job_body<typename FusedFmt<WGML_Q6_K, F32>::T, D>(P, j); break;
        default: fused_job_body<typename FusedFmt<WGML_Q8_0, F32>::T, D>(P, j); break;
        }
    }
}

// ------------------------------------------------------------- dense f32 ----
// out = A v, A row-major f32 (p.p0).  One wave per row, float4 loads, x from LDS.
__global__ __launch_bounds__(256) void gemv_f32_kernel(const GemvParams p, int vec4) {
    extern __shared__ float4 smem[];
    __shared__ float red[16];
    float *xs = reinterpret_cast<float *>(smem);
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const uint32_t nrows = p.nrows, ncols = p.ncols;
    float rms = 1.f;
    if (p.norm_w) rms = block_rms_scale(p, red);  // needs ncols % 4 == 0 and aligned x
    for (uint32_t i = tid; i < ncols; i += blockDim.x)
        xs[i] = p.norm_w ? (p.x[i] * rms) * p.norm_w[i] : p.x[i];
    __syncthreads();
    const uint32_t row = blockIdx.x * nwaves + wave;
    if (row >= nrows) return;
    const float *ar = reinterpret_cast<const float *>(p.p0) + (size_t)row * ncols;
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
        float *out = p.out;
        if (p.dyn_pos) out += (size_t)(*p.dyn_pos) * p.out_pos_stride;
        float v = total;
        if (p.bias) v += p.bias[row];
        if (p.accumulate) v += out[row];
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

constexpr size_t kMaxLds = 128 * 1024;

// Workgroups of `fn` that fit a CU with `lds` bytes of dynamic LDS (opting in to more than
// 64 KB first); remembered per context and kernel.
int blocks_per_cu(wgml_ctx *ctx, const void *fn, int threads, size_t lds, int *blocks) {
    wgml_kernel_info &ki = ctx->kernel_info[fn];
    if (lds > 64 * 1024 && !ki.opted_in) {
        // gfx950 has 160 KB of LDS per CU; above 64 KB a kernel must opt in once.
        WGML_CHECK_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)kMaxLds));
        ki.opted_in = true;
    }
    if (ki.lds != lds) {
        int nb = 0;
        WGML_CHECK_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, fn, threads, lds));
        ki.blocks_per_cu = nb > 0 ? nb : 1;
        ki.lds = lds;
    }
    *blocks = ki.blocks_per_cu;
    const int cap = ctx->tuning[WGML_TUNE_GEMV_WG_PER_CU];
    if (cap > 0 && cap < *blocks) *blocks = cap;
    return WGML_OK;
}

// Shares `ngroups` row-groups out over at most `max_wgs` workgroups of up to
// `max_waves` waves: every workgroup gets the same count c (the last one the
// remainder), and the fewest waves are active that still give every wave at most
// ceil(c / max_waves) groups, so that the waves of a workgroup finish together.
// A wave parks one result per lane, so it takes at most `max_per_wave` groups (64 results
// divided by the results of a group): very tall matrices get more workgroups than the
// machine holds at once.
struct WgPlan {
    uint32_t groups_per_wg, active_waves, wgs;
};
WgPlan plan_groups(uint32_t ngroups, uint32_t max_wgs, uint32_t max_waves, uint32_t max_per_wave,
                   uint32_t min_c = 1) {
    if (ngroups == 0) return {1, 1, 1};
    if (max_wgs < 1) max_wgs = 1;
    uint32_t c = (ngroups + max_wgs - 1) / max_wgs;
    if (c > max_per_wave * max_waves) c = max_per_wave * max_waves;
    // small matrices: a few groups per workgroup rather than one wave per workgroup
    const uint32_t floor_c = max_waves < 4 ? max_waves : 4;
    if (c < floor_c) c = floor_c;
    if (c < min_c) c = min_c;
    if (c > ngroups) c = ngroups;
    const uint32_t wgs = (ngroups + c - 1) / c;
    c = (ngroups + wgs - 1) / wgs;
    const uint32_t k = (c + max_waves - 1) / max_waves;
    const uint32_t nw = (c + k - 1) / k;
    return {c, nw, wgs};
}

template <class F, int R, int D, int MAXT, int MINW = MAXT / 256, bool XPART = false>
int launch_variant_i8(wgml_ctx *ctx, const GemvParams &p0, size_t lds) {
    int per_cu = 1;
    WGML_TRY(blocks_per_cu(ctx, (const void *)gemv_quant_i8_kernel<F, R, D, MAXT, MINW, XPART>, MAXT,
                           lds, &per_cu));
    const uint32_t cu = ctx->n_cu > 0 ? (uint32_t)ctx->n_cu : 256u;
    // One workgroup per CU with all its waves at work rather than two half-empty ones
    // (each would stage x), as long as that still gives every CU a workgroup (min_c).
    const uint32_t ngroups = (p0.nrows + R - 1) / R;
    uint32_t min_c = (ngroups + cu - 1) / cu;
    if (min_c > MAXT / 64) min_c = MAXT / 64;
    const WgPlan plan = plan_groups(ngroups, cu * (uint32_t)per_cu, MAXT / 64, 64 / R, min_c);
    GemvParams p = p0;
    p.active_waves = plan.active_waves;
    gemv_quant_i8_kernel<F, R, D, MAXT, MINW, XPART><<<dim3(plan.wgs), dim3(MAXT), lds, ctx->stream>>>(p);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

template <class F, int R, int D>
int launch_rd_i8(wgml_ctx *ctx, const GemvParams &p, size_t lds, int waves) {
    switch (waves) {
    case 16: return launch_variant_i8<F, R, D, 1024>(ctx, p, lds);
    case 8: return launch_variant_i8<F, R, D, 512>(ctx, p, lds);
    default: return launch_variant_i8<F, R, D, 256>(ctx, p, lds);
    }
}

// SWEEP: the variants the tuning keys select (rows per wave, waves per workgroup, depth) exist
// for this format; otherwise only the default one.
template <class F, bool SWEEP = true>
int launch_fmt_i8(wgml_ctx *ctx, const GemvParams &p) {
    constexpr int PCH = F::TILE / 16, MF = F::NXB + F::NSUM;
    const uint32_t ntiles = p.ncols / F::TILE;
    const uint32_t ntiles_pad = ((ntiles + 63) / 64) * 64;
    const size_t lds = (size_t)ntiles_pad * 2 * PCH * 16 + (size_t)ntiles_pad * MF * 4;
    if (lds > kMaxLds)
        return set_error(WGML_E_UNSUPPORTED,
                         "gemv_quant: %u columns need %zu bytes of LDS (limit %zu)", p.ncols, lds,
                         kMaxLds);
    // Defaults from a sweep over the Llama-2-7B shapes on MI355X: one row per
    // wave and 16-wave workgroups (x is staged once per 16 rows in flight), and
    // no register ring for Q4_K and Q6_K: a deeper pipeline measured slower at every
    // shape, also with exact waits (11008x4096 Q4_K: 7.7 us at depth 1, 8.1 at 2, 8.8
    // at 3; Q6_K spills from depth 2 on).
    int R = ctx->tuning[WGML_TUNE_GEMV_ROWS_PER_WAVE], waves = ctx->tuning[WGML_TUNE_GEMV_WAVES_PER_WG],
        depth = ctx->tuning[WGML_TUNE_GEMV_DEPTH];
    const bool q8 = F::TILE == 32;
    // (GPT-2 124M's shapes, Q8_0 rows of 768 columns: 16-wave workgroups are as fast as 8-wave
    // ones or faster -- 3072x768 3.3 against 3.6 us, 50257x768 11.1 against 13.4 -- and the
    // tall output projection gains again from two rows per wave, 10.7 us)
    if (!R) R = (q8 && SWEEP && p.ncols <= 1024 && p.nrows >= 16384) ? 2 : 1;
    if (!waves) waves = 16;
    if (waves == 12) waves = 16;  // 12-wave workgroups exist for the fused launches only
    // Q8_0 rows of five and more steps (over 8192 columns): four tiles in flight per wave
    // (4096x11008: 11.0 us against 13.4); everywhere else one tile is as fast or faster
    if (!depth) depth = (q8 && ntiles > 256 && SWEEP) ? 4 : 1;
    if (p.ln_g && (p.ncols >> 2) > 3u * (uint32_t)waves * 64u)  // XP float4 per thread
        return set_error(WGML_E_UNSUPPORTED, "gemv_quant: %u columns are too many for the folded "
                                             "LayerNorm", p.ncols);
    if (p.part_n) {
        // the input is merged from attention partial results: one configuration (16-wave
        // workgroups with room for the partial results in registers)
        if constexpr (SWEEP) return launch_variant_i8<F, 1, 1, 1024, 4, true>(ctx, p, lds);
        return set_error(WGML_E_UNSUPPORTED, "gemv_quant: no merging kernel for this format");
    }
    if constexpr (SWEEP) {
        if (R == 2) {
            if (depth >= 2) return launch_rd_i8<F, 2, 2>(ctx, p, lds, waves);
            return launch_rd_i8<F, 2, 1>(ctx, p, lds, waves);
        }
        if (depth >= 4) return launch_rd_i8<F, 1, 4>(ctx, p, lds, waves);
        if (depth == 3) return launch_rd_i8<F, 1, 3>(ctx, p, lds, waves);
        if (depth == 2) return launch_rd_i8<F, 1, 2>(ctx, p, lds, waves);
        if constexpr (std::is_same_v<F, IFmtQ4K> || std::is_same_v<F, IFmtQ8_0>) {
            // these fit 64 vector registers without spilling: two workgroups per CU
            if (waves == 16) return launch_variant_i8<F, 1, 1, 1024, 8>(ctx, p, lds);
        }
        return launch_rd_i8<F, 1, 1>(ctx, p, lds, waves);
    } else {
        if (p.ln_g && (p.ncols >> 2) > 3u * 1024u)
            return set_error(WGML_E_UNSUPPORTED, "gemv_quant: %u columns are too many for the "
                                                 "folded LayerNorm", p.ncols);
        return launch_variant_i8<F, 1, 1, 1024>(ctx, p, lds);
    }
}

// fp32-activation path: the same body with x staged as floats.  16-wave workgroups, one per
// compute unit (the expansion needs the registers), or 8-wave workgroups with two tiles in flight
// per wave when WGML_TUNE_GEMV_WAVES_PER_WG is 8.
template <class WF>
int launch_fmt_f32(wgml_ctx *ctx, const GemvParams &p) {
    using F = FFmt<WF>;
    const uint32_t ntiles = p.ncols / F::TILE;
    const uint32_t ntiles_pad = ((ntiles + 63) / 64) * 64;
    const size_t lds = (size_t)ntiles_pad * F::CHUNKS * 16 + (size_t)ntiles_pad * F::NSUM * 4;
    if (lds > kMaxLds)
        return set_error(WGML_E_UNSUPPORTED,
                         "gemv_quant: %u columns need %zu bytes of LDS (limit %zu)", p.ncols, lds,
                         kMaxLds);
    if (p.part_n) return launch_variant_i8<F, 1, 1, 1024, 4, true>(ctx, p, lds);
    const int waves = ctx->tuning[WGML_TUNE_GEMV_WAVES_PER_WG];
    if (p.ln_g && (p.ncols >> 2) > 3u * (waves == 8 ? 512u : 1024u))  // XP float4 per thread
        return set_error(WGML_E_UNSUPPORTED, "gemv_quant: %u columns are too many for the folded "
                                             "LayerNorm", p.ncols);
    if (waves == 8) return launch_variant_i8<F, 1, 2, 512, 2>(ctx, p, lds);
    return launch_variant_i8<F, 1, 1, 1024, 4>(ctx, p, lds);
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
        if (lds > kMaxLds)
            return set_error(WGML_E_UNSUPPORTED, "gemv_f32: %u columns exceed the LDS limit", ncols);
        int unused = 0;  // opts in to more than 64 KB of LDS when the row needs it
        WGML_TRY(blocks_per_cu(ctx, (const void *)gemv_f32_kernel, 256, lds, &unused));
        const int vec4 = (ncols % 4 == 0) && ((uintptr_t)a % 16 == 0);
        GemvParams p{};
        p.p0 = reinterpret_cast<const uint8_t *>(a);
        p.x = v;
        p.out = out;
        p.nrows = nrows;
        p.ncols = ncols;
        gemv_f32_kernel<<<dim3((nrows + 3) / 4), dim3(256), lds, ctx->stream>>>(p, vec4);
    }
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

bool gemv_partials_supported(const wgml_ctx *, const wgml_qmat *m) {
    return m && (m->type == WGML_Q4_K || m->type == WGML_Q6_K || m->type == WGML_Q8_0);
}

int launch_gemv_quant(wgml_ctx *ctx, float *out, const wgml_qmat *m, const float *v,
                      const GemvEpilogue &ep) {
    GemvParams p{};
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
    p.dyn_pos = ep.dyn_pos;
    p.out_pos_stride = ep.out_pos_stride;
    p.norm_w = ep.norm_w;
    p.norm_eps = ep.norm_eps;
    p.ln_g = ep.ln_gamma;
    p.ln_b = ep.ln_beta;
    p.act = ep.act;
    const bool main_fmt = m->type == WGML_Q4_K || m->type == WGML_Q6_K || m->type == WGML_Q8_0;
    if (ep.partials.n) {
        const AttnPartials &a = ep.partials;
        if (!gemv_partials_supported(ctx, m) || a.n > 16 || !a.o || !a.ml || a.head_size == 0 ||
            a.head_size % 4 != 0 || a.hsp < a.head_size || a.hsp % 4 != 0 ||
            m->ncols % a.head_size != 0 || m->ncols >= (1u << 20) || a.head_size > 4096 || ep.ln_gamma)
            return set_error(WGML_E_INVALID, "gemv_quant: these attention partial results cannot "
                                             "be merged by this product");
        p.part_o = a.o;
        p.part_ml = a.ml;
        p.part_n = a.n;
        p.part_hsp = a.hsp;
        p.part_hs = a.head_size;
        p.part_hs_inv = (uint32_t)(((uint64_t(1) << 32) + a.head_size - 1) / a.head_size);
        p.x = nullptr;
    } else if ((uintptr_t)v % 16 != 0) {
        return set_error(WGML_E_INVALID, "gemv_quant: the input vector must be 16-byte aligned");
    }
    (void)main_fmt;
    if ((p.ln_g || p.act) && m->type == WGML_F32)
        return set_error(WGML_E_UNSUPPORTED,
                         "gemv_quant: LayerNorm / activation folding needs a quantized matrix");
    if (m->type == WGML_F32) {
        const size_t lds = (size_t)m->ncols * 4;
        if (lds > kMaxLds)
            return set_error(WGML_E_UNSUPPORTED, "gemv_f32: %u columns exceed the LDS limit",
                             m->ncols);
        int unused = 0;  // opts in to more than 64 KB of LDS when the row needs it
        WGML_TRY(blocks_per_cu(ctx, (const void *)gemv_f32_kernel, 256, lds, &unused));
        gemv_f32_kernel<<<dim3((m->nrows + 3) / 4), dim3(256), lds, ctx->stream>>>(p, 1);
        WGML_CHECK_LAUNCH();
        ctx->launches++;
        return WGML_OK;
    }
    switch (m->type) {  // formats that exist as integer-dot kernels only
    case WGML_Q4_0: return launch_fmt_i8<IFmtQ4_0, false>(ctx, p);
    case WGML_Q4_1: return launch_fmt_i8<IFmtQ4_1, false>(ctx, p);
    case WGML_Q5_0: return launch_fmt_i8<IFmtQ5_0, false>(ctx, p);
    case WGML_Q5_1: return launch_fmt_i8<IFmtQ5_1, false>(ctx, p);
    case WGML_Q5_K: return launch_fmt_i8<IFmtQ5K, false>(ctx, p);
    case WGML_Q8_K: return launch_fmt_i8<IFmtQ8K, false>(ctx, p);
    default: break;
    }
    if (!ctx->tuning[WGML_TUNE_GEMV_F32_ACTIVATIONS]) {
        switch (m->type) {
        case WGML_Q4_K: return launch_fmt_i8<IFmtQ4K>(ctx, p);
        case WGML_Q6_K: return launch_fmt_i8<IFmtQ6K>(ctx, p);
        case WGML_Q8_0: return launch_fmt_i8<IFmtQ8_0>(ctx, p);
        default: break;
        }
    }
    switch (m->type) {
    case WGML_Q4_K: return launch_fmt_f32<FmtQ4K>(ctx, p);
    case WGML_Q6_K: return launch_fmt_f32<FmtQ6K>(ctx, p);
    case WGML_Q8_0: return launch_fmt_f32<FmtQ8_0>(ctx, p);
    default: return set_error(WGML_E_UNSUPPORTED, "gemv_quant: unsupported type %d", m->type);
    }
}

// LDS a workgroup of the shared body needs for x: two int8 planes + per-tile scales and sums
// (integer dot), or the floats themselves + per-tile sums (fp32 activations).
template <class F>
static size_t lds_bytes_of(uint32_t ncols) {
    const uint32_t ntiles = ncols / F::TILE;
    const size_t ntiles_pad = ((ntiles + 63) / 64) * 64;
    if (F::F32X) return ntiles_pad * (F::TILE / 4) * 16 + ntiles_pad * F::NSUM * 4;
    return ntiles_pad * 2 * (F::TILE / 16) * 16 + ntiles_pad * (F::NXB + F::NSUM) * 4;
}
static size_t lds_bytes_fused(int type, uint32_t ncols, bool f32) {
    switch (type) {
    case WGML_Q4_K: return f32 ? lds_bytes_of<FFmt<FmtQ4K>>(ncols) : lds_bytes_of<IFmtQ4K>(ncols);
    case WGML_Q6_K: return f32 ? lds_bytes_of<FFmt<FmtQ6K>>(ncols) : lds_bytes_of<IFmtQ6K>(ncols);
    case WGML_Q8_0: return f32 ? lds_bytes_of<FFmt<FmtQ8_0>>(ncols) : lds_bytes_of<IFmtQ8_0>(ncols);
    case WGML_Q5_K: return lds_bytes_of<IFmtQ5K>(ncols);
    case WGML_Q8_K: return lds_bytes_of<IFmtQ8K>(ncols);
    default: return lds_bytes_of<IFmtQ4_0>(ncols);  // the four 32-element block formats
    }
}

static bool main_format(int type) { return type == WGML_Q4_K || type == WGML_Q6_K || type == WGML_Q8_0; }

bool gemv_fused_supported(const wgml_qmat *m) {
    if (!m) return false;
    switch (m->type) {
    case WGML_Q4_K: case WGML_Q6_K: case WGML_Q8_0: case WGML_Q5_K: case WGML_Q8_K: case WGML_Q4_0:
    case WGML_Q4_1: case WGML_Q5_0: case WGML_Q5_1: return true;
    default: return false;
    }
}

// One launch takes matrices of one format (any of the nine), or a mix of Q4_K / Q6_K / Q8_0; with
// fp32 activations only those three.
bool gemv_fused_set_supported(const wgml_ctx *ctx, const wgml_qmat *const *mats, int n) {
    bool same = true, all_main = true;
    for (int i = 0; i < n; ++i) {
        if (!gemv_fused_supported(mats[i])) return false;
        same = same && mats[i]->type == mats[0]->type;
        all_main = all_main && main_format(mats[i]->type);
    }
    if (ctx->tuning[WGML_TUNE_GEMV_F32_ACTIVATIONS]) return all_main;
    return same || all_main;
}

template <int D, int MAXT, int MINW>
static int launch_gemv_fused_variant(wgml_ctx *ctx, const FusedGemv &f, uint32_t *plan_only = nullptr) {
    constexpr uint32_t nwaves = MAXT / 64;
    if (f.njobs < 1 || f.njobs > 3)
        return set_error(WGML_E_INVALID, "gemv_fused: %d jobs", f.njobs);
    if ((uintptr_t)f.x % 16 != 0)
        return set_error(WGML_E_INVALID, "gemv_fused: the input vector must be 16-byte aligned");
    FusedParams P{};
    P.njobs = f.njobs;
    P.x = f.x;
    P.norm_w = f.norm_w;
    P.norm_eps = f.norm_eps;
    P.ln_g = f.ln_gamma;
    P.ln_b = f.ln_beta;
    P.pos = f.pos;
    P.head_size = f.head_size ? f.head_size : 2;
    P.rope_base = f.rope_base;
    P.rope_cs = reinterpret_cast<const float2 *>(f.rope_cs);
    const uint32_t ncols = f.jobs[0].a->ncols;
    P.ncols = ncols;
    const bool f32 = ctx->tuning[WGML_TUNE_GEMV_F32_ACTIVATIONS] != 0;
    size_t lds = 0;
    uint64_t bytes[3] = {0, 0, 0};
    uint32_t ngroups[3];
    for (int i = 0; i < f.njobs; ++i) {
        const FusedGemvJob &s = f.jobs[i];
        if (!gemv_fused_supported(s.a) || s.a->ncols != ncols)
            return set_error(WGML_E_INVALID, "gemv_fused: job %d has an unsupported matrix", i);
        if (f32 && !main_format(s.a->type))
            return set_error(WGML_E_UNSUPPORTED, "gemv_fused: fp32 activations exist for Q4_K, Q6_K "
                                                 "and Q8_0 only");
        GemvJob &j = P.jobs[i];
        j.a0 = s.a->p0; j.a1 = s.a->p1; j.a2 = s.a->p2; j.a3 = s.a->p3;
        j.out = s.out;
        j.bias = s.bias;
        j.nrows = s.a->nrows;
        if (s.row0 || s.nrows) {  // a slice of the rows: move the plane pointers to its first row
            const uint32_t n = s.nrows ? s.nrows : s.a->nrows - s.row0;
            if (s.mode == JOB_SILU || (uint64_t)s.row0 + n > s.a->nrows)
                return set_error(WGML_E_INVALID, "gemv_fused: job %d: bad row slice", i);
            const uint64_t r = s.row0, nb = r * (ncols / 256), nb32 = r * (ncols / 32);
            switch (s.a->type) {
            case WGML_Q4_K: j.a0 += nb * 144; break;
            case WGML_Q5_K: j.a0 += nb * 176; break;
            case WGML_Q8_K: j.a0 += nb * 292; break;
            case WGML_Q6_K: j.a0 += nb * 128; j.a1 += nb * 64; j.a2 += nb * 16; j.a3 += nb * 2; break;
            case WGML_Q8_0: j.a0 += r * ncols; j.a1 += nb32 * 2; break;
            case WGML_Q4_0: j.a0 += nb32 * 18; break;
            case WGML_Q4_1: j.a0 += nb32 * 20; break;
            case WGML_Q5_0: j.a0 += nb32 * 22; break;
            default: j.a0 += nb32 * 24; break;  // Q5_1
            }
            j.nrows = n;
        }
        j.type = s.a->type;
        j.mode = s.mode;
        j.accumulate = s.accumulate;
        j.out_pos_stride = s.out_pos_stride;
        bytes[i] = s.a->gguf_bytes / s.a->nrows * j.nrows;
        if (s.mode == JOB_SILU) {
            if (!s.b || s.b->type != s.a->type || s.b->nrows != s.a->nrows || s.b->ncols != ncols)
                return set_error(WGML_E_INVALID, "gemv_fused: job %d: gate/up matrices differ", i);
            j.b0 = s.b->p0; j.b1 = s.b->p1; j.b2 = s.b->p2; j.b3 = s.b->p3;
            bytes[i] += s.b->gguf_bytes;
            ngroups[i] = j.nrows;
        } else {
            if (s.mode == JOB_ROPE && (j.nrows % 2 != 0 || P.head_size % 2 != 0))
                return set_error(WGML_E_INVALID, "gemv_fused: RoPE needs even row counts");
            ngroups[i] = (j.nrows + 1) / 2;
        }
        const size_t l = lds_bytes_fused(j.type, ncols, f32);
        if (l > lds) lds = l;
    }
    if (lds > kMaxLds)
        return set_error(WGML_E_UNSUPPORTED, "gemv_fused: %u columns need %zu bytes of LDS", ncols,
                         lds);
    if (P.ln_g && (ncols >> 2) > 3u * (uint32_t)MAXT)  // XP float4 per thread
        return set_error(WGML_E_UNSUPPORTED,
                         "gemv_fused: %u columns are too many for the folded LayerNorm", ncols);
    // one kernel per format when all matrices share it, else the mixed one
    int fmt = P.jobs[0].type, slot = 0;
    for (int i = 1; i < f.njobs; ++i)
        if (P.jobs[i].type != fmt) fmt = 0;
    if (fmt == 0)
        for (int i = 0; i < f.njobs; ++i)
            if (!main_format(P.jobs[i].type))
                return set_error(WGML_E_UNSUPPORTED, "gemv_fused: formats can be mixed among Q4_K, "
                                                     "Q6_K and Q8_0 only");
    // the mixed-format kernel is held to 96 registers (5 waves per SIMD): it fits without
    // spilling, and the waves of a workgroup start sooner the fewer registers they take
    void (*kern)(const FusedParams) = gemv_fused_kernel<D, MAXT, (MAXT == 1024 ? 5 : MINW), 0>;
    (void)slot;
    if (f32) {
        kern = gemv_fused_kernel<D, MAXT, MINW, 0, true>;
        switch (fmt) {
        case WGML_Q4_K: kern = gemv_fused_kernel<D, MAXT, MINW, WGML_Q4_K, true>; break;
        case WGML_Q6_K: kern = gemv_fused_kernel<D, MAXT, MINW, WGML_Q6_K, true>; break;
        case WGML_Q8_0: kern = gemv_fused_kernel<D, MAXT, MINW, WGML_Q8_0, true>; break;
        default: break;
        }
    } else {
        switch (fmt) {
        case WGML_Q4_K: kern = gemv_fused_kernel<D, MAXT, MINW, WGML_Q4_K>; break;
        case WGML_Q6_K: kern = gemv_fused_kernel<D, MAXT, MINW, WGML_Q6_K>; break;
        case WGML_Q8_0: kern = gemv_fused_kernel<D, MAXT, MINW, WGML_Q8_0>; break;
        case WGML_Q5_K: kern = gemv_fused_kernel<D, MAXT, MINW, WGML_Q5_K>; break;
        case WGML_Q8_K: kern = gemv_fused_kernel<D, MAXT, MINW, WGML_Q8_K>; break;
        case WGML_Q4_0: kern = gemv_fused_kernel<D, MAXT, MINW, WGML_Q4_0>; break;
        case WGML_Q4_1: kern = gemv_fused_kernel<D, MAXT, MINW, WGML_Q4_1>; break;
        case WGML_Q5_0: kern = gemv_fused_kernel<D, MAXT, MINW, WGML_Q5_0>; break;
        case WGML_Q5_1: kern = gemv_fused_kernel<D, MAXT, MINW, WGML_Q5_1>; break;
        default: break;
        }
    }
    int cached_blocks = 1;
    WGML_TRY(blocks_per_cu(ctx, (const void *)kern, MAXT, lds, &cached_blocks));
    const uint32_t cu = ctx->n_cu > 0 ? (uint32_t)ctx->n_cu : 256u;
    const uint32_t resident = cu * (uint32_t)cached_blocks;
    // Every workgroup streams about the same number of bytes: the smallest per-
    // workgroup budget T is searched for which the matrices together need no more
    // workgroups than the machine holds at once.
    double bpg[3], lo = 0.0, hi = 0.0;
    for (int i = 0; i < f.njobs; ++i) {
        bpg[i] = (double)bytes[i] / (double)ngroups[i];
        hi += (double)bytes[i];
    }
    auto wgs_needed = [&](double T) {
        uint64_t n = 0;
        for (int i = 0; i < f.njobs; ++i) {
            uint64_t c = (uint64_t)(T / bpg[i]);
            if (c < 1) c = 1;
            n += (ngroups[i] + c - 1) / c;
        }
        return n;
    };
    for (int it = 0; it < 50; ++it) {
        const double mid = 0.5 * (lo + hi);
        if (wgs_needed(mid) <= resident) hi = mid; else lo = mid;
    }
    uint32_t begin = 0, max_nw = 1;
    for (int i = 0; i < f.njobs; ++i) {
        uint32_t c = (uint32_t)(hi / bpg[i]);
        if (c < 1) c = 1;
        const WgPlan plan = plan_groups(ngroups[i], (ngroups[i] + c - 1) / c, nwaves, 32);
        P.jobs[i].wg_begin = begin;
        P.jobs[i].wg_count = plan.wgs;
        P.jobs[i].active_waves = plan.active_waves;
        if (plan.active_waves > max_nw) max_nw = plan.active_waves;
        begin += plan.wgs;
    }
    if (plan_only) {  // the caller only asks how many row pairs the launch has
        *plan_only = 0;
        for (int i = 0; i < f.njobs; ++i) *plan_only += ngroups[i];
        return WGML_OK;
    }
    kern<<<dim3(begin), dim3(MAXT), lds, ctx->stream>>>(P);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int launch_gemv_fused(wgml_ctx *ctx, const FusedGemv &f) {
    const int depth = ctx->tuning[WGML_TUNE_GEMV_DEPTH], waves = ctx->tuning[WGML_TUNE_GEMV_WAVES_PER_WG];
    (void)depth;  // deeper register rings spill in the fused kernels
    if (waves == 12) return launch_gemv_fused_variant<1, 768, 1>(ctx, f);
    if (waves == 16) return launch_gemv_fused_variant<1, 1024, 1>(ctx, f);
    // 12-wave workgroups for launches with a little less than one row pair per wave of a
    // machine full of 16-wave workgroups (Q/K/V of 4096/1024/1024 rows: 8.6 us against 9.6;
    // small launches are better off with the 16-wave kernel: GPT-2's Q/K/V 5.1 us against 7.1)
    uint32_t pairs = 0;
    WGML_TRY((launch_gemv_fused_variant<1, 1024, 1>(ctx, f, &pairs)));
    const uint32_t cu = ctx->n_cu > 0 ? (uint32_t)ctx->n_cu : 256u;
    if (pairs > cu * 8 && pairs <= cu * 16) return launch_gemv_fused_variant<1, 768, 1>(ctx, f);
    return launch_gemv_fused_variant<1, 1024, 1>(ctx, f);
}

}  // namespace wgml

extern "C" {

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
