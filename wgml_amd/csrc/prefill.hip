// Batched prompt processing ("prefill"): the decoder's matrix products for up to 128
// tokens at once, as a GEMM on the matrix cores.  The reference has no such path -- it
// pushes the prompt through its batch-1 step one token at a time
// (wgml-chat/src/chat_llama2.rs:155-228 with the forced-token rule of
// wgml-chat/src/sampler.rs:102-107) -- so this is new functionality whose results are
// held against exactly that: N sequential decode steps.
//
//   out[t][r] = sum_k W[r][k] * X[t][k]      W: Q4_K / Q6_K / Q8_0 as stored for the GEMV
//
// Weights are expanded in registers with the reference's dequantization arithmetic (fp32),
// activations are scaled per token by a power of two so that they stay in f16 range, products
// accumulate in fp32 on v_mfma_f32_16x16x32_f16.  Two precisions:
//   split f16 (default)  each operand is a pair of f16 numbers, hi = f16(v) and
//                        lo = f16(v - hi); the product is W_hi X_hi + W_hi X_lo + W_lo X_hi, three
//                        MFMAs per term group into one fp32 accumulator, results to fp32 rounding
//                        (about 1e-6 of a row's magnitude).  The low parts are small: weights are
//                        expanded times 2^8 and activations scaled to 512 < max |x| <= 1024 so that
//                        they stay clear of the bottom of the f16 range (the matrix cores take
//                        subnormal f16 inputs as they are, so what falls below loses precision
//                        gradually, not all at once);
//   plain f16            both operands rounded to f16 once, one MFMA: about 3e-4 of a row's RMS.
//
// Tiling.  A workgroup (8 waves) owns 64 rows of one matrix -- four blocks of 16 -- and
// a contiguous range of K, walked in iterations of two 64-element chunks.  Per iteration
// the workgroup stages both chunks of the activations (all tokens) in LDS; waves 0-3
// multiply the first chunk with their row block's weights, waves 4-7 the second, so an
// activation word fetched from L2 serves 64 rows and every weight element is expanded
// exactly once, by one wave, for all NT blocks of 16 tokens (NT accumulators of 16x16 per
// wave).  Two LDS buffers: the next pair of chunks is on its way from memory while the
// current one is multiplied, one barrier per iteration.  At the end waves 4-7 hand
// their sums to waves 0-3 through LDS.  (K is padded to a whole number of pairs of chunks.)
//
// On this machine a SIMD does not overlap the vector instructions of one wave with the MFMAs
// of another to any useful degree (measured: two MFMA-then-VALU waves per SIMD take the sum of
// both parts), and the two waves of a SIMD run in step between barriers.  So the overlap is
// made inside each wave: while it issues the MFMAs of iteration it, it expands the weights of
// iteration it + 1 (fetched during iteration it - 1), a few vector instructions after every
// MFMA, and it requests its LDS words two steps ahead.  The expansion is written for few
// instructions: bytes masked four at a time and converted with the byte-to-float
// instructions, one multiply-add per element, one packed conversion per pair for the high
// parts, one mixed-precision multiply-add per element for the low parts, lane offsets of 32
// bits on uniform bases for every load.
//
// One launch can cover up to three matrices that multiply the same activations (Q, K
// and V; gate and up): their row tiles are numbered side by side.  A matrix too short to
// give every compute unit a tile has its K range split between ks workgroups; they leave
// partial sums that gemm_reduce_kernel adds in a fixed order (or, for a plain `x += W h`,
// the prep_x_kernel that reads x next).  Workgroup w takes part w % ks of tile w / ks: the
// eight XCDs are handed workgroups in turn, so each sees 1 / ks of the activations only.
//
// Activations are stored in the order the B operand wants them (written by
// prep_x_kernel): for chunk c, token block n, half s2 of the chunk, lane (g, j) finds
// the 8 halves  X[16 n + j][64 c + 32 s2 + 8 g .. + 7]  as one 16-byte word at
// word index ((c * NT + n) * 2 + s2) * 64 + 16 g + j: a chunk is NT KiB contiguous.
// That word is the B operand of one 16x16x32 MFMA (lane (g, j) supplies k = 8 g .. 8 g + 7
// of the 32 for token j); the A operand follows the same assignment of k to lanes.
#include <hip/hip_fp16.h>

#include <type_traits>

#include "common.h"
#include "device_utils.h"

using namespace wgml;

namespace {

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // plain vector: arrays of it stay in registers

constexpr uint32_t KC = 64;    // elements of K per chunk
constexpr uint32_t KWAVES = 8;  // waves of a workgroup: 4 row blocks x 2 chunks per iteration

struct GemmMat {
    const uint8_t *p0, *p1, *p2, *p3;  // matrix planes (as wgml_qmat)
    float *out;                        // [T][out_stride]
    const float *bias;                 // optional, per row
    uint32_t nrows, out_stride;
    uint32_t tile0;                    // first 64-row tile of this matrix in grid.x
    uint32_t roff;                     // rows of the matrices before this one in the launch
    uint32_t rope;                     // the reduction rotates this matrix' rows (GemmArgs::rope_*)
};

struct GemmArgs {
    GemmMat m[3];
    uint32_t nmat;
    const u32x4 *xh;                   // packed f16 activations (see above)
    const u32x4 *xl;                   // their low parts in the same order (split precision only)
    uint32_t xl_offset;                // bytes from xh to xl
    const float *xscale;               // [tpad] factor to multiply a token's results with
    uint32_t ncols, kpad, T, tpad;
    int accumulate;                    // out += result
    float *part;                       // [ks][T][total_rows] partial sums (ks > 1)
    uint32_t ks;                       // ways K is split between workgroups (grid.y)
    uint32_t total_rows;               // rows of all matrices of the launch
    int defer;                         // ks > 1: leave the partial sums to the next kernel
    // rotary encoding applied by gemm_reduce_rope_kernel to the matrices marked `rope`
    uint32_t rope_head_size, rope_pos0;
    float rope_base;
    int rope_neox;
};

__device__ __forceinline__ half4 to_half4(float a, float b, float c, float d) {
    half4 h;
    h[0] = (_Float16)a;
    h[1] = (_Float16)b;
    h[2] = (_Float16)c;
    h[3] = (_Float16)d;
    return h;
}

// Weights are expanded times 2^8 (an exact scaling, undone with the activations' factor at the
// end): a low part f16(w - hi) of a typical weight (0.01 .. 0.1) is then a normal f16 number.
// Weights beyond 65504 / 2^8 = 255.875 would overflow f16: launch_gemm_quant_multi refuses a
// matrix whose bound (wgml_qmat::max_abs) exceeds that.
constexpr float kWeightScale = 256.f;

// The value as the compiler must take it: what follows is not merged with what computed it.
__device__ __forceinline__ uint32_t opaque(uint32_t v) {
    asm("" : "+v"(v));
    return v;
}

// A load from uniform base + 32-bit lane offset.  The empty asm keeps the offset a 32-bit VGPR
// at the point of use, so that the load takes the base from scalar registers and the offset as
// it is: no 64-bit address arithmetic per lane and iteration.
template <class T>
__device__ __forceinline__ T load_at(const uint8_t *uniform_base, uint32_t lane_offset) {
    asm volatile("" : "+v"(lane_offset));
    return *reinterpret_cast<const T *>(uniform_base + lane_offset);
}

// ---- weight fragments -----------------------------------------------------------
// Lane (g, j) of a wave holds, for chunk c of row j of the tile, the 16 elements
//     k = 64 c + 32 s2 + 8 g + 4 e + i        (s2, e in 0..1, i in 0..3)
// lane_init() computes the lane's byte offsets into the matrix planes once (matrices are below
// 4 GiB), load() fetches the bytes, pre() decodes what the 16 share (scales), elem<I>() computes
// element I = 4 (2 s2 + e) + i as the reference's dequantize does (quantization.rs:29-42,
// 204-244, 322-389), in fp32 (a fused multiply-add where the reference multiplies and subtracts:
// one rounding less).  They reach the matrix cores either rounded to f16 or as a pair of f16
// numbers whose sum is the fp32 value to about 2^-21 (hi = f16(w), lo = f16(w - hi)), all times 2^8.
// The element-wise interface lets the kernel spread the expansion between its MFMAs.
struct GemmQ4K {
    struct Raw {
        uint4 hdr;  // d, dmin, 12 bytes of packed scales
        uint2 qs;   // bytes 8 g .. 8 g + 7 of the chunk's 32: low nibbles s2 = 0, high s2 = 1
    };
    struct Pre {
        float dd[2], mm[2];  // per s2: d * scale, dmin * min
    };
    struct Lane {
        uint32_t hdr, qs;
    };
    __device__ static void lane_init(Lane &l, uint32_t ncols, uint32_t row, uint32_t g) {
        l.hdr = row * (ncols / 256) * 144;
        l.qs = l.hdr + 16 + 8 * g;
    }
    __device__ static void load(Raw &r, const GemmMat &m, uint32_t, const Lane &l, uint32_t chunk) {
        const uint8_t *blk = m.p0 + (size_t)(chunk >> 2) * 144;
        r.hdr = load_at<uint4>(blk, l.hdr);
        r.qs = load_at<uint2>(blk + (chunk & 3) * 32, l.qs);
    }
    __device__ static void pre(Pre &p, const Raw &r, uint32_t, uint32_t chunk, uint32_t) {
        const uint4 hdr = r.hdr;
        const uint32_t j = chunk & 3;
        const float d = f16_bits_to_f32((uint16_t)(hdr.x & 0xffffu)) * kWeightScale;
        const float dmin = f16_bits_to_f32((uint16_t)(hdr.x >> 16)) * kWeightScale;
        // get_scale_min_k4 for sub-blocks 2j and 2j + 1, on the three words of packed scales
        // (no byte array: the index is not a compile-time constant)
        uint32_t s1, m1, s2, m2;
        if (j < 2) {
            const uint32_t sh = 16 * j;
            s1 = (hdr.y >> sh) & 63u;
            m1 = (hdr.z >> sh) & 63u;
            s2 = (hdr.y >> (sh + 8)) & 63u;
            m2 = (hdr.z >> (sh + 8)) & 63u;
        } else {
            const uint32_t sh = 16 * (j - 2);
            s1 = ((hdr.w >> sh) & 15u) | (((hdr.y >> (sh + 6)) & 3u) << 4);
            m1 = ((hdr.w >> (sh + 4)) & 15u) | (((hdr.z >> (sh + 6)) & 3u) << 4);
            s2 = ((hdr.w >> (sh + 8)) & 15u) | (((hdr.y >> (sh + 14)) & 3u) << 4);
            m2 = ((hdr.w >> (sh + 12)) & 15u) | (((hdr.z >> (sh + 14)) & 3u) << 4);
        }
        p.dd[0] = d * (float)s1;
        p.mm[0] = dmin * (float)m1;
        p.dd[1] = d * (float)s2;
        p.mm[1] = dmin * (float)m2;
    }
    template <int I>
    __device__ static float elem(const Pre &p, const Raw &r, uint32_t) {
        constexpr int s2 = I / 8, e = (I / 4) & 1, b = I & 3;
        // the four nibbles of a word are masked at once; each is then one byte-to-float conversion
        const uint32_t four = opaque(((e ? r.qs.y : r.qs.x) >> (4 * s2)) & 0x0f0f0f0fu);
        return fmaf(p.dd[s2], (float)((four >> (8 * b)) & 0xffu), -p.mm[s2]);
    }
};

struct GemmQ6K {
    struct Raw {
        uint2 ql[2];  // per s2: 8 bytes of low nibbles
        uint2 qh;     // 8 bytes of high bit pairs
        uint32_t scw;  // the four scales of this 64-element chunk
        uint32_t d;
    };
    struct Pre {
        float ds[2], off[2];  // per s2: d * scale, -32 d * scale
        uint32_t hi_nib;      // odd chunks take the high nibbles
    };
    struct Lane {
        uint32_t ql, qh, sc, d;
    };
    __device__ static void lane_init(Lane &l, uint32_t ncols, uint32_t row, uint32_t g) {
        const uint32_t blk = row * (ncols / 256);
        l.ql = blk * 128 + 8 * g;
        l.qh = blk * 64 + 8 * g;
        l.sc = blk * 16;
        l.d = blk * 2;
    }
    __device__ static void load(Raw &r, const GemmMat &m, uint32_t, const Lane &l, uint32_t chunk) {
        const size_t blk = chunk >> 2;
        const uint32_t c = chunk & 3, i = c >> 1;
        const uint8_t *ql = m.p0 + blk * 128 + 64 * i;
        r.ql[0] = load_at<uint2>(ql, l.ql);
        r.ql[1] = load_at<uint2>(ql + 32, l.ql);
        r.qh = load_at<uint2>(m.p1 + blk * 64 + 32 * i, l.qh);
        r.scw = load_at<uint32_t>(m.p2 + blk * 16 + 8 * i + 4 * (c & 1), l.sc);
        r.d = load_at<uint16_t>(m.p3 + blk * 2, l.d);
    }
    // element e = 64 (c & 1) + 32 s2 + 8 g + b of the 128-element half: quarter
    // e / 32 = 2 (c & 1) + s2 picks the nibble (high for quarters 2, 3), the bit pair of
    // qh[8 g + b] (shift 2 * quarter) and the scale (8 g + b) / 16 + 2 * quarter
    __device__ static void pre(Pre &p, const Raw &r, uint32_t, uint32_t chunk, uint32_t g) {
        const float d = f16_bits_to_f32((uint16_t)r.d) * kWeightScale;
        p.hi_nib = chunk & 1;
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            p.ds[s2] = d * (float)(int8_t)((r.scw >> (8 * ((g >> 1) + 2 * s2))) & 0xffu);
            p.off[s2] = -32.f * p.ds[s2];
        }
    }
    template <int I>
    __device__ static float elem(const Pre &p, const Raw &r, uint32_t) {
        constexpr int s2 = I / 8, e = (I / 4) & 1, b = I & 3;
        // the four 6-bit values of a word pair are put together at once (bytes 0 .. 63), each is
        // then one byte-to-float conversion; (q - 32) ds as one multiply-add with -32 ds
        const uint32_t l = ((e ? r.ql[s2].y : r.ql[s2].x) >> (4 * p.hi_nib)) & 0x0f0f0f0fu;
        const uint32_t h = ((e ? r.qh.y : r.qh.x) >> (2 * (2 * p.hi_nib + s2))) & 0x03030303u;
        const uint32_t four = opaque(l | (h << 4));
        return fmaf(p.ds[s2], (float)((four >> (8 * b)) & 0xffu), p.off[s2]);
    }
};

struct GemmQ8_0 {
    struct Raw {
        uint2 q[2];  // per s2 (= 32-element block of the chunk): 8 quants
        uint32_t d[2];
    };
    struct Pre {
        float d[2], off[2];  // per s2: d, -128 d
    };
    struct Lane {
        uint32_t q, d;
    };
    __device__ static void lane_init(Lane &l, uint32_t ncols, uint32_t row, uint32_t g) {
        l.q = row * ncols + 8 * g;
        l.d = row * (ncols / 32) * 2;
    }
    // rows are a multiple of 32 elements long: a 32-element block of the (padded) K range may
    // not exist; the last one is then read in its place and expanded to zeros
    __device__ static void load(Raw &r, const GemmMat &m, uint32_t ncols, const Lane &l, uint32_t chunk) {
        const uint32_t b0 = chunk * 2, nb = ncols / 32;
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            const uint32_t b = min(b0 + s2, nb - 1);
            r.q[s2] = load_at<uint2>(m.p0 + (size_t)b * 32, l.q);
            r.d[s2] = load_at<uint16_t>(m.p1 + (size_t)b * 2, l.d);
        }
    }
    __device__ static void pre(Pre &p, const Raw &r, uint32_t ncols, uint32_t chunk, uint32_t) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            p.d[s2] = chunk * 2 + s2 < ncols / 32 ? f16_bits_to_f32((uint16_t)r.d[s2]) * kWeightScale : 0.f;
            p.off[s2] = -128.f * p.d[s2];
        }
    }
    template <int I>
    __device__ static float elem(const Pre &p, const Raw &r, uint32_t) {
        constexpr int s2 = I / 8, e = (I / 4) & 1, b = I & 3;
        // signed bytes with the top bit flipped are q + 128 as unsigned bytes: one byte-to-float
        // conversion each, the 128 taken off by the multiply-add (exact: |q d| needs 8 + 11 bits)
        const uint32_t four = opaque((e ? r.q[s2].y : r.q[s2].x) ^ 0x80808080u);
        return fmaf(p.d[s2], (float)((four >> (8 * b)) & 0xffu), p.off[s2]);
    }
};

// Q5_K (176 B: d, dmin, scales[12] as Q4_K, 32 bytes of fifth bits, 128 bytes of nibbles;
// quantization.rs:249-317).  Chunk c is the 64-element group j = c & 3 of super-block c >> 2:
// sub-block 2 j + s2 takes the low (s2 = 0) or high nibbles of qs[32 j + l] and bit 2 j + s2 of
// qh[l], l = 8 g + 4 e + i.
struct GemmQ5K {
    struct Raw {
        uint4 hdr;
        uint2 qs, qh;
    };
    struct Pre {
        float dd[2], mm[2];
        uint32_t j2;  // 2 j
    };
    struct Lane {
        uint32_t hdr, qs, qh;
    };
    __device__ static void lane_init(Lane &l, uint32_t ncols, uint32_t row, uint32_t g) {
        l.hdr = row * (ncols / 256) * 176;
        l.qh = l.hdr + 16 + 8 * g;
        l.qs = l.hdr + 48 + 8 * g;
    }
    __device__ static void load(Raw &r, const GemmMat &m, uint32_t, const Lane &l, uint32_t chunk) {
        const uint8_t *blk = m.p0 + (size_t)(chunk >> 2) * 176;
        r.hdr = load_at<uint4>(blk, l.hdr);
        r.qh = load_at<uint2>(blk, l.qh);
        r.qs = load_at<uint2>(blk + (chunk & 3) * 32, l.qs);
    }
    __device__ static void pre(Pre &p, const Raw &r, uint32_t ncols, uint32_t chunk, uint32_t g) {
        GemmQ4K::Raw q4;
        q4.hdr = r.hdr;
        q4.qs = r.qs;
        GemmQ4K::Pre p4;
        GemmQ4K::pre(p4, q4, ncols, chunk, g);  // the scale / min layout is Q4_K's
        p.dd[0] = p4.dd[0];
        p.dd[1] = p4.dd[1];
        p.mm[0] = p4.mm[0];
        p.mm[1] = p4.mm[1];
        p.j2 = 2 * (chunk & 3);
    }
    template <int I>
    __device__ static float elem(const Pre &p, const Raw &r, uint32_t) {
        constexpr int s2 = I / 8, e = (I / 4) & 1, b = I & 3;
        const uint32_t lo = ((e ? r.qs.y : r.qs.x) >> (4 * s2)) & 0x0f0f0f0fu;
        const uint32_t hb = (((e ? r.qh.y : r.qh.x) >> (p.j2 + s2)) & 0x01010101u) << 4;
        const uint32_t four = opaque(lo | hb);
        return fmaf(p.dd[s2], (float)((four >> (8 * b)) & 0xffu), -p.mm[s2]);
    }
};

// Q8_K (292 B: f32 d, 256 int8, 16 sums that dequantization does not use; quantization.rs:170-199).
struct GemmQ8K {
    struct Raw {
        uint2 q[2];
        float d;
    };
    struct Pre {
        float d, off;
    };
    struct Lane {
        uint32_t d, q;
    };
    __device__ static void lane_init(Lane &l, uint32_t ncols, uint32_t row, uint32_t g) {
        l.d = row * (ncols / 256) * 292;
        l.q = l.d + 4 + 8 * g;
    }
    __device__ static void load(Raw &r, const GemmMat &m, uint32_t, const Lane &l, uint32_t chunk) {
        const uint8_t *blk = m.p0 + (size_t)(chunk >> 2) * 292;
        r.d = load_at<float>(blk, l.d);
        r.q[0] = load_at<uint2>(blk + (chunk & 3) * 64, l.q);
        r.q[1] = load_at<uint2>(blk + (chunk & 3) * 64 + 32, l.q);
    }
    __device__ static void pre(Pre &p, const Raw &r, uint32_t, uint32_t, uint32_t) {
        p.d = r.d * kWeightScale;
        p.off = -128.f * p.d;
    }
    template <int I>
    __device__ static float elem(const Pre &p, const Raw &r, uint32_t) {
        constexpr int s2 = I / 8, e = (I / 4) & 1, b = I & 3;
        const uint32_t four = opaque((e ? r.q[s2].y : r.q[s2].x) ^ 0x80808080u);  // q + 128 as bytes
        return fmaf(p.d, (float)((four >> (8 * b)) & 0xffu), p.off);
    }
};

// The 32-element blocks Q4_0 (18 B: d, 16 B of nibbles), Q4_1 (20 B: d, m, nibbles), Q5_0 (22 B:
// d, 32 fifth bits, nibbles), Q5_1 (24 B: d, m, fifth bits, nibbles); quantization.rs:47-162.
// Element t of a block is the low nibble of qs[t] for t < 16 and the high nibble of qs[t - 16]
// otherwise, with bit t of qh as its fifth bit.  Chunk c holds blocks 2 c (s2 = 0) and 2 c + 1;
// a lane's t = 8 g + 4 e + i, so lanes g < 2 take low nibbles and g >= 2 high nibbles of the
// same eight bytes.  Blocks are 2-byte aligned: the loads below are unaligned, which gfx950
// serves.  A block of the padded K range that does not exist reads the last one and expands to 0.
template <int BYTES, bool HAS_M, bool HAS_QH>
struct GemmLegacy {
    struct Raw {
        uint2 q[2];
        uint32_t qh[2];
        uint32_t dm[2];  // d (low half) and m (high half) as stored
    };
    struct Pre {
        float d[2], off[2];
        uint32_t hi_nib, shift;  // g >= 2; bit of qh that belongs to this lane's first element
    };
    struct Lane {
        uint32_t blk, q;
    };
    static constexpr uint32_t QS = 2 + (HAS_M ? 2 : 0) + (HAS_QH ? 4 : 0);
    __device__ static void lane_init(Lane &l, uint32_t ncols, uint32_t row, uint32_t g) {
        l.blk = row * (ncols / 32) * BYTES;
        l.q = l.blk + QS + 8 * (g & 1);
    }
    __device__ static void load(Raw &r, const GemmMat &m, uint32_t ncols, const Lane &l, uint32_t chunk) {
        const uint32_t b0 = chunk * 2, nb = ncols / 32;
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            const uint8_t *blk = m.p0 + (size_t)min(b0 + s2, nb - 1) * BYTES;
            // 2-byte aligned: halfwords are loaded as such and put together
            const uint32_t d = load_at<uint16_t>(blk, l.blk);
            uint32_t mm = 0;
            if (HAS_M) mm = load_at<uint16_t>(blk + 2, l.blk);
            r.dm[s2] = d | (mm << 16);
            r.qh[s2] = 0;
            if (HAS_QH)
                r.qh[s2] = (uint32_t)load_at<uint16_t>(blk + (HAS_M ? 4 : 2), l.blk) |
                           ((uint32_t)load_at<uint16_t>(blk + (HAS_M ? 6 : 4), l.blk) << 16);
            const uint32_t q0 = (uint32_t)load_at<uint16_t>(blk, l.q) | ((uint32_t)load_at<uint16_t>(blk + 2, l.q) << 16);
            const uint32_t q1 = (uint32_t)load_at<uint16_t>(blk + 4, l.q) | ((uint32_t)load_at<uint16_t>(blk + 6, l.q) << 16);
            r.q[s2] = make_uint2(q0, q1);
        }
    }
    __device__ static void pre(Pre &p, const Raw &r, uint32_t ncols, uint32_t chunk, uint32_t g) {
        p.hi_nib = g >> 1;
        p.shift = 8 * g;
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            const bool exists = chunk * 2 + s2 < ncols / 32;
            const float d = exists ? f16_bits_to_f32((uint16_t)(r.dm[s2] & 0xffffu)) * kWeightScale : 0.f;
            p.d[s2] = d;
            if (HAS_M)  // y = d q + m
                p.off[s2] = exists ? f16_bits_to_f32((uint16_t)(r.dm[s2] >> 16)) * kWeightScale : 0.f;
            else  // y = d (q - 8) or d (q - 16)
                p.off[s2] = (HAS_QH ? -16.f : -8.f) * d;
        }
    }
    template <int I>
    __device__ static float elem(const Pre &p, const Raw &r, uint32_t) {
        constexpr int s2 = I / 8, e = (I / 4) & 1, b = I & 3;
        uint32_t four = ((e ? r.q[s2].y : r.q[s2].x) >> (4 * p.hi_nib)) & 0x0f0f0f0fu;
        if (HAS_QH) {
            // bits t .. t + 3 of qh (t = 8 g + 4 e) moved to bit 4 of bytes 0 .. 3
            const uint32_t bits = (r.qh[s2] >> (p.shift + 4 * e)) & 15u;
            four |= ((bits * 0x00204081u) & 0x01010101u) << 4;
        }
        four = opaque(four);
        return fmaf(p.d[s2], (float)((four >> (8 * b)) & 0xffu), p.off[s2]);
    }
};
using GemmQ4_0 = GemmLegacy<18, false, false>;
using GemmQ4_1 = GemmLegacy<20, true, false>;
using GemmQ5_0 = GemmLegacy<22, false, true>;
using GemmQ5_1 = GemmLegacy<24, true, true>;

// A wave's weights for one chunk as MFMA A operands: hi[s2] (and, split precision, lo[s2]).
template <bool SPLIT>
struct AFrag {
    half2v hi[2][4];
    half2v lo[SPLIT ? 2 : 1][4];
};

// Elements 2 P and 2 P + 1 of the 16: expanded, rounded (or split) and packed.  The high part is
// rounded toward zero in the split form (one instruction for the pair): the low part holds what
// is left, w - hi, which is exact in fp32 before its own rounding to f16.
template <class F, bool SPLIT, int P>
__device__ __forceinline__ void frag_pair(AFrag<SPLIT> &f, const typename F::Pre &pre, const typename F::Raw &r,
                                          uint32_t g) {
    const float w0 = F::template elem<2 * P>(pre, r, g), w1 = F::template elem<2 * P + 1>(pre, r, g);
    constexpr int s2 = P / 4, i = P % 4;
    if constexpr (SPLIT) {
        const auto hz = __builtin_amdgcn_cvt_pkrtz(w0, w1);
        half2v h;
        __builtin_memcpy(&h, &hz, 4);
        f.hi[s2][i] = h;
        // l = f16(w - h) per half: one mixed-precision multiply-add each takes the f16 half of h as
        // it is, subtracts it from the fp32 value and rounds the difference to f16
        uint32_t hb, lb;
        __builtin_memcpy(&hb, &h, 4);
        asm("v_fma_mixlo_f16 %0, %1, -1.0, %2 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(lb) : "v"(hb), "v"(w0));
        asm("v_fma_mixhi_f16 %0, %1, -1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "+v"(lb) : "v"(hb), "v"(w1));
        half2v l;
        __builtin_memcpy(&l, &lb, 4);
        f.lo[s2][i] = l;
    } else {
        half2v h;
        h[0] = (_Float16)w0;
        h[1] = (_Float16)w1;
        f.hi[s2][i] = h;
    }
}

template <class F, bool SPLIT, int P = 0>
__device__ __forceinline__ void frag_pairs_from(AFrag<SPLIT> &f, const typename F::Pre &pre,
                                                const typename F::Raw &r, uint32_t g) {
    if constexpr (P < 8) {
        frag_pair<F, SPLIT, P>(f, pre, r, g);
        frag_pairs_from<F, SPLIT, P + 1>(f, pre, r, g);
    }
}

// Piece K of the nine a chunk's expansion is cut into: the shared part, then the eight pairs.
template <class F, bool SPLIT, int K>
__device__ __forceinline__ void frag_piece(AFrag<SPLIT> &f, typename F::Pre &pre, const typename F::Raw &r,
                                           uint32_t ncols, uint32_t chunk, uint32_t g) {
    if constexpr (K == 0) {
        F::pre(pre, r, ncols, chunk, g);
    } else {
        frag_pair<F, SPLIT, K - 1>(f, pre, r, g);
    }
}

// The pieces of row block B (of RB) that belong to step STEP of NSTEP: the RB x 9 pieces of a wave
// are spread evenly, piece K of block B goes to step (B * 9 + K) * NSTEP / (9 RB).
template <class F, bool SPLIT, int STEP, int NSTEP, int RB, int B, int K = 0>
__device__ __forceinline__ void frag_pieces_of_step(AFrag<SPLIT> &f, typename F::Pre &pre,
                                                    const typename F::Raw &r, uint32_t ncols, uint32_t chunk,
                                                    uint32_t g) {
    if constexpr (K < 9) {
        if constexpr ((B * 9 + K) * NSTEP / (9 * RB) == STEP) frag_piece<F, SPLIT, K>(f, pre, r, ncols, chunk, g);
        frag_pieces_of_step<F, SPLIT, STEP, NSTEP, RB, B, K + 1>(f, pre, r, ncols, chunk, g);
    }
}

__device__ __forceinline__ half8 as_half8(const half2v (&h)[4]) {
    half8 v;
    __builtin_memcpy(&v, h, 16);
    return v;
}

template <int I, int N, class Fn>
__device__ __forceinline__ void static_for(Fn &&fn) {
    if constexpr (I < N) {
        fn(std::integral_constant<int, I>{});
        static_for<I + 1, N>(fn);
    }
}

// SPLIT: both operands are pairs of f16 numbers (high part, low part); the product is
// W_hi X_hi + W_hi X_lo + W_lo X_hi, three MFMAs per sub-block instead of one, which leaves an
// error of about 2^-22 per term instead of 2^-11.
//
// The loop is software-pipelined: while the matrix cores multiply the weights of iteration it,
// the vector ALU expands those of iteration it + 1 (fetched during iteration it - 1) -- the two
// waves of a SIMD run in step between barriers, so the overlap has to come from inside a wave.
// RB: blocks of 16 rows per wave (a tile is 64 RB rows); every block multiplies the same LDS words.
template <class F, int NT, bool SPLIT, int RB>
__global__ __launch_bounds__(KWAVES * 64) void gemm_lds_kernel(const GemmArgs a) {
    extern __shared__ u32x4 xs[];  // [2 buffers][2 chunks][high: NT * 128 words (, low: the same)]
    constexpr uint32_t CW = NT * 128;               // words of one chunk of one part
    constexpr uint32_t CWX = SPLIT ? 2 * CW : CW;   // words of one chunk in LDS
    constexpr uint32_t NTHREADS = KWAVES * 64;
    constexpr int SW = (2 * CWX + NTHREADS - 1) / NTHREADS;  // staged words per thread
    constexpr uint32_t TILE = 64 * RB;              // rows of a workgroup
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t j = lane & 15, g = lane >> 4;
    const uint32_t rb = wave & 3, kh = wave >> 2;
    // Workgroup w works on part w % ks of the K range of tile w / ks.  Workgroups are handed to
    // the eight XCDs in turn, each with an L2 cache of its own: with the part index varying
    // fastest an XCD sees only every (8 / ks)-th part of the activations, which every tile reads
    // again, instead of all of them.
    const uint32_t ky = blockIdx.x % a.ks, tile = blockIdx.x / a.ks;
    // which matrix this tile belongs to (uniform over the workgroup)
    uint32_t mi = 0;
    if (a.nmat > 1 && tile >= a.m[1].tile0) mi = 1;
    if (a.nmat > 2 && tile >= a.m[2].tile0) mi = 2;
    const GemmMat &m = a.m[mi];
    // a wave's RB blocks of 16 rows: blocks rb, rb + 4, .. of the tile
    const uint32_t row0 = (tile - m.tile0) * TILE + 16 * rb;
    typename F::Lane wl[RB];  // where this lane's rows of the A operands lie
#pragma unroll
    for (int b = 0; b < RB; ++b) F::lane_init(wl[b], a.ncols, min(row0 + 64 * b + j, m.nrows - 1), g);
    // K is walked in pairs of chunks (kpad is a multiple of two chunks)
    const uint32_t npairs = a.kpad / (2 * KC);
    const uint32_t per = (npairs + a.ks - 1) / a.ks;
    const uint32_t p0 = min(ky * per, npairs), p1 = min(npairs, p0 + per);
    const uint32_t n_it = p1 - p0;

    floatx4 acc[RB][NT];
#pragma unroll
    for (int b = 0; b < RB; ++b) {
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[b][n] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    // Staged words of this thread: word tid + 512 q of the pair of chunks, q < SW; in memory the
    // low parts form a second array behind the high parts (a.xl, within 2 GiB of a.xh: the
    // launcher checks), so one uniform base per iteration and a 32-bit offset per word address
    // them all.  All loads are unconditional: past the end the last pair is fetched again and
    // not used.
    uint32_t soff[SW];  // byte offsets from the pair's first high word
#pragma unroll
    for (int q = 0; q < SW; ++q) {
        const uint32_t w = min(tid + NTHREADS * q, 2 * CWX - 1);
        const uint32_t ch = w / CWX, ww = w % CWX;
        soff[q] = (SPLIT && ww >= CW) ? a.xl_offset + (ch * CW + ww - CW) * 16 : (ch * CW + ww) * 16;
    }
    auto pair_at = [&](uint32_t it) { return min(p0 + it, npairs - 1); };  // uniform
    auto stage_load = [&](u32x4 (&st)[SW], uint32_t pair) {
        const char *base = reinterpret_cast<const char *>(a.xh) + (size_t)pair * (2 * CW * 16);
#pragma unroll
        for (int q = 0; q < SW; ++q) st[q] = load_at<u32x4>(reinterpret_cast<const uint8_t *>(base), soff[q]);
    };
    u32x4 st[SW];
    // Two sets of operands and of fetched bytes, used in turn: iteration it multiplies with
    // A[it & 1] while it expands R[it & 1] (the bytes of iteration it + 1) into A[~it & 1] and
    // fetches the bytes of iteration it + 2 into R[~it & 1].
    AFrag<SPLIT> A0[RB], A1[RB];
    typename F::Raw R0[RB], R1[RB];
    if (n_it > 0) {
        stage_load(st, p0);
#pragma unroll
        for (int b = 0; b < RB; ++b) {
            typename F::Raw r0;
            F::load(r0, m, a.ncols, wl[b], 2 * p0 + kh);
            F::load(R0[b], m, a.ncols, wl[b], 2 * pair_at(1) + kh);
            typename F::Pre pre0;
            F::pre(pre0, r0, a.ncols, 2 * p0 + kh, g);
            frag_pairs_from<F, SPLIT>(A0[b], pre0, r0, g);
        }
    }
    auto iteration = [&](uint32_t it, const AFrag<SPLIT>(&A)[RB], AFrag<SPLIT>(&An)[RB],
                         const typename F::Raw(&rn)[RB], typename F::Raw(&rnn)[RB]) {
        u32x4 *buf = xs + (it & 1) * 2 * CWX;
#pragma unroll
        for (int q = 0; q < SW; ++q) {
            if (2 * CWX % NTHREADS == 0 || tid + NTHREADS * q < 2 * CWX) buf[tid + NTHREADS * q] = st[q];
        }
        __syncthreads();
        const uint32_t pn = pair_at(it + 1);
        stage_load(st, pn);
#pragma unroll
        for (int b = 0; b < RB; ++b) F::load(rnn[b], m, a.ncols, wl[b], 2 * pair_at(it + 2) + kh);
        // The 2 NT steps of an iteration (one token block of one half chunk each): the LDS words of
        // step + 2 are requested, the step's MFMAs issued (every row block of the wave uses the same
        // words), and a piece of the expansion of the next iteration's weights done, in this order
        // (nothing is scheduled across a step's end).
        typename F::Pre pre[RB];
        const uint32_t cn = 2 * pn + kh;
        const u32x4 *bsrc = buf + kh * CWX + lane;
        constexpr int NSTEP = 2 * NT, AHEAD = 2;
        u32x4 bh[AHEAD + 1], bl[AHEAD + 1];
#pragma unroll
        for (int d = 0; d < AHEAD && d < NSTEP; ++d) {
            bh[d] = bsrc[((d % NT) * 2 + d / NT) * 64];
            if (SPLIT) bl[d] = bsrc[CW + ((d % NT) * 2 + d / NT) * 64];
        }
        __builtin_amdgcn_sched_barrier(0);
        static_for<0, NSTEP>([&](auto step_c) {
            constexpr int step = decltype(step_c)::value;
            constexpr int s2 = step / NT, n = step % NT, cur = step % (AHEAD + 1);
            if constexpr (step + AHEAD < NSTEP) {
                constexpr int sn = step + AHEAD, slot = sn % (AHEAD + 1);
                bh[slot] = bsrc[((sn % NT) * 2 + sn / NT) * 64];
                if (SPLIT) bl[slot] = bsrc[CW + ((sn % NT) * 2 + sn / NT) * 64];
            }
            half8 b8, l8;
            __builtin_memcpy(&b8, &bh[cur], 16);
            if constexpr (SPLIT) __builtin_memcpy(&l8, &bl[cur], 16);
            static_for<0, RB>([&](auto b_c) {
                constexpr int b = decltype(b_c)::value;
                acc[b][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(A[b].hi[s2]), b8, acc[b][n], 0, 0, 0);
                if constexpr (SPLIT) {
                    acc[b][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(A[b].lo[s2]), b8, acc[b][n], 0, 0, 0);
                    acc[b][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(A[b].hi[s2]), l8, acc[b][n], 0, 0, 0);
                }
            });
            // pieces of this step: the RB blocks' nine pieces each, one block after the other
            static_for<0, RB>([&](auto b_c) {
                constexpr int b = decltype(b_c)::value;
                frag_pieces_of_step<F, SPLIT, step, NSTEP, RB, b>(An[b], pre[b], rn[b], a.ncols, cn, g);
            });
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    for (uint32_t it = 0; it < n_it; it += 2) {
        iteration(it, A0, A1, R0, R1);
        if (it + 1 < n_it) iteration(it + 1, A1, A0, R1, R0);
    }
    // waves 4-7 hand their sums to waves 0-3 through LDS
    __syncthreads();
    float4 *red = reinterpret_cast<float4 *>(xs);  // [RB][4 row blocks][NT][64]
    if (kh == 1) {
#pragma unroll
        for (int b = 0; b < RB; ++b) {
#pragma unroll
            for (int n = 0; n < NT; ++n)
                red[((b * 4 + rb) * NT + n) * 64 + lane] =
                    make_float4(acc[b][n][0], acc[b][n][1], acc[b][n][2], acc[b][n][3]);
        }
    }
    __syncthreads();
    if (kh == 1) return;
#pragma unroll
    for (int b = 0; b < RB; ++b) {
        const uint32_t r4 = row0 + 64 * b + 4 * g;  // acc[b][n] = rows r4 .. r4 + 3 of token 16 n + j
#pragma unroll
        for (int n = 0; n < NT; ++n) {
            const float4 p = red[((b * 4 + rb) * NT + n) * 64 + lane];
            // the sums carry the factor the weights were expanded with: an exact scaling back
            constexpr float u = 1.0f / kWeightScale;
            float4 v = make_float4((acc[b][n][0] + p.x) * u, (acc[b][n][1] + p.y) * u, (acc[b][n][2] + p.z) * u,
                                   (acc[b][n][3] + p.w) * u);
            const uint32_t tok = n * 16 + j;
            if (tok >= a.T || r4 >= m.nrows) continue;
            float *o;
            bool add = false;
            if (a.ks > 1) {
                // plain partial sum
                o = a.part + ((size_t)ky * a.T + tok) * a.total_rows + m.roff + r4;
            } else {
                const float xs_t = a.xscale ? a.xscale[tok] : 1.f;
                v = make_float4(v.x * xs_t, v.y * xs_t, v.z * xs_t, v.w * xs_t);
                if (m.bias) {
                    if (r4 + 3 < m.nrows) {
                        v.x += m.bias[r4];
                        v.y += m.bias[r4 + 1];
                        v.z += m.bias[r4 + 2];
                        v.w += m.bias[r4 + 3];
                    } else {
                        v.x += m.bias[r4];
                        if (r4 + 1 < m.nrows) v.y += m.bias[r4 + 1];
                        if (r4 + 2 < m.nrows) v.z += m.bias[r4 + 2];
                    }
                }
                o = m.out + (size_t)tok * m.out_stride + r4;
                add = a.accumulate != 0;
            }
            if (r4 + 3 < m.nrows && (reinterpret_cast<uintptr_t>(o) & 15u) == 0) {
                if (add) {
                    const float4 q = *reinterpret_cast<const float4 *>(o);
                    v = make_float4(q.x + v.x, q.y + v.y, q.z + v.z, q.w + v.w);
                }
                *reinterpret_cast<float4 *>(o) = v;
            } else {
                o[0] = add ? o[0] + v.x : v.x;
                if (r4 + 1 < m.nrows) o[1] = add ? o[1] + v.y : v.y;
                if (r4 + 2 < m.nrows) o[2] = add ? o[2] + v.z : v.z;
                if (r4 + 3 < m.nrows) o[3] = add ? o[3] + v.w : v.w;
            }
        }
    }
}

// out[t][r] (= or +=) xscale[t] * (part[0][t][r] + part[1][t][r] + ...) + bias[r]
__global__ __launch_bounds__(256) void gemm_reduce_kernel(const GemmArgs a) {
    const uint32_t rg = blockIdx.x * 256 + threadIdx.x, t = blockIdx.y;  // row among all matrices
    if (rg >= a.total_rows) return;
    uint32_t mi = 0;
    if (a.nmat > 1 && rg >= a.m[1].roff) mi = 1;
    if (a.nmat > 2 && rg >= a.m[2].roff) mi = 2;
    const GemmMat &m = a.m[mi];
    const uint32_t r = rg - m.roff;
    const float *p = a.part + (size_t)t * a.total_rows + rg;
    float v = p[0];
    for (uint32_t y = 1; y < a.ks; ++y) v += p[(size_t)y * a.T * a.total_rows];
    v *= a.xscale ? a.xscale[t] : 1.f;
    if (m.bias) v += m.bias[r];
    float *o = m.out + (size_t)t * m.out_stride + r;
    *o = a.accumulate ? *o + v : v;
}

// The same for pairs of rows, with the rotary position encoding of the matrices marked for it
// (ops/rope.wgsl:35-78, the arithmetic of rope_rows_kernel below): thread (i, t) adds up the two
// rows of pair i of token t -- rows 2 i and 2 i + 1, or i' and i' + head_size / 2 within a head
// in the Neox variant -- and rotates them by the angle of position pos0 + t.  Every matrix of
// the launch has an even number of rows; nothing is accumulated onto the output.
__global__ __launch_bounds__(256) void gemm_reduce_rope_kernel(const GemmArgs a) {
    const uint32_t pg = blockIdx.x * 256 + threadIdx.x, t = blockIdx.y;  // pair among all matrices
    if (2 * pg >= a.total_rows) return;
    uint32_t mi = 0;
    if (a.nmat > 1 && 2 * pg >= a.m[1].roff) mi = 1;
    if (a.nmat > 2 && 2 * pg >= a.m[2].roff) mi = 2;
    const GemmMat &m = a.m[mi];
    const uint32_t i = pg - m.roff / 2, hs = a.rope_head_size;
    uint32_t ra = 2 * i, rb = 2 * i + 1;
    if (m.rope && a.rope_neox) {
        ra = i + (2 * i / hs) * (hs / 2);
        rb = ra + hs / 2;
    }
    const float *pa = a.part + (size_t)t * a.total_rows + m.roff + ra;
    const float *pb = a.part + (size_t)t * a.total_rows + m.roff + rb;
    float x = pa[0], y = pb[0];
    for (uint32_t k = 1; k < a.ks; ++k) {
        x += pa[(size_t)k * a.T * a.total_rows];
        y += pb[(size_t)k * a.T * a.total_rows];
    }
    const float xs_t = a.xscale ? a.xscale[t] : 1.f;
    x *= xs_t;
    y *= xs_t;
    if (m.bias) {
        x += m.bias[ra];
        y += m.bias[rb];
    }
    float *o = m.out + (size_t)t * m.out_stride;
    if (m.rope) {
        const float head_dim = (float)((i * 2) % hs);
        const float theta = powf(a.rope_base, -head_dim / (float)hs);
        float sn, cs;
        sincosf((float)(a.rope_pos0 + t) * theta, &sn, &cs);
        o[ra] = cs * x - sn * y;
        o[rb] = sn * x + cs * y;
    } else {
        o[ra] = x;
        o[rb] = y;
    }
}

// One workgroup per token: X[t] (fp32, optionally RMS-normalised with weights w as
// the reference does: (x * rsqrt(mean(x^2) + eps)) * w, ops/rms_norm.rs:55-63) -> f16
// in the packed order described at the top, times the power of two that brings the row's
// largest |x| into (512, 1024]; the factor to undo it goes to xscale[t].  Tokens from T on and columns
// from K on are zero.  With `up` non-null the input is the gated activation
// up[k] * silu(x[k]) (ops/silu.wgsl:13-27) instead of x itself (no normalisation then).
// acc[n][0..7] += part[y .. y + B - 1][off[n] .. off[n] + 7], part by part in the order of y; the
// loads of all B parts are requested before the first sum (a chain of memory round trips
// otherwise).  ystride: floats from one part to the next.
template <int B, int N>
__device__ __forceinline__ void add_part_batch(float (&acc)[N][8], const float *__restrict__ part, size_t ystride,
                                               const size_t (&off)[N], uint32_t y) {
    float4 q[B][N][2];
#pragma unroll
    for (int b = 0; b < B; ++b) {
#pragma unroll
        for (int n = 0; n < N; ++n) {
            const float4 *p = reinterpret_cast<const float4 *>(part + (size_t)(y + b) * ystride + off[n]);
            q[b][n][0] = p[0];
            q[b][n][1] = p[1];
        }
    }
#pragma unroll
    for (int b = 0; b < B; ++b) {
#pragma unroll
        for (int n = 0; n < N; ++n) {
            acc[n][0] += q[b][n][0].x;
            acc[n][1] += q[b][n][0].y;
            acc[n][2] += q[b][n][0].z;
            acc[n][3] += q[b][n][0].w;
            acc[n][4] += q[b][n][1].x;
            acc[n][5] += q[b][n][1].y;
            acc[n][6] += q[b][n][1].z;
            acc[n][7] += q[b][n][1].w;
        }
    }
}
// all ks parts, four, two or one at a time
template <int N>
__device__ __forceinline__ void add_parts(float (&acc)[N][8], const float *__restrict__ part, size_t ystride,
                                          const size_t (&off)[N], uint32_t ks) {
    uint32_t y = 0;
    for (; y + 4 <= ks; y += 4) add_part_batch<4, N>(acc, part, ystride, off, y);
    for (; y + 2 <= ks; y += 2) add_part_batch<2, N>(acc, part, ystride, off, y);
    for (; y < ks; ++y) add_part_batch<1, N>(acc, part, ystride, off, y);
}

constexpr int PREP_THREADS = 1024;
constexpr int PREP_GROUPS = 2;  // groups of 8 columns a thread keeps in registers
__global__ __launch_bounds__(PREP_THREADS) void prep_x_kernel(float *__restrict__ x, uint32_t x_stride,
                                                     const float *__restrict__ part, uint32_t part_ks,
                                                     uint32_t part_pair,
                                                     const float *__restrict__ up,
                                                     const float *__restrict__ norm_w, float eps,
                                                     uint4 *__restrict__ xh, uint4 *__restrict__ xl,
                                                     float *__restrict__ xscale, uint32_t K,
                                                     uint32_t kpad, uint32_t T) {
    __shared__ float red[16];
    const uint32_t t = blockIdx.x, tid = threadIdx.x, nt = gridDim.x / 16;
    // 16-byte word of (token t, columns 8 k8 .. 8 k8 + 7)
    auto word_index = [&](uint32_t k8) {
        const uint32_t c = k8 >> 3, s2 = (k8 >> 2) & 1, g = k8 & 3;
        return (((size_t)c * nt + (t >> 4)) * 2 + s2) * 64 + 16 * g + (t & 15);
    };
    const uint32_t ngroups = kpad / 8;
    if (t >= T) {
        for (uint32_t k8 = tid; k8 < ngroups; k8 += PREP_THREADS) {
            xh[word_index(k8)] = make_uint4(0, 0, 0, 0);
            if (xl) xl[word_index(k8)] = make_uint4(0, 0, 0, 0);
        }
        if (tid == 0) xscale[t] = 0.f;
        return;
    }
    float *xr = x + (size_t)t * x_stride;
    const float *ur = up ? up + (size_t)t * x_stride : nullptr;
    // Rows of up to 8 * PREP_GROUPS * PREP_THREADS columns are read once, 8 consecutive
    // columns per thread and group, and kept in registers (v); longer rows are re-read from
    // memory by the later passes.  (K is a multiple of 32 for every quantized format.)
    const bool cached = ngroups <= PREP_GROUPS * PREP_THREADS && K % 8 == 0 && x_stride % 4 == 0 &&
                        ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(up) |
                          reinterpret_cast<uintptr_t>(part)) & 15u) == 0;  // 16-byte loads below
    // the product before this kernel may have left  x[t] += xscale[t] * (part[0][t] + part[1][t]
    // + ...)  to be done here (part: [part_ks][T][K], xscale[t] still that product's factor)
    // With part_pair the partial sums are 2 K wide and hold a gate product in [0, K) and an up
    // product in [K, 2 K): the gated activation is formed from their sums, x and up are not
    // read (only for rows that fit the registers: the launcher sees to that).
    const float old_scale = part_ks ? xscale[t] : 0.f;
    if (part_ks && !cached) {
        for (uint32_t k = tid; k < K; k += PREP_THREADS) {
            const float *p = part + (size_t)t * K + k;
            float sum = p[0];
            for (uint32_t y = 1; y < part_ks; ++y) sum += p[(size_t)y * T * K];
            xr[k] += sum * old_scale;
        }
        __syncthreads();  // every thread reads what others wrote (same workgroup only)
    }
    float v[PREP_GROUPS][8];
    auto raw = [&](uint32_t k) -> float {  // the value before normalisation
        if (k >= K) return 0.f;
        const float xv = xr[k];
        return ur ? ur[k] * (xv / (1.0f + expf(-xv))) : xv;
    };
    if (cached) {
#pragma unroll
        for (int i = 0; i < PREP_GROUPS; ++i) {
            const uint32_t k0 = 8 * (tid + i * PREP_THREADS);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[i][e] = 0.f;
            if (k0 < K && part_ks && part_pair) {
                const size_t wide = 2 * (size_t)K;
                float gu[2][8] = {};  // sums of the gate parts and of the up parts
                const size_t off[2] = {(size_t)t * wide + k0, (size_t)t * wide + K + k0};
                add_parts<2>(gu, part, (size_t)T * wide, off, part_ks);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float xv = gu[0][e] * old_scale;
                    v[i][e] = (gu[1][e] * old_scale) * (xv / (1.0f + expf(-xv)));
                }
            } else if (k0 < K) {
                float4 *xp = reinterpret_cast<float4 *>(xr + k0);
                float4 a0 = xp[0], a1 = xp[1];
                if (part_ks) {
                    float sp[1][8] = {};
                    const size_t off[1] = {(size_t)t * K + k0};
                    add_parts<1>(sp, part, (size_t)T * K, off, part_ks);
                    a0 = make_float4(a0.x + sp[0][0] * old_scale, a0.y + sp[0][1] * old_scale,
                                     a0.z + sp[0][2] * old_scale, a0.w + sp[0][3] * old_scale);
                    a1 = make_float4(a1.x + sp[0][4] * old_scale, a1.y + sp[0][5] * old_scale,
                                     a1.z + sp[0][6] * old_scale, a1.w + sp[0][7] * old_scale);
                    xp[0] = a0;
                    xp[1] = a1;
                }
                const float xv[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
                if (ur) {
                    const float4 *up4 = reinterpret_cast<const float4 *>(ur + k0);
                    const float4 u0 = up4[0], u1 = up4[1];
                    const float uv[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[i][e] = uv[e] * (xv[e] / (1.0f + expf(-xv[e])));
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[i][e] = xv[e];
                }
            }
        }
    }
    float rs = 1.f;
    if (norm_w) {
        float ss = 0.f;
        if (cached) {
#pragma unroll
            for (int i = 0; i < PREP_GROUPS; ++i) {
#pragma unroll
                for (int e = 0; e < 8; ++e) ss = fmaf(v[i][e], v[i][e], ss);
            }
        } else {
            for (uint32_t k = tid; k < K; k += PREP_THREADS) ss = fmaf(xr[k], xr[k], ss);
        }
        rs = 1.0f / sqrtf(block_sum(ss, red) / (float)K + eps);
    }
    auto value = [&](uint32_t k, float r) { return norm_w && k < K ? (r * rs) * norm_w[k] : r; };
    float amax = 0.f;
    if (cached) {
#pragma unroll
        for (int i = 0; i < PREP_GROUPS; ++i) {
            const uint32_t k0 = 8 * (tid + i * PREP_THREADS);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                v[i][e] = value(k0 + e, v[i][e]);
                amax = fmaxf(amax, fabsf(v[i][e]));
            }
        }
    } else {
        for (uint32_t k = tid; k < K; k += PREP_THREADS) amax = fmaxf(amax, fabsf(value(k, raw(k))));
    }
    amax = block_max(amax, red);
    float down = 1.f, undo = 1.f;
    for (int it = 0; it < 120 && amax * down > 1024.f; ++it) {  // uniform over the workgroup
        down *= 0.5f;
        undo *= 2.f;
    }
    for (int it = 0; it < 100 && amax > 0.f && amax * down <= 512.f; ++it) {
        down *= 2.f;
        undo *= 0.5f;
    }
    // high parts f16(v); low parts f16(v - high) when the split-precision product is on
    auto store = [&](uint32_t k8, const float(&f)[8]) {
        _Float16 h[8], lo[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float v = f[e] * down;
            h[e] = (_Float16)v;
            lo[e] = (_Float16)(v - (float)h[e]);
        }
        uint4 w;
        __builtin_memcpy(&w, h, 16);
        xh[word_index(k8)] = w;
        if (xl) {
            __builtin_memcpy(&w, lo, 16);
            xl[word_index(k8)] = w;
        }
    };
    if (cached) {
#pragma unroll
        for (int i = 0; i < PREP_GROUPS; ++i) {
            const uint32_t k8 = tid + i * PREP_THREADS;
            if (k8 < ngroups) store(k8, v[i]);
        }
    } else {
        for (uint32_t k8 = tid; k8 < ngroups; k8 += PREP_THREADS) {
            float f[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) f[e] = value(8 * k8 + e, raw(8 * k8 + e));
            store(k8, f);
        }
    }
    if (tid == 0) xscale[t] = undo;
}

// X[t] = table[tokens[t]]  (embedding rows of the prompt tokens)
__global__ void embed_rows_kernel(float *__restrict__ x, const float *__restrict__ table,
                                  const uint32_t *__restrict__ tokens, uint32_t dim) {
    const uint32_t t = blockIdx.y, i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < dim) x[(size_t)t * dim + i] = table[(size_t)tokens[t] * dim + i];
}

// RoPE of q[t] and of the K-cache row of position pos0 + t, for every token t
// (the arithmetic of rope_kernel in ops.hip; ops/rope.wgsl:35-78 of the reference).
__global__ void rope_rows_kernel(float *__restrict__ q, uint32_t q_stride, float *__restrict__ k,
                                 uint32_t k_stride, uint32_t n_pairs, uint32_t head_size,
                                 uint32_t kv_dim, uint32_t pos0, float base_freq, int neox) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x, t = blockIdx.y;
    if (i >= n_pairs) return;
    const uint32_t p = pos0 + t;
    float *qt = q + (size_t)t * q_stride, *kt = k + (size_t)t * k_stride;
    const float head_dim = (float)((i * 2) % head_size);
    const float theta = powf(base_freq, -head_dim / (float)head_size);
    float sn, cs;
    sincosf((float)p * theta, &sn, &cs);
    uint32_t a, b;
    if (!neox) {
        a = i * 2;
        b = a + 1;
    } else {
        const uint32_t head_id = (i * 2) / head_size;
        a = i + head_id * head_size / 2;
        b = a + head_size / 2;
    }
    if (q) {
        const float x = qt[a], y = qt[b];
        qt[a] = cs * x - sn * y;
        qt[b] = sn * x + cs * y;
    }
    if (k && i * 2 < kv_dim) {
        const float x = kt[a], y = kt[b];
        kt[a] = cs * x - sn * y;
        kt[b] = sn * x + cs * y;
    }
}


// Causal attention for a run of tokens: workgroup (h, t) computes head h of token t,
// which sits at position pos0 + t and attends to cache rows 0 .. pos0 + t (the rows of
// this run were written by the K and V products before).  Same arithmetic as the decode
// kernels (ops/batched_multiquery_attention.wgsl:24-97: scores q.k / sqrt(head_size),
// softmax, weighted sum of values), as an online softmax: 16 lanes share a position,
// a wave covers four positions at a time, the four waves stride over the positions.
struct AttnRowsArgs {
    const float *q;  // [T][q_stride]
    const float *kc, *vc;  // caches: rows kv_dim apart
    float *xb;  // [T][xb_stride]
    uint32_t q_stride, xb_stride, kv_dim, kv_mul, head_size, pos0;
};

__device__ __forceinline__ float dot4f(const float4 a, const float4 b, float acc) {
    acc = fmaf(a.x, b.x, acc);
    acc = fmaf(a.y, b.y, acc);
    acc = fmaf(a.z, b.z, acc);
    return fmaf(a.w, b.w, acc);
}
__device__ __forceinline__ float4 axpby4f(const float4 a, float sa, const float4 b, float sb) {
    return make_float4(fmaf(a.x, sa, b.x * sb), fmaf(a.y, sa, b.y * sb), fmaf(a.z, sa, b.z * sb),
                       fmaf(a.w, sa, b.w * sb));
}

template <int NV4>
__global__ __launch_bounds__(256) void attn_rows_kernel(const AttnRowsArgs a) {
    constexpr int HSP = NV4 * 64;
    __shared__ float sm_m[4], sm_l[4];
    __shared__ float sm_acc[4][HSP];
    const uint32_t h = blockIdx.x, t = blockIdx.y, pos = a.pos0 + t;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t sub = lane & 15, quarter = lane >> 4, hs = a.head_size;
    const float *kb = a.kc + (size_t)(h / a.kv_mul) * hs;
    const float *vb = a.vc + (size_t)(h / a.kv_mul) * hs;
    const float inv_sqrt_hs = 1.0f / sqrtf((float)hs);
    // float4 number sub + 16 v of the head; lanes beyond the head re-read its last one
    // with a zero q and never store
    uint32_t cv[NV4];
    float4 q[NV4], acc[NV4];
#pragma unroll
    for (int v = 0; v < NV4; ++v) {
        const bool inside = (sub + 16 * v) * 4 < hs;
        cv[v] = min(sub + 16 * v, hs / 4 - 1);
        const float4 qv =
            reinterpret_cast<const float4 *>(a.q + (size_t)t * a.q_stride + (size_t)h * hs)[cv[v]];
        q[v] = inside ? qv : make_float4(0.f, 0.f, 0.f, 0.f);
        acc[v] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float mx = -INFINITY, l = 0.f;
    for (uint32_t p0 = wave * 4; p0 <= pos; p0 += 16) {  // uniform over the wave
        const uint32_t tt = p0 + quarter;
        const uint32_t tc = min(tt, pos);
        const float4 *kp = reinterpret_cast<const float4 *>(kb + (size_t)tc * a.kv_dim);
        const float4 *vp = reinterpret_cast<const float4 *>(vb + (size_t)tc * a.kv_dim);
        float4 kk[NV4], vv[NV4];
#pragma unroll
        for (int v = 0; v < NV4; ++v) kk[v] = kp[cv[v]];
#pragma unroll
        for (int v = 0; v < NV4; ++v) vv[v] = vp[cv[v]];
        float part = 0.f;
#pragma unroll
        for (int v = 0; v < NV4; ++v) part = dot4f(q[v], kk[v], part);
        const float s = row16_sum(part) * inv_sqrt_hs;
        if (tt <= pos) {  // uniform within a 16-lane row
            const float mn = fmaxf(mx, s);
            const float sc = __expf(mx - mn), p = __expf(s - mn);
            l = fmaf(l, sc, p);
#pragma unroll
            for (int v = 0; v < NV4; ++v) acc[v] = axpby4f(acc[v], sc, vv[v], p);
            mx = mn;
        }
    }
    // the four quarters of the wave
#pragma unroll
    for (int step = 16; step <= 32; step <<= 1) {
        const float om = __shfl_xor(mx, step, 64), ol = __shfl_xor(l, step, 64);
        const float M = fmaxf(mx, om);
        const float sa = mx == -INFINITY ? 0.f : __expf(mx - M);
        const float sb = om == -INFINITY ? 0.f : __expf(om - M);
        l = fmaf(l, sa, ol * sb);
#pragma unroll
        for (int v = 0; v < NV4; ++v) {
            float4 o;
            o.x = __shfl_xor(acc[v].x, step, 64);
            o.y = __shfl_xor(acc[v].y, step, 64);
            o.z = __shfl_xor(acc[v].z, step, 64);
            o.w = __shfl_xor(acc[v].w, step, 64);
            acc[v] = axpby4f(acc[v], sa, o, sb);
        }
        mx = M;
    }
    // the four waves
    if (lane == 0) {
        sm_m[wave] = mx;
        sm_l[wave] = l;
    }
    if (quarter == 0) {
#pragma unroll
        for (int v = 0; v < NV4; ++v) reinterpret_cast<float4 *>(&sm_acc[wave][0])[sub + 16 * v] = acc[v];
    }
    __syncthreads();
    for (uint32_t d = threadIdx.x; d < hs; d += 256) {
        const float M = fmaxf(fmaxf(sm_m[0], sm_m[1]), fmaxf(sm_m[2], sm_m[3]));
        float L = 0.f, o = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float wgt = sm_m[w] == -INFINITY ? 0.f : __expf(sm_m[w] - M);
            L = fmaf(sm_l[w], wgt, L);
            o = fmaf(wgt > 0.f ? sm_acc[w][d] : 0.f, wgt, o);
        }
        a.xb[(size_t)t * a.xb_stride + (size_t)h * hs + d] = o / L;
    }
}

// The same attention for 16 tokens of a run at once, on the fp32 matrix cores
// (v_mfma_f32_16x16x4_f32: operands and sums are fp32, so the arithmetic stays that of the
// step).  Workgroup (h, tb) computes head h of tokens 16 tb .. 16 tb + 15; its four waves
// share out the blocks of 16 cache rows and merge at the end, so a K or V row is read once
// per 16 tokens instead of once per token.  Per block of rows, with lane = (g, n):
//   S^T[row][token] = K · Q^T : A = K rows (lane n = row, k-slot g = dimension 16 c + 4 g + e in
//                     step (c, e)), B = Q^T (lane n = token), 4 HS16 steps -> each lane holds
//                     the scores of rows 4 g + i (i < 4) for token n;
//   online softmax per token: maximum and sum over the lane's 4 rows and the 4 lane groups;
//   O^T[dim][token] += V^T · P^T : A = V^T (lane n = dimension 16 b + n, k-slot g = row 4 g + i
//                     in step i), B = the lane's own P values -- no transposition anywhere.
template <int HS16>
__global__ __launch_bounds__(256) void attn_block_kernel(const AttnRowsArgs a, uint32_t T) {
    constexpr int HS = HS16 * 16;
    __shared__ float sm_m[4][16], sm_l[4][16];
    __shared__ float sm_o[4][HS][17];
    const uint32_t h = blockIdx.x, t0 = blockIdx.y * 16;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t n = lane & 15, g = lane >> 4;
    const size_t head_off = (size_t)(h / a.kv_mul) * HS;
    const float inv_sqrt_hs = 1.0f / sqrtf((float)HS);
    // this lane's token (the B operand of the score product); tokens past the run repeat the last
    const uint32_t tq = min(t0 + n, T - 1), pos_q = a.pos0 + tq;
    const uint32_t last_pos = a.pos0 + min(t0 + 15, T - 1);  // rows 0 .. last_pos exist
    const uint32_t nblk = last_pos / 16 + 1;
    float4 q[HS16];
#pragma unroll
    for (int c = 0; c < HS16; ++c)
        q[c] = *reinterpret_cast<const float4 *>(a.q + (size_t)tq * a.q_stride + (size_t)h * HS + 16 * c + 4 * g);
    floatx4 acc[HS16];
#pragma unroll
    for (int b = 0; b < HS16; ++b) acc[b] = floatx4{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    for (uint32_t blk = wave; blk < nblk; blk += 4) {  // uniform over the wave
        const uint32_t pbase = blk * 16;
        const float *krow = a.kc + (size_t)min(pbase + n, last_pos) * a.kv_dim + head_off + 4 * g;
        float4 k[HS16];
#pragma unroll
        for (int c = 0; c < HS16; ++c) k[c] = *reinterpret_cast<const float4 *>(krow + 16 * c);
        float v[HS16][4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float *vrow = a.vc + (size_t)min(pbase + 4 * g + i, last_pos) * a.kv_dim + head_off + n;
#pragma unroll
            for (int b = 0; b < HS16; ++b) v[b][i] = vrow[16 * b];
        }
        floatx4 s = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < HS16; ++c) {
            s = __builtin_amdgcn_mfma_f32_16x16x4f32(k[c].x, q[c].x, s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_16x16x4f32(k[c].y, q[c].y, s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_16x16x4f32(k[c].z, q[c].z, s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_16x16x4f32(k[c].w, q[c].w, s, 0, 0, 0);
        }
        // s[i] = score of row pbase + 4 g + i for token n; rows after the token's position do not count
        float sc[4], mloc = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sc[i] = pbase + 4 * g + i <= pos_q ? s[i] * inv_sqrt_hs : -INFINITY;
            mloc = fmaxf(mloc, sc[i]);
        }
        mloc = fmaxf(mloc, __shfl_xor(mloc, 16, 64));
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
        const float mn = fmaxf(m, mloc);
        const float scale = mn == -INFINITY ? 1.f : __expf(m - mn);
        float p[4], lsum = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            p[i] = sc[i] == -INFINITY ? 0.f : __expf(sc[i] - mn);
            lsum += p[i];
        }
        lsum += __shfl_xor(lsum, 16, 64);
        lsum += __shfl_xor(lsum, 32, 64);
        l = fmaf(l, scale, lsum);
        m = mn;
#pragma unroll
        for (int b = 0; b < HS16; ++b) {
            acc[b] = floatx4{acc[b][0] * scale, acc[b][1] * scale, acc[b][2] * scale, acc[b][3] * scale};
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(v[b][i], p[i], acc[b], 0, 0, 0);
        }
    }
    // acc[b][i] = O^T[dimension 16 b + 4 g + i][token n] of this wave's rows; merge the four waves
    if (g == 0) {
        sm_m[wave][n] = m;
        sm_l[wave][n] = l;
    }
#pragma unroll
    for (int b = 0; b < HS16; ++b) {
#pragma unroll
        for (int i = 0; i < 4; ++i) sm_o[wave][16 * b + 4 * g + i][n] = acc[b][i];
    }
    __syncthreads();
    for (uint32_t idx = threadIdx.x; idx < 16 * HS; idx += 256) {
        const uint32_t tok = idx / HS, d = idx % HS;
        if (t0 + tok >= T) continue;
        const float M = fmaxf(fmaxf(sm_m[0][tok], sm_m[1][tok]), fmaxf(sm_m[2][tok], sm_m[3][tok]));
        float L = 0.f, o = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float wgt = sm_m[w][tok] == -INFINITY ? 0.f : __expf(sm_m[w][tok] - M);
            L = fmaf(sm_l[w][tok], wgt, L);
            o = fmaf(sm_o[w][d][tok], wgt, o);
        }
        a.xb[(size_t)(t0 + tok) * a.xb_stride + (size_t)h * HS + d] = o / L;
    }
}


// How many workgroups split K (a power of two, at least 8 iterations each).
//   plain f16: two workgroups fit a compute unit; split while tiles x ks stays within 1.5 per unit.
//   split f16: one workgroup per unit (128 KB of LDS); pick the ks that minimises the number
//   of rounds the grid needs, counted in whole-K units (rounds / ks), with a charge per
//   doubling for the partial sums it adds.
uint32_t gemm_k_split(const wgml_ctx *ctx, uint32_t tiles, uint32_t kpad, bool split) {
    const uint32_t nchunks = kpad / KC;
    const int forced = ctx->tuning[WGML_TUNE_GEMM_K_SPLIT];  // 0: by matrix shape
    if (forced) return min((uint32_t)forced, max(nchunks / 2, 1u));  // K is walked in pairs of chunks
    const uint32_t cu = ctx->n_cu > 0 ? (uint32_t)ctx->n_cu : 256u;
    if (!split) {
        uint32_t ks = 1;
        while (ks < 8 && tiles * ks * 2 <= cu + cu / 2 && nchunks / (ks * 2) >= 8) ks *= 2;
        return ks;
    }
    uint32_t best = 1;
    float best_cost = 1e30f, charge = 0.f;
    for (uint32_t ks = 1; ks <= 8 && (ks == 1 || nchunks / ks >= 8); ks *= 2, charge += 0.08f) {
        const float cost = (float)((tiles * ks + cu - 1) / cu) / (float)ks + charge;
        if (cost < best_cost) {
            best_cost = cost;
            best = ks;
        }
    }
    return best;
}

template <class F, int NT, bool SPLIT, int RB>
int launch_gemm_kernel(wgml_ctx *ctx, const GemmArgs &a, dim3 grid) {
    // 2 buffers x 2 chunks x NT x 2 KiB (x 2 parts); the sums handed over at the end need RB x NT x 4 KiB
    const size_t lds = max((size_t)NT * 8192 * (SPLIT ? 2 : 1), (size_t)RB * NT * 4096);
    wgml_kernel_info &ki = ctx->kernel_info[(const void *)gemm_lds_kernel<F, NT, SPLIT, RB>];
    if (lds > 64 * 1024 && !ki.opted_in) {
        // gfx950 has 160 KB of LDS per CU; above 64 KB a kernel must opt in once
        WGML_CHECK_HIP(hipFuncSetAttribute((const void *)gemm_lds_kernel<F, NT, SPLIT, RB>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        ki.opted_in = true;
    }
    gemm_lds_kernel<F, NT, SPLIT, RB><<<grid, dim3(KWAVES * 64), lds, ctx->stream>>>(a);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

template <class F, bool SPLIT, int RB>
int launch_gemm_prec(wgml_ctx *ctx, GemmArgs &a, uint32_t tiles) {
    const dim3 grid(tiles * a.ks);
    switch (a.tpad / 16) {  // token blocks: 1, 2, 4 or 8
    case 8: WGML_TRY((launch_gemm_kernel<F, 8, SPLIT, RB>(ctx, a, grid))); break;
    case 4: WGML_TRY((launch_gemm_kernel<F, 4, SPLIT, RB>(ctx, a, grid))); break;
    case 2: WGML_TRY((launch_gemm_kernel<F, 2, SPLIT, RB>(ctx, a, grid))); break;
    default: WGML_TRY((launch_gemm_kernel<F, 1, SPLIT, RB>(ctx, a, grid))); break;
    }
    if (a.ks > 1 && !a.defer) {
        if (a.rope_head_size)
            gemm_reduce_rope_kernel<<<dim3((a.total_rows / 2 + 255) / 256, a.T), dim3(256), 0, ctx->stream>>>(a);
        else
            gemm_reduce_kernel<<<dim3((a.total_rows + 255) / 256, a.T), dim3(256), 0, ctx->stream>>>(a);
        WGML_CHECK_LAUNCH();
        ctx->launches++;
    }
    return WGML_OK;
}

template <class F>
int launch_gemm_fmt(wgml_ctx *ctx, GemmArgs &a, uint32_t tiles) {
    // one block of 16 rows per wave: two (tiles of 128 rows, half the LDS reads per MFMA) ran each
    // iteration 20 % faster per row but filled the compute units worse, no gain over a prompt pass
    return a.xl ? launch_gemm_prec<F, true, 1>(ctx, a, tiles) : launch_gemm_prec<F, false, 1>(ctx, a, tiles);
}

}  // namespace

namespace wgml {

uint32_t prefill_tpad(uint32_t T) { return T <= 16 ? 16 : T <= 32 ? 32 : T <= 64 ? 64 : 128; }
uint32_t prefill_kpad(uint32_t K) { return (K + 2 * KC - 1) / (2 * KC) * (2 * KC); }

int ensure_prefill_scratch(wgml_ctx *ctx, size_t xh_bytes) {
    if (!ctx->prefill_xscale)
        WGML_CHECK_HIP(hipMalloc((void **)&ctx->prefill_xscale, kPrefillMaxTokens * sizeof(float)));
    if (xh_bytes <= ctx->prefill_xh_bytes) return WGML_OK;
    // work already enqueued may still read the old buffer: retire it, free with the context
    if (ctx->prefill_xh) ctx->retired.push_back(ctx->prefill_xh);
    ctx->prefill_xh = nullptr;
    ctx->prefill_xh_bytes = 0;
    xh_bytes = (xh_bytes + 255) & ~(size_t)255;
    // two arrays: the f16 activations and, behind them, their low parts (split precision)
    WGML_CHECK_HIP(hipMalloc(&ctx->prefill_xh, 2 * xh_bytes));
    ctx->prefill_xl = (char *)ctx->prefill_xh + xh_bytes;
    ctx->prefill_xh_bytes = xh_bytes;
    return WGML_OK;
}

int launch_prefill_prep(wgml_ctx *ctx, float *x, uint32_t x_stride, const float *up,
                        const float *norm_w, float eps, void *xh, float *xscale, uint32_t K,
                        uint32_t T) {
    // partial sums a product with defer_reduce left: for x (K wide; x is its output), or for a
    // gate / up pair (2 K wide; x and up are then not read)
    const uint32_t pending = ctx->gemm_pending_ks, pair = ctx->gemm_pending_pair;
    ctx->gemm_pending_ks = 0;
    ctx->gemm_pending_pair = 0;
    if (pending && pair &&
        !(up && K % 8 == 0 && x_stride % 4 == 0 && prefill_kpad(K) / 8 <= (uint32_t)(PREP_GROUPS * PREP_THREADS) &&
          ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(up)) & 15u) == 0))
        return set_error(WGML_E_INVALID, "prefill_prep: pending gate/up partial sums need a gated row of at "
                                         "most %d columns", 8 * PREP_GROUPS * PREP_THREADS);
    prep_x_kernel<<<dim3(prefill_tpad(T)), dim3(PREP_THREADS), 0, ctx->stream>>>(
        x, x_stride, pending ? ctx->gemm_part : nullptr, pending, pair, up, norm_w, eps,
        reinterpret_cast<uint4 *>(xh), ctx->gemm_precise ? reinterpret_cast<uint4 *>(ctx->prefill_xl) : nullptr,
        xscale, K, prefill_kpad(K), T);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

// x[t] += the partial sums a product with defer_reduce left, for callers whose next
// kernel is not launch_prefill_prep.
__global__ void gemm_flush_kernel(float *x, uint32_t x_stride, const float *part, uint32_t ks,
                                  const float *xscale, uint32_t K, uint32_t T) {
    const uint32_t k = blockIdx.x * blockDim.x + threadIdx.x, t = blockIdx.y;
    if (k >= K) return;
    const float *p = part + (size_t)t * K + k;
    float sum = p[0];
    for (uint32_t y = 1; y < ks; ++y) sum += p[(size_t)y * T * K];
    x[(size_t)t * x_stride + k] += sum * xscale[t];
}

int launch_gemm_flush(wgml_ctx *ctx, float *x, uint32_t x_stride, const float *xscale, uint32_t K,
                      uint32_t T) {
    const uint32_t pending = ctx->gemm_pending_ks;
    ctx->gemm_pending_ks = 0;
    if (!pending) return WGML_OK;
    gemm_flush_kernel<<<dim3((K + 255) / 256, T), dim3(256), 0, ctx->stream>>>(x, x_stride, ctx->gemm_part,
                                                                          pending, xscale, K, T);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int ensure_gemm_partials(wgml_ctx *ctx, size_t bytes) {
    if (bytes <= ctx->gemm_part_bytes) return WGML_OK;
    if (ctx->gemm_part) ctx->retired.push_back(ctx->gemm_part);  // may still be read by queued work
    ctx->gemm_part = nullptr;
    ctx->gemm_part_bytes = 0;
    bytes = (bytes + (size_t(8) << 20)) & ~((size_t(1) << 20) - 1);  // grow in steps
    WGML_CHECK_HIP(hipMalloc((void **)&ctx->gemm_part, bytes));
    ctx->gemm_part_bytes = bytes;
    return WGML_OK;
}

int launch_gemm_quant_multi(wgml_ctx *ctx, const GemmTarget *targets, int n, const void *xh,
                            const float *xscale, uint32_t T, int accumulate, bool defer_reduce,
                            GemmRope *rope) {
    if (T == 0 || T > kPrefillMaxTokens)
        return set_error(WGML_E_INVALID, "gemm_quant: %u tokens (1..%u)", T, kPrefillMaxTokens);
    if (n < 1 || n > 3) return set_error(WGML_E_INVALID, "gemm_quant: %d matrices (1..3)", n);
    const wgml_qmat *first = targets[0].m;
    GemmArgs a{};
    uint32_t tiles = 0;
    for (int i = 0; i < n; ++i) {
        const wgml_qmat *q = targets[i].m;
        if (q->type != first->type || q->ncols != first->ncols)
            return set_error(WGML_E_INVALID, "gemm_quant: matrices of one launch differ in format or width");
        if (!(q->max_abs <= kGemmMaxWeight))
            return set_error(WGML_E_UNSUPPORTED,
                             "gemm_quant: a weight of magnitude up to %g does not fit the f16 operands of "
                             "the batched product (up to %g only); use the per-token product",
                             (double)q->max_abs, (double)kGemmMaxWeight);
        // the kernel addresses a matrix plane with 32-bit lane offsets (at most 1 byte per element)
        if ((uint64_t)q->nrows * q->ncols >= (uint64_t(1) << 32) - 4096)
            return set_error(WGML_E_UNSUPPORTED, "gemm_quant: a matrix of %u x %u elements (below 2^32 only)",
                             q->nrows, q->ncols);
        GemmMat &g = a.m[i];
        g.p0 = q->p0;
        g.p1 = q->p1;
        g.p2 = q->p2;
        g.p3 = q->p3;
        g.out = targets[i].out;
        g.bias = targets[i].bias;
        g.nrows = q->nrows;
        g.rope = targets[i].rope ? 1u : 0u;
        g.out_stride = targets[i].out_stride;
        g.tile0 = tiles;
        g.roff = a.total_rows;
        tiles += (q->nrows + 63) / 64;
        a.total_rows += q->nrows;
    }
    a.nmat = (uint32_t)n;
    a.xh = reinterpret_cast<const u32x4 *>(xh);
    a.xl = ctx->gemm_precise ? reinterpret_cast<const u32x4 *>(ctx->prefill_xl) : nullptr;
    if (a.xl) {
        // the kernel addresses the low parts relative to the high parts with 32 bits
        const ptrdiff_t d = reinterpret_cast<const char *>(a.xl) - reinterpret_cast<const char *>(a.xh);
        if (d <= 0 || d >= (ptrdiff_t(1) << 31))
            return set_error(WGML_E_INVALID, "gemm_quant: the activations are not the context's packed buffer");
        a.xl_offset = (uint32_t)d;
    }
    a.xscale = xscale;
    a.ncols = first->ncols;
    a.kpad = prefill_kpad(first->ncols);
    a.T = T;
    a.tpad = prefill_tpad(T);
    a.accumulate = accumulate;
    if (ctx->gemm_pending_ks)
        return set_error(WGML_E_INVALID, "gemm_quant: the partial sums a previous product left for its "
                                         "output were not added yet (launch_prefill_prep / launch_gemm_flush)");
    a.ks = gemm_k_split(ctx, tiles, a.kpad, a.xl != nullptr);
    if (a.ks > 1) {
        WGML_TRY(ensure_gemm_partials(ctx, (size_t)a.ks * T * a.total_rows * sizeof(float)));
        a.part = ctx->gemm_part;
        // the caller's next kernel adds the partial sums up itself (one matrix, plain += only)
        const bool residual = n == 1 && accumulate && !targets[0].bias;
        // a gate / up pair whose next kernel is the gated launch_prefill_prep on (gate out, up out)
        const bool pair = n == 2 && !accumulate && !targets[0].bias && !targets[1].bias &&
                          targets[0].m->nrows == targets[1].m->nrows && targets[0].m->nrows % 8 == 0 &&
                          targets[0].m->nrows <= 8u * 2 * 1024;
        a.defer = defer_reduce && (residual || pair);
        if (a.defer) {
            ctx->gemm_pending_ks = a.ks;
            ctx->gemm_pending_pair = pair ? 1 : 0;
        }
    }
    if (rope) {
        // the kernel that adds the partial sums rotates the marked targets, if there is one and
        // rows come in pairs
        bool pairs = a.ks > 1 && !a.defer && !accumulate && rope->head_size >= 2 && rope->head_size % 2 == 0;
        for (int i = 0; i < n; ++i)
            pairs = pairs && targets[i].m->nrows % 2 == 0 &&
                    (!targets[i].rope || targets[i].m->nrows % rope->head_size == 0);
        rope->applied = pairs;
        if (pairs) {
            a.rope_head_size = rope->head_size;
            a.rope_pos0 = rope->pos0;
            a.rope_base = rope->base_freq;
            a.rope_neox = rope->variant == WGML_ROPE_NEOX;
        }
    }
    switch (first->type) {
    case WGML_Q4_K: return launch_gemm_fmt<GemmQ4K>(ctx, a, tiles);
    case WGML_Q6_K: return launch_gemm_fmt<GemmQ6K>(ctx, a, tiles);
    case WGML_Q8_0: return launch_gemm_fmt<GemmQ8_0>(ctx, a, tiles);
    case WGML_Q5_K: return launch_gemm_fmt<GemmQ5K>(ctx, a, tiles);
    case WGML_Q8_K: return launch_gemm_fmt<GemmQ8K>(ctx, a, tiles);
    case WGML_Q4_0: return launch_gemm_fmt<GemmQ4_0>(ctx, a, tiles);
    case WGML_Q4_1: return launch_gemm_fmt<GemmQ4_1>(ctx, a, tiles);
    case WGML_Q5_0: return launch_gemm_fmt<GemmQ5_0>(ctx, a, tiles);
    case WGML_Q5_1: return launch_gemm_fmt<GemmQ5_1>(ctx, a, tiles);
    default:
        return set_error(WGML_E_UNSUPPORTED, "gemm_quant: matrix type %d has no batched product "
                                             "(the nine quantized block formats only)", first->type);
    }
}

int launch_gemm_quant(wgml_ctx *ctx, float *out, uint32_t out_stride, const wgml_qmat *m,
                      const void *xh, const float *xscale, uint32_t T, const float *bias,
                      int accumulate, bool defer_reduce) {
    const GemmTarget t{m, out, out_stride, bias};
    return launch_gemm_quant_multi(ctx, &t, 1, xh, xscale, T, accumulate, defer_reduce);
}

int launch_embed_rows(wgml_ctx *ctx, float *x, const float *table, const uint32_t *d_tokens,
                      uint32_t dim, uint32_t T) {
    embed_rows_kernel<<<dim3((dim + 255) / 256, T), dim3(256), 0, ctx->stream>>>(x, table, d_tokens,
                                                                                 dim);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int launch_rope_rows(wgml_ctx *ctx, int variant, uint32_t head_size, uint32_t kv_dim, uint32_t pos0,
                     float base_freq, float *q, uint32_t q_len, uint32_t q_stride, float *k,
                     uint32_t k_stride, uint32_t T) {
    const uint32_t n_pairs = q_len / 2;
    rope_rows_kernel<<<dim3((n_pairs + 63) / 64, T), dim3(64), 0, ctx->stream>>>(
        q, q_stride, k, k_stride, n_pairs, head_size, kv_dim, pos0, base_freq,
        variant == WGML_ROPE_NEOX);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int launch_attention_rows(wgml_ctx *ctx, const wgml_attn_params &p, uint32_t pos0, uint32_t T,
                          const float *q, uint32_t q_stride, const float *kc, const float *vc,
                          float *xb, uint32_t xb_stride) {
    if (p.head_size % 4 != 0 || p.head_size > 256 || p.kv_dim % 4 != 0 || q_stride % 4 != 0)
        return set_error(WGML_E_UNSUPPORTED,
                         "attention over a run of tokens: head_size %u (multiple of 4, <= 256)",
                         p.head_size);
    AttnRowsArgs a{q, kc, vc, xb, q_stride, xb_stride, p.kv_dim, p.kv_mul, p.head_size, pos0};
    if (p.head_size % 16 == 0 && p.head_size <= 128 && !ctx->tuning[WGML_TUNE_PREFILL_ATTENTION_PER_TOKEN]) {
        // 16 tokens per workgroup on the fp32 matrix cores
        const dim3 bgrid(p.n_heads, (T + 15) / 16), bblock(256);
        switch (p.head_size / 16) {
        case 1: attn_block_kernel<1><<<bgrid, bblock, 0, ctx->stream>>>(a, T); break;
        case 2: attn_block_kernel<2><<<bgrid, bblock, 0, ctx->stream>>>(a, T); break;
        case 3: attn_block_kernel<3><<<bgrid, bblock, 0, ctx->stream>>>(a, T); break;
        case 4: attn_block_kernel<4><<<bgrid, bblock, 0, ctx->stream>>>(a, T); break;
        case 5: attn_block_kernel<5><<<bgrid, bblock, 0, ctx->stream>>>(a, T); break;
        case 6: attn_block_kernel<6><<<bgrid, bblock, 0, ctx->stream>>>(a, T); break;
        case 7: attn_block_kernel<7><<<bgrid, bblock, 0, ctx->stream>>>(a, T); break;
        default: attn_block_kernel<8><<<bgrid, bblock, 0, ctx->stream>>>(a, T); break;
        }
        WGML_CHECK_LAUNCH();
        ctx->launches++;
        return WGML_OK;
    }
    const dim3 grid(p.n_heads, T), block(256);
    switch ((p.head_size + 63) / 64) {
    case 1: attn_rows_kernel<1><<<grid, block, 0, ctx->stream>>>(a); break;
    case 2: attn_rows_kernel<2><<<grid, block, 0, ctx->stream>>>(a); break;
    case 3: attn_rows_kernel<3><<<grid, block, 0, ctx->stream>>>(a); break;
    default: attn_rows_kernel<4><<<grid, block, 0, ctx->stream>>>(a); break;
    }
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

}  // namespace wgml

extern "C" {

// 1 (default): products of the batched path take both operands as pairs of f16 numbers (error
// about 2^-22 per term, three MFMAs per sub-block); 0: plain f16 operands (2^-11, one MFMA).
int wgml_ctx_set_gemm_precision(wgml_ctx *ctx, int level) {
    WGML_REQUIRE(ctx != nullptr, "wgml_ctx_set_gemm_precision: null context");
    WGML_REQUIRE(level == 0 || level == 1, "wgml_ctx_set_gemm_precision: level %d not in {0, 1}", level);
    ctx->gemm_precise = level;
    return WGML_OK;
}

// out[t] = M x[t] for T <= 128 vectors at once (x: T x ncols, out: T x nrows, both
// row-major f32) on the matrix cores; the batched counterpart of wgml_gemv_quant.
int wgml_gemm_quant(wgml_ctx *ctx, wgml_view out, const wgml_qmat *m, wgml_view x, uint32_t n_tokens) {
    WGML_REQUIRE(ctx && m, "wgml_gemm_quant: null argument");
    WGML_TRY(check_view(out, "wgml_gemm_quant: out"));
    WGML_TRY(check_view(x, "wgml_gemm_quant: x"));
    WGML_REQUIRE(n_tokens >= 1 && n_tokens <= kPrefillMaxTokens,
                 "wgml_gemm_quant: %u tokens (1..%u)", n_tokens, kPrefillMaxTokens);
    WGML_REQUIRE((uint64_t)x.len == (uint64_t)n_tokens * m->ncols,
                 "Gemm: dimension mismatch (x has %u elements, expected %u x %u)", x.len, n_tokens,
                 m->ncols);
    WGML_REQUIRE((uint64_t)out.len == (uint64_t)n_tokens * m->nrows,
                 "Gemm: dimension mismatch (out has %u elements, expected %u x %u)", out.len,
                 n_tokens, m->nrows);
    const size_t xh_bytes = (size_t)kPrefillMaxTokens * prefill_kpad(m->ncols) * 2;
    WGML_TRY(ensure_prefill_scratch(ctx, xh_bytes));
    // a prompt pass that failed half way may have left partial sums owed to its next packing
    // kernel: they are not this product's (the packing kernel would add them to x)
    ctx->gemm_pending_ks = 0;
    ctx->gemm_pending_pair = 0;
    WGML_TRY(launch_prefill_prep(ctx, view_ptr(x), m->ncols, nullptr, nullptr, 0.f, ctx->prefill_xh,
                                 ctx->prefill_xscale, m->ncols, n_tokens));
    return launch_gemm_quant(ctx, view_ptr(out), m->nrows, m, ctx->prefill_xh, ctx->prefill_xscale,
                             n_tokens, nullptr, 0, false);
}

}  // extern "C"
