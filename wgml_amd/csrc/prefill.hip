// Batched prompt processing ("prefill"): the decoder's matrix products for up to 128
// tokens at once, as a GEMM on the matrix cores.  The reference has no such path -- it
// pushes the prompt through its batch-1 step one token at a time
// (wgml-chat/src/chat_llama2.rs:155-228 with the forced-token rule of
// wgml-chat/src/sampler.rs:102-107) -- so this is new functionality whose results are
// held against exactly that: N sequential decode steps.
//
//   out[t][r] = sum_k W[r][k] * X[t][k]      W: Q4_K / Q6_K / Q8_0 as stored for the GEMV
//
// Weights are expanded to f16 in registers with the reference's dequantization
// arithmetic (fp32, then rounded to f16), activations are f16 (scaled per token by a
// power of two so that they stay in range), products accumulate in fp32 on
// v_mfma_f32_16x16x32_f16.  With f16 inputs the results differ from the fp32 path
// by about 3e-4 of a row's RMS (the tests bound it at 1e-3).
//
// Tiling.  A workgroup owns 16 matrix rows and all tokens; its 8 waves split K: wave w
// takes the 64-element chunks w, w + 8, ...  so that every weight element is expanded
// exactly once, by one wave, and used for all NT blocks of 16 tokens (NT accumulators
// of 16x16 per wave).  The 8 partial sums meet in LDS at the end, added in a fixed order.
// Nothing is shared between the waves before that, so the loop has no barrier: each wave
// keeps the loads of its next chunk (weights and activations) in flight while it
// multiplies the current one.
//
// Activations are stored in the order the B operand wants them (written by
// prep_x_kernel): for chunk c, token block n, half s2 of the chunk, lane (g, j) finds
// the 8 halves  X[16 n + j][64 c + 32 s2 + 8 g .. + 7]  as one 16-byte word at
// word index ((c * NT + n) * 2 + s2) * 64 + 16 g + j: a wave's load is 1 KiB contiguous.
// That word is the B operand of one 16x16x32 MFMA (lane (g, j) supplies k = 8 g .. 8 g + 7
// of the 32 for token j); the A operand follows the same assignment of k to lanes.
#include <hip/hip_fp16.h>

#include "common.h"
#include "device_utils.h"

using namespace wgml;

namespace {

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr uint32_t KC = 64;    // elements of K per chunk
constexpr uint32_t KWAVES = 8;  // waves of a workgroup = ways K is split

struct GemmArgs {
    const uint8_t *p0, *p1, *p2, *p3;  // matrix planes (as wgml_qmat)
    const uint4 *xh;                   // packed f16 activations (see above)
    const float *xscale;               // [tpad] factor to multiply a token's results with
    float *out;                        // [T][out_stride]
    const float *bias;                 // optional, per row
    uint32_t nrows, ncols, kpad, T, tpad, out_stride;
    int accumulate;                    // out += result
};

__device__ __forceinline__ half4 to_half4(float a, float b, float c, float d) {
    half4 h;
    h[0] = (_Float16)a;
    h[1] = (_Float16)b;
    h[2] = (_Float16)c;
    h[3] = (_Float16)d;
    return h;
}

// ---- weight fragments -----------------------------------------------------------
// Lane (g, j) of a wave holds, for chunk c of row j of the tile, the 16 elements
//     k = 64 c + 32 s2 + 8 g + 4 e + i        (s2, e in 0..1, i in 0..3)
// load() fetches their bytes, frag() expands them as the reference's dequantize does
// (quantization.rs:29-42, 204-244, 322-389) and rounds to f16: a4[2 s2 + e][i].
struct GemmQ4K {
    struct Raw {
        uint4 hdr;  // d, dmin, 12 bytes of packed scales
        uint2 qs;   // bytes 8 g .. 8 g + 7 of the chunk's 32: low nibbles s2 = 0, high s2 = 1
    };
    __device__ static void load(Raw &r, const GemmArgs &a, uint32_t row, uint32_t chunk, uint32_t g) {
        const uint8_t *blk = a.p0 + ((size_t)row * (a.ncols / 256) + (chunk >> 2)) * 144;
        r.hdr = *reinterpret_cast<const uint4 *>(blk);
        r.qs = *reinterpret_cast<const uint2 *>(blk + 16 + (chunk & 3) * 32 + 8 * g);
    }
    __device__ static void frag(const Raw &r, const GemmArgs &, uint32_t chunk, uint32_t,
                                half4 (&a4)[4]) {
        const uint4 hdr = r.hdr;
        const uint32_t j = chunk & 3;
        const float d = f16_bits_to_f32((uint16_t)(hdr.x & 0xffffu));
        const float dmin = f16_bits_to_f32((uint16_t)(hdr.x >> 16));
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
        const float d1 = d * (float)s1, mm1 = dmin * (float)m1;
        const float d2 = d * (float)s2, mm2 = dmin * (float)m2;
        auto four = [&](uint32_t q, float dd, float mm) {
            return to_half4(dd * (float)(q & 15u) - mm, dd * (float)((q >> 8) & 15u) - mm,
                            dd * (float)((q >> 16) & 15u) - mm, dd * (float)((q >> 24) & 15u) - mm);
        };
        a4[0] = four(r.qs.x, d1, mm1);
        a4[1] = four(r.qs.y, d1, mm1);
        a4[2] = four(r.qs.x >> 4, d2, mm2);
        a4[3] = four(r.qs.y >> 4, d2, mm2);
    }
};

struct GemmQ6K {
    struct Raw {
        uint2 ql[2];  // per s2: 8 bytes of low nibbles
        uint2 qh;     // 8 bytes of high bit pairs
        uint32_t scw;  // the four scales of this 64-element chunk
        uint32_t d;
    };
    __device__ static void load(Raw &r, const GemmArgs &a, uint32_t row, uint32_t chunk, uint32_t g) {
        const size_t blk = (size_t)row * (a.ncols / 256) + (chunk >> 2);
        const uint32_t c = chunk & 3, i = c >> 1;
        const uint8_t *ql = a.p0 + blk * 128 + 64 * i + 8 * g;
        r.ql[0] = *reinterpret_cast<const uint2 *>(ql);
        r.ql[1] = *reinterpret_cast<const uint2 *>(ql + 32);
        r.qh = *reinterpret_cast<const uint2 *>(a.p1 + blk * 64 + 32 * i + 8 * g);
        r.scw = *reinterpret_cast<const uint32_t *>(a.p2 + blk * 16 + 8 * i + 4 * (c & 1));
        r.d = *reinterpret_cast<const uint16_t *>(a.p3 + blk * 2);
    }
    __device__ static void frag(const Raw &r, const GemmArgs &, uint32_t chunk, uint32_t g,
                                half4 (&a4)[4]) {
        // element e = 64 (c & 1) + 32 s2 + 8 g + b of the 128-element half: quarter
        // e / 32 = 2 (c & 1) + s2 picks the nibble (high for quarters 2, 3), the bit pair of
        // qh[8 g + b] (shift 2 * quarter) and the scale (8 g + b) / 16 + 2 * quarter
        const uint32_t hi_nib = chunk & 1;
        const float d = f16_bits_to_f32((uint16_t)r.d);
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            const float ds = d * (float)(int8_t)((r.scw >> (8 * ((g >> 1) + 2 * s2))) & 0xffu);
            const uint32_t hsh = 2 * (2 * hi_nib + s2);
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                uint32_t l = e ? r.ql[s2].y : r.ql[s2].x;
                if (hi_nib) l >>= 4;
                const uint32_t h = (e ? r.qh.y : r.qh.x) >> hsh;
                float v[4];
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const int q = (int)(((l >> (8 * b)) & 15u) | (((h >> (8 * b)) & 3u) << 4)) - 32;
                    v[b] = ds * (float)q;
                }
                a4[2 * s2 + e] = to_half4(v[0], v[1], v[2], v[3]);
            }
        }
    }
};

struct GemmQ8_0 {
    struct Raw {
        uint2 q[2];  // per s2 (= 32-element block of the chunk): 8 quants
        uint32_t d[2];
    };
    // rows are a multiple of 32 elements long: the second half of the last chunk may not
    // exist; it is then read from the first half and expanded to zeros
    __device__ static void load(Raw &r, const GemmArgs &a, uint32_t row, uint32_t chunk, uint32_t g) {
        const uint32_t b0 = chunk * 2, nb = a.ncols / 32;
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            const uint32_t b = min(b0 + s2, nb - 1);
            r.q[s2] = *reinterpret_cast<const uint2 *>(a.p0 + (size_t)row * a.ncols + b * 32 + 8 * g);
            r.d[s2] = *reinterpret_cast<const uint16_t *>(a.p1 + ((size_t)row * nb + b) * 2);
        }
    }
    __device__ static void frag(const Raw &r, const GemmArgs &a, uint32_t chunk, uint32_t,
                                half4 (&a4)[4]) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            const bool exists = chunk * 2 + s2 < a.ncols / 32;
            const float d = exists ? f16_bits_to_f32((uint16_t)r.d[s2]) : 0.f;
            const uint32_t x = exists ? r.q[s2].x : 0u, y = exists ? r.q[s2].y : 0u;
            a4[2 * s2] = to_half4(sb0(x) * d, sb1(x) * d, sb2(x) * d, sb3(x) * d);
            a4[2 * s2 + 1] = to_half4(sb0(y) * d, sb1(y) * d, sb2(y) * d, sb3(y) * d);
        }
    }
};

template <class F, int NT, int RB>
__global__ __launch_bounds__(KWAVES * 64) void gemm_quant_f16_kernel(const GemmArgs a) {
    extern __shared__ float4 red[];  // [KWAVES][NT][64]
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t j = lane & 15, g = lane >> 4;
    const uint32_t row0 = blockIdx.x * (16 * RB);
    uint32_t row[RB];  // this lane's rows of the A operands
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) row[rb] = min(row0 + 16 * rb + j, a.nrows - 1);
    const uint32_t nchunks = a.kpad / KC;
    // chunks of this wave: wave, wave + 8, ...
    const uint32_t n_my = nchunks > wave ? (nchunks - wave + KWAVES - 1) / KWAVES : 0;

    floatx4 acc[RB][NT];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[rb][n] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    // Every load is unconditional (a chunk number past the end re-reads the last chunk and
    // is never multiplied): the compiler can then count outstanding loads exactly instead
    // of draining them all before each use.  The weight bytes of the next chunk are
    // requested when a chunk's arithmetic starts; each activation word of the next chunk
    // is requested into the register of the one it replaces right after that one's last use.
    typename F::Raw ra[RB], rb_[RB];
    uint4 b[NT][2];
    auto chunk_of = [&](uint32_t i) { return min(wave + KWAVES * i, nchunks - 1); };
    auto load_a = [&](typename F::Raw(&r)[RB], uint32_t i) {
        const uint32_t c = chunk_of(i);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) F::load(r[rb], a, row[rb], c, g);
    };
    auto compute = [&](const typename F::Raw(&r)[RB], uint32_t i) {
        const uint32_t c = wave + KWAVES * i;
        const uint4 *next = a.xh + (size_t)chunk_of(i + 1) * NT * 128 + lane;
        half4 a4[RB][4];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) F::frag(r[rb], a, c, g, a4[rb]);
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                half8 bw;
                __builtin_memcpy(&bw, &b[n][s2], 16);
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    half8 aw;
                    __builtin_memcpy(&aw, &a4[rb][2 * s2], 16);  // a4[2 s2], a4[2 s2 + 1]: 8 consecutive k
                    acc[rb][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aw, bw, acc[rb][n], 0, 0, 0);
                }
                b[n][s2] = next[(n * 2 + s2) * 64];
            }
        }
    };
    if (n_my > 0) {
        load_a(ra, 0);
        {
            const uint4 *first = a.xh + (size_t)chunk_of(0) * NT * 128 + lane;
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
#pragma unroll
                for (int n = 0; n < NT; ++n) b[n][s2] = first[(n * 2 + s2) * 64];
            }
        }
        for (uint32_t i = 0; i < n_my; i += 2) {
            load_a(rb_, i + 1);
            compute(ra, i);
            if (i + 1 < n_my) {
                load_a(ra, i + 2);
                compute(rb_, i + 1);
            }
        }
    }
    // the partial sums of the 8 waves, added in wave order, one row block at a time
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        if (rb > 0) __syncthreads();
#pragma unroll
        for (int n = 0; n < NT; ++n)
            red[(wave * NT + n) * 64 + lane] =
                make_float4(acc[rb][n][0], acc[rb][n][1], acc[rb][n][2], acc[rb][n][3]);
        __syncthreads();
        for (uint32_t idx = tid; idx < NT * 64; idx += KWAVES * 64) {
            const uint32_t n = idx >> 6, l = idx & 63;
            float4 v = red[n * 64 + l];
#pragma unroll
            for (uint32_t w = 1; w < KWAVES; ++w) {
                const float4 p = red[(w * NT + n) * 64 + l];
                v = make_float4(v.x + p.x, v.y + p.y, v.z + p.z, v.w + p.w);
            }
            // v = out[token 16 n + (l & 15)][first row of the block + 4 (l >> 4) .. + 3]
            const uint32_t tok = n * 16 + (l & 15), r4 = row0 + 16 * rb + 4 * (l >> 4);
            if (tok >= a.T || r4 >= a.nrows) continue;
            const float xs_t = a.xscale ? a.xscale[tok] : 1.f;
            v = make_float4(v.x * xs_t, v.y * xs_t, v.z * xs_t, v.w * xs_t);
            float *o = a.out + (size_t)tok * a.out_stride + r4;
            if (r4 + 3 < a.nrows && (reinterpret_cast<uintptr_t>(o) & 15u) == 0) {
                if (a.bias) {
                    v.x += a.bias[r4];
                    v.y += a.bias[r4 + 1];
                    v.z += a.bias[r4 + 2];
                    v.w += a.bias[r4 + 3];
                }
                if (a.accumulate) {
                    const float4 p = *reinterpret_cast<const float4 *>(o);
                    v = make_float4(p.x + v.x, p.y + v.y, p.z + v.z, p.w + v.w);
                }
                *reinterpret_cast<float4 *>(o) = v;
                continue;
            }
            const float vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (r4 + i < a.nrows) {
                    float e = vv[i];
                    if (a.bias) e += a.bias[r4 + i];
                    o[i] = a.accumulate ? o[i] + e : e;
                }
            }
        }
    }
}

// One workgroup per token: X[t] (fp32, optionally RMS-normalised with weights w as
// the reference does: (x * rsqrt(mean(x^2) + eps)) * w, ops/rms_norm.rs:55-63) -> f16
// in the packed order described at the top, divided by a power of two if needed so that
// |x| <= 1024; the factor to undo it goes to xscale[t].  Tokens from T on and columns
// from K on are zero.  With `up` non-null the input is the gated activation
// up[k] * silu(x[k]) (ops/silu.wgsl:13-27) instead of x itself (no normalisation then).
constexpr int PREP_THREADS = 1024;
constexpr int PREP_GROUPS = 2;  // groups of 8 columns a thread keeps in registers
__global__ __launch_bounds__(PREP_THREADS) void prep_x_kernel(const float *__restrict__ x, uint32_t x_stride,
                                                     const float *__restrict__ up,
                                                     const float *__restrict__ norm_w, float eps,
                                                     uint4 *__restrict__ xh,
                                                     float *__restrict__ xscale, uint32_t K,
                                                     uint32_t kpad, uint32_t T) {
    __shared__ float red[16];
    const uint32_t t = blockIdx.x, tid = threadIdx.x, nt = gridDim.x / 16;
    // 16-byte word of (token t, columns 8 k8 .. 8 k8 + 7)
    auto word = [&](uint32_t k8) -> uint4 & {
        const uint32_t c = k8 >> 3, s2 = (k8 >> 2) & 1, g = k8 & 3;
        return xh[(((size_t)c * nt + (t >> 4)) * 2 + s2) * 64 + 16 * g + (t & 15)];
    };
    const uint32_t ngroups = kpad / 8;
    if (t >= T) {
        for (uint32_t k8 = tid; k8 < ngroups; k8 += PREP_THREADS) word(k8) = make_uint4(0, 0, 0, 0);
        if (tid == 0) xscale[t] = 0.f;
        return;
    }
    const float *xr = x + (size_t)t * x_stride;
    const float *ur = up ? up + (size_t)t * x_stride : nullptr;
    // Rows of up to 8 * PREP_GROUPS * PREP_THREADS columns are read once and kept in
    // registers (v); longer rows are re-read from memory by the later passes.
    const bool cached = ngroups <= PREP_GROUPS * PREP_THREADS;
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
            for (int e = 0; e < 8; ++e) v[i][e] = k0 + e < kpad ? raw(k0 + e) : 0.f;
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
    auto store = [&](uint32_t k8, const float(&f)[8]) {
        _Float16 h[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) h[e] = (_Float16)(f[e] * down);
        uint4 w;
        __builtin_memcpy(&w, h, 16);
        word(k8) = w;
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
    {
        const float x = qt[a], y = qt[b];
        qt[a] = cs * x - sn * y;
        qt[b] = sn * x + cs * y;
    }
    if (i * 2 < kv_dim) {
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

int g_force_row_blocks = 0;  // 0: by matrix height; 1 or 2: forced (tests)

template <class F, int RB>
int launch_gemm_rb(wgml_ctx *ctx, const GemmArgs &a) {
    const uint32_t nt = a.tpad / 16;  // token blocks: 1, 2, 4 or 8
    const dim3 grid((a.nrows + 16 * RB - 1) / (16 * RB)), block(KWAVES * 64);
    const size_t lds = (size_t)KWAVES * nt * 64 * sizeof(float4);
    switch (nt) {
    case 8: gemm_quant_f16_kernel<F, 8, RB><<<grid, block, lds, ctx->stream>>>(a); break;
    case 4: gemm_quant_f16_kernel<F, 4, RB><<<grid, block, lds, ctx->stream>>>(a); break;
    case 2: gemm_quant_f16_kernel<F, 2, RB><<<grid, block, lds, ctx->stream>>>(a); break;
    default: gemm_quant_f16_kernel<F, 1, RB><<<grid, block, lds, ctx->stream>>>(a); break;
    }
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

// Two row blocks per wave halve the activation traffic per product (each activation word
// serves 32 rows) at the price of half as many workgroups: worth it once those still
// cover half of the compute units.
template <class F>
int launch_gemm_fmt(wgml_ctx *ctx, const GemmArgs &a) {
    const uint32_t cu = ctx->n_cu > 0 ? (uint32_t)ctx->n_cu : 256u;
    const bool two = g_force_row_blocks ? g_force_row_blocks == 2 : a.nrows / 32 >= cu / 2;
    return two ? launch_gemm_rb<F, 2>(ctx, a) : launch_gemm_rb<F, 1>(ctx, a);
}

}  // namespace

namespace wgml {

uint32_t prefill_tpad(uint32_t T) { return T <= 16 ? 16 : T <= 32 ? 32 : T <= 64 ? 64 : 128; }
uint32_t prefill_kpad(uint32_t K) { return (K + KC - 1) / KC * KC; }

int ensure_prefill_scratch(wgml_ctx *ctx, size_t xh_bytes) {
    if (!ctx->prefill_xscale)
        WGML_CHECK_HIP(hipMalloc((void **)&ctx->prefill_xscale, kPrefillMaxTokens * sizeof(float)));
    if (xh_bytes <= ctx->prefill_xh_bytes) return WGML_OK;
    // work already enqueued may still read the old buffer: retire it, free with the context
    if (ctx->prefill_xh) ctx->retired.push_back(ctx->prefill_xh);
    ctx->prefill_xh = nullptr;
    ctx->prefill_xh_bytes = 0;
    WGML_CHECK_HIP(hipMalloc(&ctx->prefill_xh, xh_bytes));
    ctx->prefill_xh_bytes = xh_bytes;
    return WGML_OK;
}

int launch_prefill_prep(wgml_ctx *ctx, const float *x, uint32_t x_stride, const float *up,
                        const float *norm_w, float eps, void *xh, float *xscale, uint32_t K,
                        uint32_t T) {
    prep_x_kernel<<<dim3(prefill_tpad(T)), dim3(PREP_THREADS), 0, ctx->stream>>>(
        x, x_stride, up, norm_w, eps, reinterpret_cast<uint4 *>(xh), xscale, K, prefill_kpad(K), T);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

int launch_gemm_quant(wgml_ctx *ctx, float *out, uint32_t out_stride, const wgml_qmat *m,
                      const void *xh, const float *xscale, uint32_t T, const float *bias,
                      int accumulate) {
    if (T == 0 || T > kPrefillMaxTokens)
        return set_error(WGML_E_INVALID, "gemm_quant: %u tokens (1..%u)", T, kPrefillMaxTokens);
    GemmArgs a{};
    a.p0 = m->p0;
    a.p1 = m->p1;
    a.p2 = m->p2;
    a.p3 = m->p3;
    a.xh = reinterpret_cast<const uint4 *>(xh);
    a.xscale = xscale;
    a.out = out;
    a.bias = bias;
    a.nrows = m->nrows;
    a.ncols = m->ncols;
    a.kpad = prefill_kpad(m->ncols);
    a.T = T;
    a.tpad = prefill_tpad(T);
    a.out_stride = out_stride;
    a.accumulate = accumulate;
    switch (m->type) {
    case WGML_Q4_K: return launch_gemm_fmt<GemmQ4K>(ctx, a);
    case WGML_Q6_K: return launch_gemm_fmt<GemmQ6K>(ctx, a);
    case WGML_Q8_0: return launch_gemm_fmt<GemmQ8_0>(ctx, a);
    default:
        return set_error(WGML_E_UNSUPPORTED, "gemm_quant: matrix type %d (Q8_0, Q4_K, Q6_K only)",
                         m->type);
    }
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

// Test hook: 0 = choose rows per workgroup by matrix height, 1 = 16 rows, 2 = 32 rows.
WGML_API int wgml_debug_set_gemm_row_blocks(int n) {
    g_force_row_blocks = n == 1 || n == 2 ? n : 0;
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
    WGML_TRY(launch_prefill_prep(ctx, view_ptr(x), m->ncols, nullptr, nullptr, 0.f, ctx->prefill_xh,
                                 ctx->prefill_xscale, m->ncols, n_tokens));
    return launch_gemm_quant(ctx, view_ptr(out), m->nrows, m, ctx->prefill_xh, ctx->prefill_xscale,
                             n_tokens, nullptr, 0);
}

}  // extern "C"
