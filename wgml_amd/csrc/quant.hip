// Quantized matrices on the device: GGUF block layouts (quantization.rs:29-42,
// 204-244, 322-389 of the reference), their re-layout into aligned planes, and
// the bit-exact dequantization kernels.
//
// This file must be compiled with -ffp-contract=off: the reference's CPU
// dequantizers round every product and difference separately
// (quantization.rs:233-236, 366, 370) and the kernels below must match them bit
// for bit.
#include "common.h"
#include "device_utils.h"

using namespace wgml;

namespace {

constexpr uint32_t QK8_0 = 32, QK_K = 256;
constexpr uint32_t Q8_0_BYTES = 34, Q4_K_BYTES = 144, Q6_K_BYTES = 210;

inline uint64_t align256(uint64_t v) { return (v + 255) & ~uint64_t(255); }

// ---- re-layout kernels (run once per matrix at load) ------------------------

// raw: nblocks x {u16 d; i8 qs[32]} (2-byte aligned) -> qs plane + d plane.
__global__ void repack_q8_0(const uint16_t *__restrict__ raw, uint32_t *__restrict__ qs,
                            uint16_t *__restrict__ d, uint64_t nblocks) {
    uint64_t b = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const uint16_t *src = raw + b * 17;
    d[b] = src[0];
    uint32_t *dst = qs + b * 8;
#pragma unroll
    for (int k = 0; k < 8; ++k) dst[k] = (uint32_t)src[1 + 2 * k] | ((uint32_t)src[2 + 2 * k] << 16);
}

// raw: nblocks x {u8 ql[128]; u8 qh[64]; i8 scales[16]; u16 d} (2-byte aligned).
__global__ void repack_q6_k(const uint16_t *__restrict__ raw, uint16_t *__restrict__ ql,
                            uint16_t *__restrict__ qh, uint16_t *__restrict__ sc,
                            uint16_t *__restrict__ d, uint64_t nblocks) {
    // One wave-quarter (16 lanes) would be enough; keep it simple: 105 halfwords
    // per block, one thread per halfword.
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t b = i / 105;
    uint32_t h = (uint32_t)(i % 105);
    if (b >= nblocks) return;
    uint16_t v = raw[b * 105 + h];
    if (h < 64) ql[b * 64 + h] = v;
    else if (h < 96) qh[b * 32 + (h - 64)] = v;
    else if (h < 104) sc[b * 8 + (h - 96)] = v;
    else d[b] = v;
}

// ---- largest weight magnitude (computed once per matrix at load) --------------
// An upper bound on |w| over the dequantized matrix: Q8_0 and Q8_K |d| max|q| (exact); Q4_K and
// Q5_K max(|dmin m|, |d sc 15 (31) - dmin m|) per sub-block (the two ends of the quant range);
// Q6_K |d| |scale| 32 per sub-block; the 32-element blocks the ends of their ranges likewise.  The batched
// products expand weights into f16 times 2^8 and need it within 255.875.  NaN / inf scales give
// inf.  Non-negative floats order like their bit patterns, so the maximum is an atomicMax on
// the bits.
__device__ __forceinline__ float nan_to_inf(float v) { return v == v ? v : INFINITY; }

__global__ void max_abs_kernel(int type, const uint8_t *__restrict__ p0,
                               const uint8_t *__restrict__ p1, const uint8_t *__restrict__ p2,
                               const uint8_t *__restrict__ p3, uint64_t nblocks,
                               uint32_t *__restrict__ out_bits) {
    float best = 0.f;
    for (uint64_t b = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; b < nblocks;
         b += (uint64_t)gridDim.x * blockDim.x) {
        float v = 0.f;
        if (type == WGML_Q8_0) {
            const int8_t *q = reinterpret_cast<const int8_t *>(p0) + b * 32;
            int m = 0;
            for (int k = 0; k < 32; ++k) m = max(m, abs((int)q[k]));
            v = fabsf(f16_bits_to_f32(reinterpret_cast<const uint16_t *>(p1)[b])) * (float)m;
        } else if (type == WGML_Q4_K) {
            const uint8_t *blk = p0 + b * Q4_K_BYTES;
            const float d = f16_bits_to_f32(*(const uint16_t *)(blk + 0));
            const float dmin = f16_bits_to_f32(*(const uint16_t *)(blk + 2));
            for (uint32_t j = 0; j < 8; ++j) {
                uint8_t sc, m;
                get_scale_min_k4(j, blk + 4, sc, m);
                // w = d sc q - dmin m is linear in q = 0..15: the extremes are its ends.  A term
                // with a zero factor counts as zero even when the other factor is inf.
                const float a = sc ? d * (float)sc * 15.f : 0.f, c = m ? dmin * (float)m : 0.f;
                v = fmaxf(v, fmaxf(nan_to_inf(fabsf(c)), nan_to_inf(fabsf(a - c))));
            }
        } else if (type == WGML_Q6_K) {
            const float d = fabsf(f16_bits_to_f32(reinterpret_cast<const uint16_t *>(p3)[b]));
            const int8_t *sc = reinterpret_cast<const int8_t *>(p2) + b * 16;
            int m = 0;
            for (int k = 0; k < 16; ++k) m = max(m, abs((int)sc[k]));
            v = m ? d * (float)m * 32.f : 0.f;
        } else if (type == WGML_Q5_K) {  // as Q4_K with quants 0..31
            const uint8_t *blk = p0 + b * 176;
            const float d = f16_bits_to_f32(*(const uint16_t *)(blk + 0));
            const float dmin = f16_bits_to_f32(*(const uint16_t *)(blk + 2));
            for (uint32_t j = 0; j < 8; ++j) {
                uint8_t sc, m;
                get_scale_min_k4(j, blk + 4, sc, m);
                const float a = sc ? d * (float)sc * 31.f : 0.f, c = m ? dmin * (float)m : 0.f;
                v = fmaxf(v, fmaxf(nan_to_inf(fabsf(c)), nan_to_inf(fabsf(a - c))));
            }
        } else if (type == WGML_Q8_K) {
            const uint8_t *blk = p0 + b * 292;
            float d;
            __builtin_memcpy(&d, blk, 4);
            const int8_t *q = reinterpret_cast<const int8_t *>(blk + 4);
            int m = 0;
            for (int k = 0; k < 256; ++k) m = max(m, abs((int)q[k]));
            v = m ? fabsf(d) * (float)m : 0.f;
        } else {  // the 32-element blocks: y = d (q - 8), d q + m, d (q - 16), d q + m
            const bool has_m = type == WGML_Q4_1 || type == WGML_Q5_1;
            const bool has_qh = type == WGML_Q5_0 || type == WGML_Q5_1;
            const uint32_t bytes = 18 + (has_m ? 2 : 0) + (has_qh ? 4 : 0);
            const uint8_t *blk = p0 + b * bytes;
            uint16_t db, mb = 0;
            __builtin_memcpy(&db, blk, 2);
            if (has_m) __builtin_memcpy(&mb, blk + 2, 2);
            const float d = f16_bits_to_f32(db), m = f16_bits_to_f32(mb);
            const float top = has_qh ? 31.f : 15.f;
            if (has_m) v = fmaxf(nan_to_inf(fabsf(m)), nan_to_inf(fabsf(d * top + m)));
            else v = fabsf(d) * (has_qh ? 16.f : 8.f);
        }
        best = fmaxf(best, nan_to_inf(v));
    }
    best = wave_max(best);
    if ((threadIdx.x & 63) == 0) atomicMax(out_bits, __float_as_uint(best));
}

// ---- dequantization kernels ---------------------------------------------------

// quantization.rs:38-41
__global__ void dequant_q8_0(const int8_t *__restrict__ qs, const uint16_t *__restrict__ d,
                             float *__restrict__ out, uint64_t n) {
    uint64_t e = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n) return;
    float scale = f16_bits_to_f32(d[e / QK8_0]);
    out[e] = (float)qs[e] * scale;
}

// quantization.rs:347-389; one thread per byte of qs (two outputs).
__global__ void dequant_q4_k(const uint8_t *__restrict__ blocks, float *__restrict__ out,
                             uint64_t nblocks) {
    uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t b = t / 128;
    uint32_t l = (uint32_t)(t % 128);  // byte index in qs
    if (b >= nblocks) return;
    const uint8_t *blk = blocks + b * Q4_K_BYTES;
    float d = f16_bits_to_f32(*(const uint16_t *)(blk + 0));
    float dmin = f16_bits_to_f32(*(const uint16_t *)(blk + 2));
    const uint8_t *scales = blk + 4;
    uint32_t j = l / 32;  // 64-element group
    uint8_t sc1, m1, sc2, m2;
    get_scale_min_k4(2 * j, scales, sc1, m1);
    get_scale_min_k4(2 * j + 1, scales, sc2, m2);
    float d1 = d * (float)sc1, mm1 = dmin * (float)m1;
    float d2 = d * (float)sc2, mm2 = dmin * (float)m2;
    uint8_t q = blk[16 + l];
    float *o = out + b * QK_K + j * 64 + (l % 32);
    o[0] = d1 * (float)(q & 0xF) - mm1;
    o[32] = d2 * (float)(q >> 4) - mm2;
}

// quantization.rs:214-243; one thread per (block, half i, l): four outputs.
__global__ void dequant_q6_k(const uint8_t *__restrict__ ql, const uint8_t *__restrict__ qh,
                             const int8_t *__restrict__ sc, const uint16_t *__restrict__ dd,
                             float *__restrict__ out, uint64_t nblocks) {
    uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t b = t / 64;
    uint32_t i = (uint32_t)(t % 64) / 32, l = (uint32_t)(t % 32);
    if (b >= nblocks) return;
    float d = f16_bits_to_f32(dd[b]);
    uint32_t is = l / 16;
    uint8_t ql0 = ql[b * 128 + i * 64 + l], ql32 = ql[b * 128 + i * 64 + l + 32];
    uint8_t h = qh[b * 64 + i * 32 + l];
    int q1 = (int)((ql0 & 0xF) | (((h >> 0) & 3) << 4)) - 32;
    int q2 = (int)((ql32 & 0xF) | (((h >> 2) & 3) << 4)) - 32;
    int q3 = (int)((ql0 >> 4) | (((h >> 4) & 3) << 4)) - 32;
    int q4 = (int)((ql32 >> 4) | (((h >> 6) & 3) << 4)) - 32;
    const int8_t *s = sc + b * 16 + i * 8 + is;
    float *o = out + b * QK_K + i * 128 + l;
    o[0] = d * (float)s[0] * (float)q1;
    o[32] = d * (float)s[2] * (float)q2;
    o[64] = d * (float)s[4] * (float)q3;
    o[96] = d * (float)s[6] * (float)q4;
}

// quantization.rs:16-24
__global__ void f16_to_f32_kernel(const uint16_t *__restrict__ in, float *__restrict__ out,
                                  uint32_t n) {
    uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = f16_bits_to_f32(in[i]);
}

// ---- formats that the reference expands to f32 at load ----------------------
// GgufTensorData::to_gpu_matrix (gguf.rs:131-184) keeps Q8_0 / Q4_K / Q6_K
// quantized and dequantizes everything else; these kernels do that expansion on
// the device from the raw GGUF bytes (one thread per element; byte loads, the
// blocks are only 2-byte aligned).  Arithmetic as Block*::dequantize
// (quantization.rs:16-24, 53-68, 82-98, 112-131, 146-167, 195-201, 274-317).
__device__ __forceinline__ uint16_t ld_u16(const uint8_t *p) {
    return (uint16_t)(p[0] | ((uint16_t)p[1] << 8));
}
__device__ __forceinline__ uint32_t ld_u32(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

template <int TYPE>
__global__ void dequant_raw_kernel(const uint8_t *__restrict__ raw, float *__restrict__ out,
                                   uint64_t n) {
    const uint64_t e = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n) return;
    if (TYPE == WGML_F16) {
        out[e] = f16_bits_to_f32(ld_u16(raw + e * 2));
    } else if (TYPE == WGML_Q4_0 || TYPE == WGML_Q4_1 || TYPE == WGML_Q5_0 || TYPE == WGML_Q5_1) {
        constexpr int BYTES = TYPE == WGML_Q4_0 ? 18 : TYPE == WGML_Q4_1 ? 20 : TYPE == WGML_Q5_0 ? 22 : 24;
        constexpr bool HAS_M = TYPE == WGML_Q4_1 || TYPE == WGML_Q5_1;
        constexpr bool HAS_QH = TYPE == WGML_Q5_0 || TYPE == WGML_Q5_1;
        const uint8_t *b = raw + (e / 32) * BYTES;
        const uint32_t k = (uint32_t)(e % 32), j = k & 15;
        const float d = f16_bits_to_f32(ld_u16(b));
        const uint8_t *qs = b + 2 + (HAS_M ? 2 : 0) + (HAS_QH ? 4 : 0);
        uint32_t x = k < 16 ? (qs[j] & 0x0Fu) : (uint32_t)(qs[j] >> 4);
        if (HAS_QH) {
            const uint32_t qh = ld_u32(b + 2 + (HAS_M ? 2 : 0));
            x |= k < 16 ? ((qh >> j) << 4) & 0x10u : (qh >> (j + 12)) & 0x10u;
        }
        if (HAS_M) {
            const float m = f16_bits_to_f32(ld_u16(b + 2));
            out[e] = (float)x * d + m;
        } else {
            out[e] = (float)((int)x - (HAS_QH ? 16 : 8)) * d;
        }
    } else if (TYPE == WGML_Q8_K) {
        const uint8_t *b = raw + (e / QK_K) * 292;
        const float d = __uint_as_float(ld_u32(b));
        out[e] = d * (float)(int8_t)b[4 + e % QK_K];
    } else if (TYPE == WGML_Q5_K) {
        const uint8_t *b = raw + (e / QK_K) * 176;
        const uint32_t k = (uint32_t)(e % QK_K), sub = k >> 5, l = k & 31;  // 8 sub-blocks of 32
        const float d = f16_bits_to_f32(ld_u16(b)), dmin = f16_bits_to_f32(ld_u16(b + 2));
        uint8_t sc, mn;
        get_scale_min_k4(sub, b + 4, sc, mn);
        const uint8_t q = b[48 + (sub >> 1) * 32 + l];
        const uint32_t nib = (sub & 1) ? (uint32_t)(q >> 4) : (q & 0x0Fu);
        const uint32_t x = nib + ((b[16 + l] >> sub) & 1u) * 16u;
        out[e] = (d * (float)sc) * (float)x - dmin * (float)mn;
    }
}

// True for the formats expanded to f32 at load: F16 only, as GgufTensorData::to_gpu_matrix
// does (gguf.rs:131-184: every block format stays quantized on the GPU).
bool expands_to_f32(int type) { return type == WGML_F16; }

// Block formats whose bytes stay exactly as in the GGUF file (no re-layout).
bool kept_raw(int type) {
    return type == WGML_F32 || type == WGML_Q4_K || type == WGML_Q4_0 || type == WGML_Q4_1 ||
           type == WGML_Q5_0 || type == WGML_Q5_1 || type == WGML_Q5_K || type == WGML_Q8_K;
}

uint32_t block_elems(int type) {
    switch (type) {
    case WGML_F32: case WGML_F16: return 1;
    case WGML_Q4_0: case WGML_Q4_1: case WGML_Q5_0: case WGML_Q5_1: return 32;
    case WGML_Q8_0: return QK8_0;
    case WGML_Q4_K: case WGML_Q5_K: case WGML_Q6_K: case WGML_Q8_K: return QK_K;
    default: return 0;
    }
}

uint32_t block_bytes(int type) {
    switch (type) {
    case WGML_F32: return 4;
    case WGML_F16: return 2;
    case WGML_Q4_0: return 18;
    case WGML_Q4_1: return 20;
    case WGML_Q5_0: return 22;
    case WGML_Q5_1: return 24;
    case WGML_Q8_0: return Q8_0_BYTES;
    case WGML_Q4_K: return Q4_K_BYTES;
    case WGML_Q5_K: return 176;
    case WGML_Q6_K: return Q6_K_BYTES;
    case WGML_Q8_K: return 292;
    default: return 0;
    }
}

}  // namespace

namespace wgml {

int launch_dequantize(wgml_ctx *ctx, float *out, const wgml_qmat *m) {
    uint64_t n = (uint64_t)m->nrows * m->ncols;
    const int T = 256;
    switch (m->type) {
    case WGML_F32:
        WGML_CHECK_HIP(hipMemcpyAsync(out, m->p0, n * 4, hipMemcpyDeviceToDevice, ctx->stream));
        break;
    case WGML_Q8_0:
        dequant_q8_0<<<dim3((unsigned)((n + T - 1) / T)), dim3(T), 0, ctx->stream>>>(
            (const int8_t *)m->p0, (const uint16_t *)m->p1, out, n);
        break;
    case WGML_Q4_K: {
        uint64_t nb = n / QK_K, nt = nb * 128;
        dequant_q4_k<<<dim3((unsigned)((nt + T - 1) / T)), dim3(T), 0, ctx->stream>>>(m->p0, out,
                                                                                      nb);
        break;
    }
    case WGML_Q6_K: {
        uint64_t nb = n / QK_K, nt = nb * 64;
        dequant_q6_k<<<dim3((unsigned)((nt + T - 1) / T)), dim3(T), 0, ctx->stream>>>(
            m->p0, m->p1, (const int8_t *)m->p2, (const uint16_t *)m->p3, out, nb);
        break;
    }
    case WGML_Q4_0: case WGML_Q4_1: case WGML_Q5_0: case WGML_Q5_1: case WGML_Q5_K: case WGML_Q8_K: {
        const dim3 g((unsigned)((n + T - 1) / T)), b(T);
        switch (m->type) {
        case WGML_Q4_0: dequant_raw_kernel<WGML_Q4_0><<<g, b, 0, ctx->stream>>>(m->p0, out, n); break;
        case WGML_Q4_1: dequant_raw_kernel<WGML_Q4_1><<<g, b, 0, ctx->stream>>>(m->p0, out, n); break;
        case WGML_Q5_0: dequant_raw_kernel<WGML_Q5_0><<<g, b, 0, ctx->stream>>>(m->p0, out, n); break;
        case WGML_Q5_1: dequant_raw_kernel<WGML_Q5_1><<<g, b, 0, ctx->stream>>>(m->p0, out, n); break;
        case WGML_Q5_K: dequant_raw_kernel<WGML_Q5_K><<<g, b, 0, ctx->stream>>>(m->p0, out, n); break;
        default: dequant_raw_kernel<WGML_Q8_K><<<g, b, 0, ctx->stream>>>(m->p0, out, n); break;
        }
        break;
    }
    default: return set_error(WGML_E_UNSUPPORTED, "dequantize: unsupported type %d", m->type);
    }
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

}  // namespace wgml

extern "C" {

uint32_t wgml_quant_block_elems(int type) { return block_elems(type); }

uint64_t wgml_quant_bytes(int type, uint64_t nelems) {
    uint32_t be = block_elems(type);
    if (!be || nelems % be) return 0;
    return nelems / be * block_bytes(type);
}

int wgml_quant_matrix_create(wgml_ctx *ctx, int type, uint32_t nrows, uint32_t ncols,
                             const void *gguf_bytes, wgml_qmat **out) {
    WGML_REQUIRE(ctx && out && gguf_bytes, "wgml_quant_matrix_create: null argument");
    *out = nullptr;
    uint32_t be = block_elems(type);
    if (!be)
        return set_error(WGML_E_UNSUPPORTED,
                         "wgml_quant_matrix_create: quantization type %d is not supported "
                         "(F32, Q8_0, Q4_0, Q4_1, Q5_0, Q5_1, Q4_K, Q5_K, Q6_K, Q8_K; F16 is "
                         "expanded to f32)",
                         type);
    WGML_REQUIRE(nrows > 0 && ncols > 0, "wgml_quant_matrix_create: empty matrix %ux%u", nrows,
                 ncols);
    WGML_REQUIRE(ncols % be == 0,
                 "wgml_quant_matrix_create: ncols %u is not a multiple of the block length %u",
                 ncols, be);
    // x is staged as float4; every quantized block length is a multiple of 4, f32 needs it too.
    WGML_REQUIRE(ncols % 4 == 0, "wgml_quant_matrix_create: ncols %u must be a multiple of 4",
                 ncols);
    uint64_t nelem = (uint64_t)nrows * ncols;
    uint64_t nblocks = nelem / be;
    uint64_t gguf = nblocks * block_bytes(type);

    const bool expand = expands_to_f32(type);
    wgml_qmat *m = new wgml_qmat();
    m->ctx = ctx;
    ctx_retain(ctx);
    m->type = expand ? (int)WGML_F32 : type;
    m->nrows = nrows;
    m->ncols = ncols;
    m->gguf_bytes = expand ? nelem * 4 : gguf;  // what a GEMV over this matrix streams

    uint64_t o1 = 0, o2 = 0, o3 = 0, total = 0;
    if (expand) total = align256(nelem * 4);
    switch (expand ? -1 : type) {
    case WGML_F32: case WGML_Q4_K: case WGML_Q4_0: case WGML_Q4_1: case WGML_Q5_0: case WGML_Q5_1:
    case WGML_Q5_K: case WGML_Q8_K:
        total = align256(gguf);
        break;
    case WGML_Q8_0:
        o1 = align256(nblocks * 32);
        total = o1 + align256(nblocks * 2);
        break;
    case WGML_Q6_K:
        o1 = align256(nblocks * 128);
        o2 = o1 + align256(nblocks * 64);
        o3 = o2 + align256(nblocks * 16);
        total = o3 + align256(nblocks * 2);
        break;
    }
    // 256 spare bytes so that whole-wave 16-byte loads of a partly filled last
    // tile never leave the allocation.
    total += 256;
    hipError_t e = hipMalloc((void **)&m->base, total);
    if (e != hipSuccess) {
        ctx_release(ctx);
        delete m;
        return set_error(WGML_E_OOM, "wgml_quant_matrix_create: hipMalloc(%llu) failed: %s",
                         (unsigned long long)total, hipGetErrorString(e));
    }
    m->alloc_bytes = total;
    m->p0 = m->base;
    m->p1 = m->base + o1;
    m->p2 = m->base + o2;
    m->p3 = m->base + o3;

    auto fail = [&](hipError_t err, const char *what) {
        (void)hipFree(m->base);
        ctx_release(ctx);
        delete m;
        return set_error(WGML_E_HIP, "wgml_quant_matrix_create: %s: %s", what,
                         hipGetErrorString(err));
    };

    if (kept_raw(type)) {
        e = hipMemcpyAsync(m->base, gguf_bytes, gguf, hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) return fail(e, "upload");
    } else {
        uint8_t *raw = nullptr;
        e = hipMalloc((void **)&raw, gguf);
        if (e != hipSuccess) return fail(e, "staging hipMalloc");
        e = hipMemcpyAsync(raw, gguf_bytes, gguf, hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess) {
            const int T = 256;
            if (type == WGML_Q8_0) {
                repack_q8_0<<<dim3((unsigned)((nblocks + T - 1) / T)), dim3(T), 0, ctx->stream>>>(
                    (const uint16_t *)raw, (uint32_t *)m->p0, (uint16_t *)m->p1, nblocks);
            } else if (expand) {  // F16
                dequant_raw_kernel<WGML_F16><<<dim3((unsigned)((nelem + T - 1) / T)), dim3(T), 0,
                                               ctx->stream>>>(raw, reinterpret_cast<float *>(m->p0), nelem);
            } else {
                uint64_t nt = nblocks * 105;
                repack_q6_k<<<dim3((unsigned)((nt + T - 1) / T)), dim3(T), 0, ctx->stream>>>(
                    (const uint16_t *)raw, (uint16_t *)m->p0, (uint16_t *)m->p1,
                    (uint16_t *)m->p2, (uint16_t *)m->p3, nblocks);
            }
            e = hipGetLastError();
        }
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        (void)hipFree(raw);
        if (e != hipSuccess) return fail(e, "re-layout");
    }
    if (block_bytes(type) && type != WGML_F16 && type != WGML_F32) {
        // the formats the batched products take: bound their largest weight once
        uint32_t *bits = ctx->d_scalar + 8;
        e = hipMemsetAsync(bits, 0, 4, ctx->stream);
        if (e == hipSuccess) {
            const uint64_t want = (nblocks + 255) / 256;
            max_abs_kernel<<<dim3((unsigned)(want < 2048 ? want : 2048)), dim3(256), 0, ctx->stream>>>(
                type, m->p0, m->p1, m->p2, m->p3, nblocks, bits);
            e = hipGetLastError();
        }
        if (e == hipSuccess)
            e = hipMemcpyAsync(ctx->h_scalar + 8, bits, 4, hipMemcpyDeviceToHost, ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) return fail(e, "weight bound");
        memcpy(&m->max_abs, ctx->h_scalar + 8, 4);
    }
    *out = m;
    return WGML_OK;
}

int wgml_quant_matrix_destroy(wgml_qmat *m) {
    if (!m) return WGML_OK;
    if (m->ctx && m->ctx->stream) (void)hipStreamSynchronize(m->ctx->stream);
    if (m->base) (void)hipFree(m->base);
    ctx_release(m->ctx);
    delete m;
    return WGML_OK;
}

int wgml_quant_matrix_shape(const wgml_qmat *m, int *type, uint32_t *nrows, uint32_t *ncols) {
    WGML_REQUIRE(m != nullptr, "wgml_quant_matrix_shape: null matrix");
    if (type) *type = m->type;
    if (nrows) *nrows = m->nrows;
    if (ncols) *ncols = m->ncols;
    return WGML_OK;
}

uint64_t wgml_quant_matrix_gguf_bytes(const wgml_qmat *m) { return m ? m->gguf_bytes : 0; }

int wgml_quant_matrix_weight_bound(const wgml_qmat *m, float *bound) {
    WGML_REQUIRE(m && bound, "wgml_quant_matrix_weight_bound: null argument");
    *bound = m->max_abs;
    return WGML_OK;
}

int wgml_dequantize(wgml_ctx *ctx, wgml_view out, const wgml_qmat *m) {
    WGML_REQUIRE(ctx && m, "wgml_dequantize: null argument");
    WGML_TRY(check_view(out, "wgml_dequantize: out"));
    WGML_REQUIRE((uint64_t)out.len == (uint64_t)m->nrows * m->ncols,
                 "wgml_dequantize: out has %u elements, matrix has %llu", out.len,
                 (unsigned long long)m->nrows * m->ncols);
    return launch_dequantize(ctx, view_ptr(out), m);
}

int wgml_f16_to_f32(wgml_ctx *ctx, wgml_view out, const wgml_buf *in, uint64_t in_offset_bytes) {
    WGML_REQUIRE(ctx && in, "wgml_f16_to_f32: null argument");
    WGML_TRY(check_view(out, "wgml_f16_to_f32: out"));
    WGML_REQUIRE(in_offset_bytes % 2 == 0 && in_offset_bytes + 2ull * out.len <= in->bytes,
                 "wgml_f16_to_f32: input range exceeds buffer");
    if (out.len == 0) return WGML_OK;
    f16_to_f32_kernel<<<dim3((out.len + 255) / 256), dim3(256), 0, ctx->stream>>>(
        (const uint16_t *)((const char *)in->ptr + in_offset_bytes), view_ptr(out), out.len);
    WGML_CHECK_LAUNCH();
    ctx->launches++;
    return WGML_OK;
}

}  // extern "C"
