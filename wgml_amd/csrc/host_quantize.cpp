// Host-side input makers: ggml's reference quantizers for Q8_0 / Q4_K / Q6_K and
// a counter-based random generator.  The reference only de-quantizes
// (quantization.rs); its weights come from GGUF files written by ggml, whose
// published algorithms (quantize_row_q8_0_ref, quantize_row_q4_K_ref with
// make_qkx2_quants, quantize_row_q6_K_ref with make_qx_quants) are restated
// here so that synthetic models can be built in-process.  Pure host code.
#include <algorithm>
#include <cmath>
#include <thread>

#include "common.h"

using namespace wgml;

namespace {

constexpr int QK8_0 = 32, QK_K = 256;
constexpr float GROUP_MAX_EPS = 1e-15f;

// IEEE binary32 -> binary16, round to nearest even, overflow to infinity.
uint16_t f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t e = (x >> 23) & 0xffu;
    uint32_t mant = x & 0x7fffffu;
    if (e == 0xff) return (uint16_t)(sign | 0x7c00u | (mant ? 0x200u : 0));
    const int exp = (int)e - 127 + 15;
    if (exp >= 31) return (uint16_t)(sign | 0x7c00u);
    if (exp <= 0) {
        if (exp < -10) return (uint16_t)sign;
        mant |= 0x800000u;
        const int shift = 14 - exp;
        uint32_t h = mant >> shift;
        const uint32_t rem = mant & ((1u << shift) - 1), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (h & 1))) h++;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((uint32_t)exp << 10) | (mant >> 13);
    const uint32_t rem = mant & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) h++;
    return (uint16_t)(sign | h);
}

float f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu, mant = h & 0x3ffu;
    float v;
    if (e == 0) v = std::ldexp((float)mant, -24);
    else if (e != 31) v = std::ldexp((float)(mant + 1024), (int)e - 25);
    else v = mant ? NAN : INFINITY;
    uint32_t bits;
    memcpy(&bits, &v, 4);
    bits |= sign;
    memcpy(&v, &bits, 4);
    return v;
}

inline int nearest_int(float fval) {
    float val = fval + 12582912.f;
    int i;
    memcpy(&i, &val, sizeof(int));
    return (i & 0x007fffff) - 0x00400000;
}

#pragma pack(push, 1)
struct block_q8_0 {
    uint16_t d;
    int8_t qs[QK8_0];
};
struct block_q4_K {
    uint16_t d, dmin;
    uint8_t scales[12];
    uint8_t qs[QK_K / 2];
};
struct block_q6_K {
    uint8_t ql[QK_K / 2];
    uint8_t qh[QK_K / 4];
    int8_t scales[QK_K / 16];
    uint16_t d;
};
#pragma pack(pop)

void quantize_row_q8_0(const float *x, block_q8_0 *y, int64_t k) {
    const int64_t nb = k / QK8_0;
    for (int64_t i = 0; i < nb; i++) {
        float amax = 0.0f;
        for (int j = 0; j < QK8_0; j++) amax = std::max(amax, std::fabs(x[i * QK8_0 + j]));
        const float d = amax / ((1 << 7) - 1);
        const float id = d ? 1.0f / d : 0.0f;
        y[i].d = f32_to_f16(d);
        for (int j = 0; j < QK8_0; ++j) y[i].qs[j] = (int8_t)std::round(x[i * QK8_0 + j] * id);
    }
}

float make_qkx2_quants(int n, int nmax, const float *x, const float *weights, uint8_t *L,
                       float *the_min, uint8_t *Laux, float rmin, float rdelta, int nstep,
                       bool use_mad) {
    float min = x[0], max = x[0];
    float sum_w = weights[0], sum_x = sum_w * x[0];
    for (int i = 1; i < n; ++i) {
        if (x[i] < min) min = x[i];
        if (x[i] > max) max = x[i];
        float w = weights[i];
        sum_w += w;
        sum_x += w * x[i];
    }
    if (min > 0) min = 0;
    if (max == min) {
        for (int i = 0; i < n; ++i) L[i] = 0;
        *the_min = -min;
        return 0.f;
    }
    float iscale = nmax / (max - min);
    float scale = 1 / iscale;
    float best_mad = 0;
    for (int i = 0; i < n; ++i) {
        int l = nearest_int(iscale * (x[i] - min));
        L[i] = (uint8_t)std::max(0, std::min(nmax, l));
        float diff = scale * L[i] + min - x[i];
        diff = use_mad ? std::fabs(diff) : diff * diff;
        best_mad += weights[i] * diff;
    }
    if (nstep < 1) {
        *the_min = -min;
        return scale;
    }
    for (int is = 0; is <= nstep; ++is) {
        iscale = (rmin + rdelta * is + nmax) / (max - min);
        float sum_l = 0, sum_l2 = 0, sum_xl = 0;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int(iscale * (x[i] - min));
            l = std::max(0, std::min(nmax, l));
            Laux[i] = (uint8_t)l;
            float w = weights[i];
            sum_l += w * l;
            sum_l2 += w * l * l;
            sum_xl += w * l * x[i];
        }
        float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0) {
                this_min = 0;
                this_scale = sum_xl / sum_l2;
            }
            float mad = 0;
            for (int i = 0; i < n; ++i) {
                float diff = this_scale * Laux[i] + this_min - x[i];
                diff = use_mad ? std::fabs(diff) : diff * diff;
                mad += weights[i] * diff;
            }
            if (mad < best_mad) {
                for (int i = 0; i < n; ++i) L[i] = Laux[i];
                best_mad = mad;
                scale = this_scale;
                min = this_min;
            }
        }
    }
    *the_min = -min;
    return scale;
}

inline void get_scale_min_k4(int j, const uint8_t *q, uint8_t *d, uint8_t *m) {
    if (j < 4) {
        *d = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j - 0] >> 6) << 4));
    }
}

void quantize_row_q4_K(const float *x, block_q4_K *y, int64_t k) {
    const int64_t nb = k / QK_K;
    uint8_t L[QK_K], Laux[32];
    float weights[32], mins[QK_K / 32], scales[QK_K / 32];
    for (int64_t i = 0; i < nb; i++) {
        float max_scale = 0, max_min = 0;
        for (int j = 0; j < QK_K / 32; ++j) {
            float sum_x2 = 0;
            for (int l = 0; l < 32; ++l) sum_x2 += x[32 * j + l] * x[32 * j + l];
            float av_x = std::sqrt(sum_x2 / 32);
            for (int l = 0; l < 32; ++l) weights[l] = av_x + std::fabs(x[32 * j + l]);
            scales[j] = make_qkx2_quants(32, 15, x + 32 * j, weights, L + 32 * j, &mins[j], Laux,
                                         -1.f, 0.1f, 20, false);
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
        float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
        memset(y[i].scales, 0, sizeof(y[i].scales));
        for (int j = 0; j < QK_K / 32; ++j) {
            uint8_t ls = (uint8_t)std::min(63, nearest_int(inv_scale * scales[j]));
            uint8_t lm = (uint8_t)std::min(63, nearest_int(inv_min * mins[j]));
            if (j < 4) {
                y[i].scales[j] = ls;
                y[i].scales[j + 4] = lm;
            } else {
                y[i].scales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                y[i].scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
                y[i].scales[j - 0] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        y[i].d = f32_to_f16(max_scale / 63.f);
        y[i].dmin = f32_to_f16(max_min / 63.f);

        uint8_t sc, m;
        for (int j = 0; j < QK_K / 32; ++j) {
            get_scale_min_k4(j, y[i].scales, &sc, &m);
            const float d = f16_to_f32(y[i].d) * sc;
            if (!d) continue;
            const float dm = f16_to_f32(y[i].dmin) * m;
            for (int ii = 0; ii < 32; ++ii) {
                int l = nearest_int((x[32 * j + ii] + dm) / d);
                l = std::max(0, std::min(15, l));
                L[32 * j + ii] = (uint8_t)l;
            }
        }
        uint8_t *q = y[i].qs;
        for (int j = 0; j < QK_K; j += 64) {
            for (int l = 0; l < 32; ++l) q[l] = (uint8_t)(L[j + l] | (L[j + l + 32] << 4));
            q += 32;
        }
        x += QK_K;
    }
}

float make_qx_quants(int n, int nmax, const float *x, int8_t *L, int rmse_type) {
    float max = 0, amax = 0;
    for (int i = 0; i < n; ++i) {
        float ax = std::fabs(x[i]);
        if (ax > amax) {
            amax = ax;
            max = x[i];
        }
    }
    if (amax < GROUP_MAX_EPS) {
        for (int i = 0; i < n; ++i) L[i] = 0;
        return 0.f;
    }
    float iscale = -nmax / max;
    (void)rmse_type;  // only the rmse_type == 1 branch (weights x^2) is used for Q6_K
    float sumlx = 0, suml2 = 0;
    for (int i = 0; i < n; ++i) {
        int l = nearest_int(iscale * x[i]);
        l = std::max(-nmax, std::min(nmax - 1, l));
        L[i] = (int8_t)(l + nmax);
        float w = x[i] * x[i];
        sumlx += w * x[i] * l;
        suml2 += w * l * l;
    }
    float scale = suml2 ? sumlx / suml2 : 0.0f;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; ++is) {
        if (is == 0) continue;
        iscale = -(nmax + 0.1f * is) / max;
        sumlx = suml2 = 0;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int(iscale * x[i]);
            l = std::max(-nmax, std::min(nmax - 1, l));
            float w = x[i] * x[i];
            sumlx += w * x[i] * l;
            suml2 += w * l * l;
        }
        if (suml2 > 0 && sumlx * sumlx > best * suml2) {
            for (int i = 0; i < n; ++i) {
                int l = nearest_int(iscale * x[i]);
                L[i] = (int8_t)(nmax + std::max(-nmax, std::min(nmax - 1, l)));
            }
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

void quantize_row_q6_K(const float *x, block_q6_K *y, int64_t k) {
    const int64_t nb = k / QK_K;
    int8_t L[QK_K];
    float scales[QK_K / 16];
    for (int64_t i = 0; i < nb; i++) {
        float max_scale = 0, max_abs_scale = 0;
        for (int ib = 0; ib < QK_K / 16; ++ib) {
            const float scale = make_qx_quants(16, 32, x + 16 * ib, L + 16 * ib, 1);
            scales[ib] = scale;
            const float abs_scale = std::fabs(scale);
            if (abs_scale > max_abs_scale) {
                max_abs_scale = abs_scale;
                max_scale = scale;
            }
        }
        if (max_abs_scale < GROUP_MAX_EPS) {
            memset(&y[i], 0, sizeof(block_q6_K));
            y[i].d = f32_to_f16(0.f);
            x += QK_K;
            continue;
        }
        float iscale = -128.f / max_scale;
        y[i].d = f32_to_f16(1 / iscale);
        for (int ib = 0; ib < QK_K / 16; ++ib)
            y[i].scales[ib] = (int8_t)std::min(127, nearest_int(iscale * scales[ib]));
        for (int j = 0; j < QK_K / 16; ++j) {
            float d = f16_to_f32(y[i].d) * y[i].scales[j];
            if (!d) continue;
            for (int ii = 0; ii < 16; ++ii) {
                int l = nearest_int(x[16 * j + ii] / d);
                l = std::max(-32, std::min(31, l));
                L[16 * j + ii] = (int8_t)(l + 32);
            }
        }
        uint8_t *ql = y[i].ql;
        uint8_t *qh = y[i].qh;
        for (int j = 0; j < QK_K; j += 128) {
            for (int l = 0; l < 32; ++l) {
                const uint8_t q1 = L[j + l + 0] & 0xF;
                const uint8_t q2 = L[j + l + 32] & 0xF;
                const uint8_t q3 = L[j + l + 64] & 0xF;
                const uint8_t q4 = L[j + l + 96] & 0xF;
                ql[l + 0] = (uint8_t)(q1 | (q3 << 4));
                ql[l + 32] = (uint8_t)(q2 | (q4 << 4));
                qh[l] = (uint8_t)((L[j + l] >> 4) | ((L[j + l + 32] >> 4) << 2) |
                                  ((L[j + l + 64] >> 4) << 4) | ((L[j + l + 96] >> 4) << 6));
            }
            ql += 64;
            qh += 32;
        }
        x += QK_K;
    }
}

int pick_threads(int nthreads, uint64_t work_items) {
    if (nthreads <= 0) {
        nthreads = (int)std::thread::hardware_concurrency();
        if (nthreads <= 0) nthreads = 1;
        if (nthreads > 16) nthreads = 16;
    }
    if ((uint64_t)nthreads > work_items) nthreads = (int)std::max<uint64_t>(1, work_items);
    return nthreads;
}

template <class Fn>
void parallel_for(uint64_t n, int nthreads, Fn fn) {
    nthreads = pick_threads(nthreads, n);
    if (nthreads == 1) {
        fn(0, n);
        return;
    }
    std::vector<std::thread> ts;
    const uint64_t per = (n + nthreads - 1) / nthreads;
    for (int t = 0; t < nthreads; ++t) {
        const uint64_t b = (uint64_t)t * per, e = std::min(n, b + per);
        if (b >= e) break;
        ts.emplace_back([=] { fn(b, e); });
    }
    for (auto &t : ts) t.join();
}

inline uint64_t splitmix64(uint64_t z) {
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

inline uint64_t counter_hash(uint64_t seed, uint64_t i) { return splitmix64(splitmix64(seed) ^ i); }

}  // namespace

extern "C" {

int wgml_quantize(int type, const float *src, void *dst, uint64_t nelems, int nthreads) {
    WGML_REQUIRE(src && dst, "wgml_quantize: null argument");
    if (type == WGML_F32) {
        memcpy(dst, src, nelems * 4);
        return WGML_OK;
    }
    if (type != WGML_Q8_0 && type != WGML_Q4_K && type != WGML_Q6_K)
        return set_error(WGML_E_UNSUPPORTED,
                         "wgml_quantize: no quantizer for type %d (Q8_0, Q4_K, Q6_K only)", type);
    const uint32_t be = wgml_quant_block_elems(type);
    WGML_REQUIRE(nelems % be == 0, "wgml_quantize: %llu elements is not a whole number of blocks",
                 (unsigned long long)nelems);
    const uint64_t nblocks = nelems / be;
    parallel_for(nblocks, nthreads, [=](uint64_t b, uint64_t e) {
        switch (type) {
        case WGML_Q8_0:
            quantize_row_q8_0(src + b * QK8_0, (block_q8_0 *)dst + b, (int64_t)(e - b) * QK8_0);
            break;
        case WGML_Q4_K:
            quantize_row_q4_K(src + b * QK_K, (block_q4_K *)dst + b, (int64_t)(e - b) * QK_K);
            break;
        case WGML_Q6_K:
            quantize_row_q6_K(src + b * QK_K, (block_q6_K *)dst + b, (int64_t)(e - b) * QK_K);
            break;
        }
    });
    return WGML_OK;
}

// Block*::dequantize of the reference (quantization.rs:16-42, 204-244, 322-389),
// on the host: used where the reference expands a tensor at load
// (token_embd, models/llama2/transformer.rs:239-242).
int wgml_dequantize_host(int type, const void *src, float *dst, uint64_t nelems, int nthreads) {
    WGML_REQUIRE(src && dst, "wgml_dequantize_host: null argument");
    if (type == WGML_F32) {
        memcpy(dst, src, nelems * 4);
        return WGML_OK;
    }
    if (type == WGML_F16) {
        const uint16_t *h = (const uint16_t *)src;
        parallel_for(nelems, nthreads, [=](uint64_t b, uint64_t e) {
            for (uint64_t i = b; i < e; ++i) dst[i] = f16_to_f32(h[i]);
        });
        return WGML_OK;
    }
    const uint32_t be = wgml_quant_block_elems(type);
    if (!be) return set_error(WGML_E_UNSUPPORTED, "wgml_dequantize_host: unsupported type %d", type);
    if (type != WGML_Q8_0 && type != WGML_Q4_K && type != WGML_Q6_K) {
        WGML_REQUIRE(nelems % be == 0,
                     "wgml_dequantize_host: %llu elements is not a whole number of blocks",
                     (unsigned long long)nelems);
        const uint8_t *raw = (const uint8_t *)src;
        auto u16 = [](const uint8_t *p) { return (uint16_t)(p[0] | ((uint16_t)p[1] << 8)); };
        auto u32 = [](const uint8_t *p) {
            return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
        };
        parallel_for(nelems / be, nthreads, [=](uint64_t b0, uint64_t b1) {
            for (uint64_t bi = b0; bi < b1; ++bi) {
                float *y = dst + bi * be;
                if (type == WGML_Q8_K) {  // quantization.rs:195-201
                    const uint8_t *b = raw + bi * 292;
                    float d;
                    memcpy(&d, b, 4);
                    for (int j = 0; j < QK_K; ++j) y[j] = d * (float)(int8_t)b[4 + j];
                } else if (type == WGML_Q5_K) {  // quantization.rs:274-317
                    const uint8_t *b = raw + bi * 176;
                    const float d = f16_to_f32(u16(b)), dmin = f16_to_f32(u16(b + 2));
                    const uint8_t *sc = b + 4, *qh = b + 16, *qs = b + 48;
                    for (int sub = 0; sub < 8; ++sub) {
                        uint8_t s8, m8;
                        if (sub < 4) {
                            s8 = sc[sub] & 63;
                            m8 = sc[sub + 4] & 63;
                        } else {
                            s8 = (uint8_t)((sc[sub + 4] & 0xF) | ((sc[sub - 4] >> 6) << 4));
                            m8 = (uint8_t)((sc[sub + 4] >> 4) | ((sc[sub] >> 6) << 4));
                        }
                        const float dl = d * (float)s8, ml = dmin * (float)m8;
                        for (int l = 0; l < 32; ++l) {
                            const uint8_t q = qs[(sub >> 1) * 32 + l];
                            const int x = ((sub & 1) ? (q >> 4) : (q & 0xF)) + (((qh[l] >> sub) & 1) ? 16 : 0);
                            y[sub * 32 + l] = dl * (float)x - ml;
                        }
                    }
                } else {  // Q4_0 / Q4_1 / Q5_0 / Q5_1: quantization.rs:53-68, 82-98, 112-131, 146-167
                    const bool has_m = type == WGML_Q4_1 || type == WGML_Q5_1;
                    const bool has_qh = type == WGML_Q5_0 || type == WGML_Q5_1;
                    const uint8_t *b = raw + bi * (18 + (has_m ? 2 : 0) + (has_qh ? 4 : 0));
                    const float d = f16_to_f32(u16(b));
                    const float m = has_m ? f16_to_f32(u16(b + 2)) : 0.f;
                    const uint32_t qh = has_qh ? u32(b + 2 + (has_m ? 2 : 0)) : 0u;
                    const uint8_t *qs = b + 2 + (has_m ? 2 : 0) + (has_qh ? 4 : 0);
                    for (uint32_t j = 0; j < 16; ++j) {
                        uint32_t x0 = qs[j] & 0x0Fu, x1 = (uint32_t)(qs[j] >> 4);
                        if (has_qh) {
                            x0 |= ((qh >> j) << 4) & 0x10u;
                            x1 |= (qh >> (j + 12)) & 0x10u;
                        }
                        if (has_m) {
                            y[j] = (float)x0 * d + m;
                            y[j + 16] = (float)x1 * d + m;
                        } else {
                            const int off = has_qh ? 16 : 8;
                            y[j] = (float)((int)x0 - off) * d;
                            y[j + 16] = (float)((int)x1 - off) * d;
                        }
                    }
                }
            }
        });
        return WGML_OK;
    }
    WGML_REQUIRE(nelems % be == 0,
                 "wgml_dequantize_host: %llu elements is not a whole number of blocks",
                 (unsigned long long)nelems);
    parallel_for(nelems / be, nthreads, [=](uint64_t b0, uint64_t b1) {
        for (uint64_t b = b0; b < b1; ++b) {
            float *y = dst + b * be;
            if (type == WGML_Q8_0) {
                const block_q8_0 &k = ((const block_q8_0 *)src)[b];
                const float d = f16_to_f32(k.d);
                for (int j = 0; j < QK8_0; ++j) y[j] = (float)k.qs[j] * d;
            } else if (type == WGML_Q4_K) {
                const block_q4_K &k = ((const block_q4_K *)src)[b];
                const float d = f16_to_f32(k.d), dmin = f16_to_f32(k.dmin);
                const uint8_t *q = k.qs;
                for (int j = 0, is = 0; j < 4; ++j, is += 2, q += 32) {
                    uint8_t sc[2], m[2];
                    for (int t = 0; t < 2; ++t) {  // get_scale_min_k4
                        const int jj = is + t;
                        if (jj < 4) {
                            sc[t] = k.scales[jj] & 63;
                            m[t] = k.scales[jj + 4] & 63;
                        } else {
                            sc[t] = (uint8_t)((k.scales[jj + 4] & 0xF) | ((k.scales[jj - 4] >> 6) << 4));
                            m[t] = (uint8_t)((k.scales[jj + 4] >> 4) | ((k.scales[jj] >> 6) << 4));
                        }
                    }
                    const float d1 = d * (float)sc[0], m1 = dmin * (float)m[0];
                    const float d2 = d * (float)sc[1], m2 = dmin * (float)m[1];
                    for (int l = 0; l < 32; ++l) y[64 * j + l] = d1 * (float)(q[l] & 0xF) - m1;
                    for (int l = 0; l < 32; ++l) y[64 * j + 32 + l] = d2 * (float)(q[l] >> 4) - m2;
                }
            } else {
                const block_q6_K &k = ((const block_q6_K *)src)[b];
                const float d = f16_to_f32(k.d);
                for (int i = 0; i < 2; ++i) {
                    const uint8_t *ql = k.ql + 64 * i, *qh = k.qh + 32 * i;
                    const int8_t *sc = k.scales + 8 * i;
                    for (int l = 0; l < 32; ++l) {
                        const int is = l / 16;
                        const int q1 = (int)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                        const int q2 = (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                        const int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                        const int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                        y[128 * i + l] = d * (float)sc[is] * (float)q1;
                        y[128 * i + l + 32] = d * (float)sc[is + 2] * (float)q2;
                        y[128 * i + l + 64] = d * (float)sc[is + 4] * (float)q3;
                        y[128 * i + l + 96] = d * (float)sc[is + 6] * (float)q4;
                    }
                }
            }
        }
    });
    return WGML_OK;
}

int wgml_rng_normal(uint64_t seed, float *out, uint64_t n, float mean, float std_, int nthreads) {
    WGML_REQUIRE(out != nullptr || n == 0, "wgml_rng_normal: null output");
    parallel_for((n + 1) / 2, nthreads, [=](uint64_t b, uint64_t e) {
        for (uint64_t p = b; p < e; ++p) {
            const uint64_t h = counter_hash(seed, p);
            // two 24-bit uniforms: u1 in (0,1], u2 in [0,1)
            const float u1 = (float)((h >> 40) + 1) * (1.0f / 16777216.0f);
            const float u2 = (float)((h >> 16) & 0xffffff) * (1.0f / 16777216.0f);
            const float r = std::sqrt(-2.0f * std::log(u1));
            const float a = 6.283185307179586f * u2;
            out[2 * p] = mean + std_ * (r * std::cos(a));
            if (2 * p + 1 < n) out[2 * p + 1] = mean + std_ * (r * std::sin(a));
        }
    });
    return WGML_OK;
}

int wgml_rng_uniform_f32(uint64_t seed, float *out, uint64_t n) {
    WGML_REQUIRE(out != nullptr || n == 0, "wgml_rng_uniform_f32: null output");
    for (uint64_t i = 0; i < n; ++i)  // top 24 bits: every value is exact in f32 and < 1
        out[i] = (float)(counter_hash(seed ^ 0xc2b2ae35u, i) >> 40) * (1.0f / 16777216.0f);
    return WGML_OK;
}

int wgml_rng_uniform_u32(uint64_t seed, uint32_t *out, uint64_t n, uint32_t bound) {
    WGML_REQUIRE(out != nullptr || n == 0, "wgml_rng_uniform_u32: null output");
    WGML_REQUIRE(bound > 0, "wgml_rng_uniform_u32: bound must be positive");
    for (uint64_t i = 0; i < n; ++i) {
        const uint64_t h = counter_hash(seed ^ 0x5bd1e995u, i);
        out[i] = (uint32_t)(((h >> 32) * (uint64_t)bound) >> 32);
    }
    return WGML_OK;
}

}  // extern "C"
