// Device-side helpers: half decoding, K-quant scale unpacking, wavefront-64
// reductions built on DPP.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

namespace wgml {

// decode_f16 (quantization.rs:392-409 of the reference): the hardware
// conversion is exact for every finite half, subnormals included.
__device__ __forceinline__ float f16_bits_to_f32(uint16_t bits) {
    return __half2float(__ushort_as_half(bits));
}

// get_scale_min_k4 (quantization.rs:381-389)
__device__ __forceinline__ void get_scale_min_k4(uint32_t j, const uint8_t *q, uint8_t &d,
                                                 uint8_t &m) {
    if (j < 4) {
        d = q[j] & 63;
        m = q[j + 4] & 63;
    } else {
        d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

// ---- wavefront-64 reductions ---------------------------------------------------
// DPP controls: quad_perm [1,0,3,2] = 0xB1, quad_perm [2,3,0,1] = 0x4E,
// row_half_mirror = 0x141, row_mirror = 0x140.  After the four steps every lane
// of a 16-lane row holds the row's total; the four row totals are then read
// with v_readlane (uniform across the wave).
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(
        __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_f32<0xB1>(v);
    v += dpp_f32<0x4E>(v);
    v += dpp_f32<0x141>(v);
    v += dpp_f32<0x140>(v);
    return v;
}

__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_f32<0xB1>(v));
    v = fmaxf(v, dpp_f32<0x4E>(v));
    v = fmaxf(v, dpp_f32<0x141>(v));
    v = fmaxf(v, dpp_f32<0x140>(v));
    return v;
}

__device__ __forceinline__ float readlane_f32(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// Sum over the 64 lanes, returned in every lane (wave-uniform).  The order of
// the additions is fixed, so results are reproducible run to run.
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    return (readlane_f32(v, 0) + readlane_f32(v, 16)) + (readlane_f32(v, 32) + readlane_f32(v, 48));
}

__device__ __forceinline__ float wave_max(float v) {
    v = row16_max(v);
    return fmaxf(fmaxf(readlane_f32(v, 0), readlane_f32(v, 16)),
                 fmaxf(readlane_f32(v, 32), readlane_f32(v, 48)));
}

// Block-wide sum for blocks of up to 16 waves.  `red` must hold 16 floats.
// Every thread returns the total.  Contains two barriers.
__device__ __forceinline__ float block_sum(float v, float *red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();  // protect `red` from the previous use
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int w = 0; w < nw; ++w) t += red[w];
    return t;
}

__device__ __forceinline__ float block_max(float v, float *red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = red[0];
    for (int w = 1; w < nw; ++w) t = fmaxf(t, red[w]);
    return t;
}

// GELU, tanh form (UnaryOp::Gelu, ops/unary.rs:106-110).
__device__ __forceinline__ float gelu_tanh(float x) {
    return 0.5f * x * (1.0f + tanhf(0.79788456080286535588f * x * (1.0f + 0.044715f * x * x)));
}

// Unsigned byte k of a 32-bit word as float (v_cvt_f32_ubyteK).
__device__ __forceinline__ float ub0(uint32_t w) { return (float)(w & 0xffu); }
__device__ __forceinline__ float ub1(uint32_t w) { return (float)((w >> 8) & 0xffu); }
__device__ __forceinline__ float ub2(uint32_t w) { return (float)((w >> 16) & 0xffu); }
__device__ __forceinline__ float ub3(uint32_t w) { return (float)(w >> 24); }
// Signed byte k of a 32-bit word as float.
__device__ __forceinline__ float sb0(uint32_t w) { return (float)(int8_t)(w & 0xffu); }
__device__ __forceinline__ float sb1(uint32_t w) { return (float)(int8_t)((w >> 8) & 0xffu); }
__device__ __forceinline__ float sb2(uint32_t w) { return (float)(int8_t)((w >> 16) & 0xffu); }
__device__ __forceinline__ float sb3(uint32_t w) { return (float)((int32_t)w >> 24); }

}  // namespace wgml
