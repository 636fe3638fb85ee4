// Activation format of the K-quant tile GEMM: the rows quantized per 256-element super-block exactly as
// quantize_row_q8_K_ref does (ggml/src/ggml-quants.c:2479-2516), stored split:
//   int8 q[B][K]; float d8[B][K/256] (padded to 16 bytes); fp16 bs[B][K/256][16]
// bs = {bsum_j & 63 (j = 0..7), bsum_j >> 6 (j = 0..7)} of the eight 32-element sub-blocks.
#pragma once
#include "common.hpp"

namespace mi355 {

__host__ __device__ inline size_t q8k_d_offset(int64_t K, int64_t B) { return (size_t)B * (size_t)K; }
__host__ __device__ inline size_t q8k_bs_offset(int64_t K, int64_t B) {
    return (q8k_d_offset(K, B) + (size_t)B * (size_t)(K / QKK) * 4 + 15) & ~(size_t)15;   // bs entries are read 16 bytes at a time
}

// One wave quantizes one super-block: lane l holds elements 4l .. 4l+3.  packed: the lane's four int8 levels; d: the super-block's
// scale (every lane); sum: the integer sum of the lane's 32-element sub-block (every lane of the 8 that share it).
__device__ __forceinline__ void q8k_quantize_values(const f32x4 &v, int lane, u32 &packed, float &d, int &sum) {
    // signed value of the first element with the largest magnitude
    float amax = 0.0f, vmax = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float ax = fabsf(v[i]);
        if (ax > amax) { amax = ax; vmax = v[i]; }
    }
    // over the wave: the largest magnitude, the lowest lane among equals (magnitudes order as their bit patterns), then that lane's value
    {
        u32 hi = __builtin_bit_cast(u32, amax), lo = 63u - (u32)lane;
        wave_max_key(hi, lo);
        amax = __builtin_bit_cast(float, hi);
        vmax = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, vmax), (int)(63u - lo)));
    }

    int lv[4] = {0, 0, 0, 0};
    d = 0.0f;
    if (amax != 0.0f) {
        const float iscale = -127.0f / vmax;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int n = (int)rintf(iscale * v[i]);
            lv[i] = n < 127 ? n : 127;
        }
        d = 1.0f / iscale;
    }
    sum = lanes_sum_i<8>(lv[0] + lv[1] + lv[2] + lv[3]);
    packed = (u32)(lv[0] & 0xFF) | ((u32)(lv[1] & 0xFF) << 8) | ((u32)(lv[2] & 0xFF) << 16) | ((u32)(lv[3] & 0xFF) << 24);
}

// The same, stored: q, d8, bs point at the super-block's entries.
__device__ __forceinline__ void q8k_quantize_wave(const f32x4 &v, int lane, int8_t *__restrict__ q, float *__restrict__ d8, _Float16 *__restrict__ bs) {
    u32 packed;
    float d;
    int sum;
    q8k_quantize_values(v, lane, packed, d, sum);
    *(u32 *)(q + lane * 4) = packed;
    if (lane == 0) *d8 = d;
    if ((lane & 7) == 0) {
        bs[lane >> 3] = (_Float16)(float)(sum & 63);
        bs[8 + (lane >> 3)] = (_Float16)(float)(sum >> 6);
    }
}

}  // namespace mi355
