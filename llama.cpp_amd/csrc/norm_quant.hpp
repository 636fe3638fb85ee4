// RMS_NORM -> MUL(weight) [-> Q8_1 | Q8_K] of one row by one 256-thread group (ggml_compute_forward_rms_norm_f32,
// ggml/src/ggml-cpu/ggml-cpu.c:6741-6805; quantize_row_q8_1_ref, ggml/src/ggml-quants.c:220-253).  A device function, so that
// a launch which finishes rows can also normalise them; every rounding of the reduction is spelled out, so all callers give
// the same bits.
#pragma once
#include "common.hpp"
#include "q8k.hpp"
#include "tiles.hpp"

namespace mi355 {

// Q8_1 of the 4 values held by each of 8 neighbouring lanes (one 32-element block); writes the
// split activation layout.  Mirrors k_quantize_q8_1 (quantize.hip) instruction for instruction.
__device__ __forceinline__ void quantize_block_lane(const f32x4 &v, bool live, int8_t *__restrict__ qplane, act_ds *__restrict__ ds,
                                                    int64_t row, int64_t k, int64_t e0) {
    const float amax = lanes_max<8>(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    int q[4];
    int sum = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        q[i] = (int)roundf(v[i] * id);
        sum += q[i];
    }
    sum = lanes_sum_i<8>(sum);
    if (!live) return;
    const u32 packed = (u32)(q[0] & 0xFF) | ((u32)(q[1] & 0xFF) << 8) | ((u32)(q[2] & 0xFF) << 16) | ((u32)(q[3] & 0xFF) << 24);
    *(u32 *)(qplane + row * k + e0) = packed;
    if (((e0 >> 2) & 7) == 0) {
        act_ds o;
        o.d = half_bits_to_float(float_to_half_bits(d));
        o.sum = sum;
        ds[row * (k >> 5) + (e0 >> 5)] = o;
    }
}

// Q8_1 of one value per lane over aligned groups of 32 lanes (quantize_row_q8_1_ref, ggml-quants.c:220-253); e = index of the
// lane's element in the row.  COH: the block is stored with device scope (four levels per store, the {d, sum} pair as one
// 8-byte store), for rows that other groups of the same launch read after a grid-wide step.
template <bool COH = false>
__device__ __forceinline__ void quantize_lane32(float v, int8_t *__restrict__ qrow, act_ds *__restrict__ srow, int64_t e) {
    const float amax = lanes_max<32>(fabsf(v));
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const int q = (int)roundf(v * id);
    const int sum = lanes_sum_i<32>(q);
    act_ds o;
    o.d = half_bits_to_float(float_to_half_bits(d));
    o.sum = sum;
    if constexpr (COH) {
        u32 packed = (u32)(q & 0xFF);
        packed |= ((u32)__shfl_down(q, 1, 64) & 0xFFu) << 8;
        packed |= ((u32)__shfl_down(q, 2, 64) & 0xFFu) << 16;
        packed |= ((u32)__shfl_down(q, 3, 64) & 0xFFu) << 24;
        if ((e & 3) == 0) __hip_atomic_store((u32 *)(qrow + e), packed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((e & 31) == 0) {
            const unsigned long long bits = (unsigned long long)__builtin_bit_cast(u32, o.d) | ((unsigned long long)(u32)o.sum << 32);
            __hip_atomic_store((unsigned long long *)(srow + (e >> 5)), bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    } else {
        qrow[e] = (int8_t)q;
        if ((e & 31) == 0) srow[e >> 5] = o;
    }
}

// One row: xr -> y row (optional) and row `row` of the activation workspace `act` (optional), which holds nrows rows of k.
// Each thread keeps its NV float4 of the row in registers (k <= 1024 * NV).  COH: the row was written by other groups of the
// same launch with device-scope stores and is read with device-scope loads.  sh: 4 floats of LDS; the caller places a
// barrier between two calls that share it.
// FMT: activation format written to `act`: 0 Q8_1 (split layout), 1 per-super-block (q8k.hpp), 2 the same as tile images (tiles.hpp)
// Called by the first 256 threads of a group; contains exactly one group barrier, which further waves of a larger group must
// match with a barrier of their own.
template <int NV, int FMT, bool COH>
// keep: where the caller wants the thread's NV pieces of the normalised row (registers), or null
// given: the thread's NV pieces of the row when the caller has just formed them (xr is not read then), or null
__device__ __forceinline__ void rms_norm_quant_row(const float *__restrict__ xr, const float *__restrict__ w, float *__restrict__ yr,
                                                   void *__restrict__ act, int64_t row, int64_t k, int64_t nrows, float eps, float *sh,
                                                   f32x4 *keep = nullptr, const f32x4 *given = nullptr) {
    const int tid = threadIdx.x;
    f32x4 v[NV], ww[NV];
    // the weight does not depend on the reduction: fetch it together with the row, one memory round trip instead of two
#pragma unroll
    for (int it = 0; it < NV; it++) {
        const int64_t e0 = ((int64_t)it * 256 + tid) * 4;
        v[it] = f32x4{0.f, 0.f, 0.f, 0.f};
        ww[it] = f32x4{1.f, 1.f, 1.f, 1.f};
        if (e0 < k) {
            if (given) {
                v[it] = given[it];
            } else if constexpr (COH) {
#pragma unroll
                for (int i = 0; i < 4; i++) v[it][i] = __hip_atomic_load(xr + e0 + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
                v[it] = *(const f32x4 *)(xr + e0);
            }
            if (w) ww[it] = *(const f32x4 *)(w + e0);
        }
    }
    float ss = 0.0f;
#pragma unroll
    for (int it = 0; it < NV; it++)
#pragma unroll
        for (int i = 0; i < 4; i++) ss = __builtin_fmaf(v[it][i], v[it][i], ss);
    ss = wave_sum_dpp(ss);
    if ((tid & 63) == 0) sh[tid >> 6] = ss;
    __syncthreads();
    ss = add_rn(add_rn(add_rn(sh[0], sh[1]), sh[2]), sh[3]);
    const float scale = 1.0f / sqrtf(add_rn(ss / (float)k, eps));
    int8_t *qplane = (int8_t *)act;
    act_ds *ds = (act_ds *)(qplane + nrows * k);
#pragma unroll
    for (int it = 0; it < NV; it++) {
        const int64_t e0 = ((int64_t)it * 256 + tid) * 4;
        const bool live = e0 < k;
        f32x4 o;
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = v[it][i] * scale;
        if (w && live) {
#pragma unroll
            for (int i = 0; i < 4; i++) o[i] = o[i] * ww[it][i];
        }
        if (yr && live) *(f32x4 *)(yr + e0) = o;
        if (keep) keep[it] = o;
        if constexpr (FMT == 2) {
            if (act && live) q8k_quantize_wave_tiled(o, tid & 63, (uint8_t *)act, k, nrows, row, e0 >> 8);   // whole wave: k is a multiple of 256
        } else if constexpr (FMT == 1) {
            if (act && live) {   // whole wave: k is a multiple of 256
                const int64_t nsb = k >> 8, sb = e0 >> 8;
                float *d8 = (float *)(qplane + q8k_d_offset(k, nrows));
                _Float16 *bs = (_Float16 *)(qplane + q8k_bs_offset(k, nrows));
                q8k_quantize_wave(o, tid & 63, qplane + row * k + sb * QKK, d8 + row * nsb + sb, bs + (row * nsb + sb) * 16);
            }
        } else {
            if (act) quantize_block_lane(o, live, qplane, ds, row, k, e0);
        }
    }
}

}  // namespace mi355
