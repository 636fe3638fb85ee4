// Bandwidth-bound quantized GEMV (batch 1..8): dst[b][n] = sum_k W[n][k] * x[b][k].
//
// One wave owns RPW consecutive weight rows and walks them in steps of 64 chunks
// (2048 elements): every lane issues one or two 16-byte streaming loads per row per step,
// to consecutive addresses across the wave, so HBM sees long linear bursts.  The
// activation chunk (already Q8_1-quantized, L2 resident) is loaded once per step and
// reused for all RPW rows and all NCOLS activation rows.  Integer dots use v_dot4_i32_i8;
// scales are applied in f32; the wave reduces with cross-lane shuffles.
#include "common.hpp"
#include "qdot.hpp"

#include <stdlib.h>

namespace mi355 {

template <int TYPE, int NCOLS, int RPW>
__device__ __forceinline__ void gemv_body(const uint8_t *__restrict__ W, const int8_t *__restrict__ aq,
                                          const act_ds *__restrict__ ads, float *__restrict__ dst, int64_t N,
                                          int64_t K, int64_t dst_stride, const row_layout &L) {
    typedef wq<TYPE> T;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * RPW;
    if (row0 >= N) return;   // whole wave exits together

    const int64_t nchunks = K >> 5;
    const int64_t nblk = K >> 5;   // Q8_1 blocks per activation row

    const uint8_t *rows[RPW];
#pragma unroll
    for (int r = 0; r < RPW; r++) {
        const int64_t row = row0 + r < N ? row0 + r : N - 1;   // clamp: tail rows recompute the last row, never stored
        rows[r] = W + row * L.row_bytes;
    }

    float acc[RPW][NCOLS];
#pragma unroll
    for (int r = 0; r < RPW; r++)
#pragma unroll
        for (int c = 0; c < NCOLS; c++) acc[r][c] = 0.0f;

    for (int64_t c0 = 0; c0 < nchunks; c0 += 64) {
        const int64_t c = c0 + lane;
        if (c < nchunks) {
            typename T::chunk w[RPW];
#pragma unroll
            for (int r = 0; r < RPW; r++) w[r] = T::load(rows[r], L, c);
#pragma unroll
            for (int col = 0; col < NCOLS; col++) {
                const act_chunk A = load_act_chunk<TYPE>(aq + col * K, ads + col * nblk, c);
#pragma unroll
                for (int r = 0; r < RPW; r++) {
                    const chunk_dots d = T::dots(w[r], A);
                    acc[r][col] += T::combine(w[r], A, d);
                }
            }
        }
    }

#pragma unroll
    for (int r = 0; r < RPW; r++)
#pragma unroll
        for (int c = 0; c < NCOLS; c++) {
            const float s = wave_sum(acc[r][c]);
            if (lane == 0 && row0 + r < N) dst[c * dst_stride + row0 + r] = s;
        }
}

template <int TYPE, int NCOLS, int RPW>
__global__ void __launch_bounds__(256) k_gemv_q(const uint8_t *__restrict__ W, const int8_t *__restrict__ aq,
                                                const act_ds *__restrict__ ads, float *__restrict__ dst, int64_t N,
                                                int64_t K, int64_t dst_stride, row_layout L) {
    gemv_body<TYPE, NCOLS, RPW>(W, aq, ads, dst, N, K, dst_stride, L);
}

// MUL_MAT_ID, one activation row per expert slot: blockIdx.y = slot = t * n_used + e.  The
// expert id is read on the device, so no host synchronisation is needed to route tokens.
template <int TYPE, int RPW>
__global__ void __launch_bounds__(256) k_gemv_id(const uint8_t *__restrict__ as, const int8_t *__restrict__ aq,
                                                 const act_ds *__restrict__ ads, const int32_t *__restrict__ ids,
                                                 int64_t ids_stride, float *__restrict__ dst, int64_t N, int64_t K,
                                                 int64_t n_expert, int64_t n_used, int64_t nb1, row_layout L) {
    const int64_t slot = blockIdx.y, t = slot / n_used, e = slot % n_used;
    int64_t ex = ids[t * ids_stride + e];
    ex = ex < 0 ? 0 : (ex >= n_expert ? n_expert - 1 : ex);   // never index outside the expert stack
    const int64_t arow = t * nb1 + e % nb1;
    gemv_body<TYPE, 1, RPW>(as + ex * N * L.row_bytes, aq + arow * K, ads + arow * (K >> 5), dst + slot * N, N, K, N, L);
}

// Same routing for weight rows that are not 16-byte aligned (byte loads): one wave per (row, slot).
template <int TYPE>
__global__ void __launch_bounds__(64) k_gemv_id_unaligned(const uint8_t *__restrict__ as, const int8_t *__restrict__ aq,
                                                          const act_ds *__restrict__ ads, const int32_t *__restrict__ ids,
                                                          int64_t ids_stride, float *__restrict__ dst, int64_t N, int64_t K,
                                                          int64_t n_expert, int64_t n_used, int64_t nb1, row_layout L) {
    const int64_t row = blockIdx.x, slot = blockIdx.y, t = slot / n_used, e = slot % n_used;
    int64_t ex = ids[t * ids_stride + e];
    ex = ex < 0 ? 0 : (ex >= n_expert ? n_expert - 1 : ex);
    const int64_t arow = t * nb1 + e % nb1;
    const uint8_t *wrow = as + (ex * N + row) * L.row_bytes;
    const int8_t *q = aq + arow * K;
    const act_ds *ds = ads + arow * (K >> 5);
    float acc = 0.0f;
    for (int64_t i = threadIdx.x; i < K; i += 64) acc += weight_value<TYPE>(wrow, L, i) * (ds[i >> 5].d * (float)q[i]);
    acc = wave_sum(acc);
    if (threadIdx.x == 0) dst[slot * N + row] = acc;
}

// Parity dump of the integer granule dots (one wave per row, activation row 0).
template <int TYPE>
__global__ void __launch_bounds__(64) k_block_dots(const uint8_t *__restrict__ W, const int8_t *__restrict__ aq,
                                                   const act_ds *__restrict__ ads, int32_t *__restrict__ out, int64_t N,
                                                   int64_t K, row_layout L) {
    typedef wq<TYPE> T;
    const int lane = threadIdx.x;
    const int64_t row = blockIdx.x;
    const int64_t nchunks = K >> 5;
    const uint8_t *wrow = W + row * L.row_bytes;
    for (int64_t c0 = 0; c0 < nchunks; c0 += 64) {
        const int64_t c = c0 + lane;
        const bool live = c < nchunks;
        const int64_t cc = live ? c : 0;
        const typename T::chunk w = T::load(wrow, L, cc);
        act_chunk A = load_act_chunk<TYPE>(aq, ads, cc);
        const chunk_dots d = T::dots(w, A);
        if constexpr (TYPE == MI355_Q4_0 || TYPE == MI355_Q8_0) {
            if (live) out[row * nchunks + c] = d.i0;
        } else if constexpr (TYPE == MI355_Q4_K) {
            // two lanes hold the halves of sub-blocks 2g and 2g+1
            const int o0 = d.i0 + __shfl_xor(d.i0, 1, 64);
            const int o1 = d.i1 + __shfl_xor(d.i1, 1, 64);
            if (live && (c & 1) == 0) {
                const int64_t sb = c >> 3;
                const int g = (int)(c & 7) >> 1;
                out[row * nchunks + sb * 8 + 2 * g] = o0;
                out[row * nchunks + sb * 8 + 2 * g + 1] = o1;
            }
        } else {   // Q6_K: 16 granules per super-block
            if (live) {
                const int64_t sb = c >> 3;
                const int ccc = (int)(c & 7), hf = ccc >> 2, r = ccc & 3;
                const int gi = 8 * hf + 2 * (r >> 1) + (r & 1);
                out[row * (nchunks * 2) + sb * 16 + gi] = d.i0;
                out[row * (nchunks * 2) + sb * 16 + gi + 4] = d.i1;
            }
        }
    }
}

template <int TYPE, int NCOLS, int RPW>
static void launch_gemv(hipStream_t s, const void *W, const void *act, float *dst, int64_t N, int64_t K, int64_t B,
                        int64_t dst_stride) {
    const row_layout L = make_row_layout(TYPE, K);
    const int8_t *aq = (const int8_t *)act;
    const act_ds *ads = (const act_ds *)(aq + B * K);
    const int64_t rows_per_group = 4 * RPW;
    const unsigned grid = (unsigned)((N + rows_per_group - 1) / rows_per_group);
    hipLaunchKernelGGL((k_gemv_q<TYPE, NCOLS, RPW>), dim3(grid), dim3(256), 0, s, (const uint8_t *)W, aq, ads, dst, N, K,
                       dst_stride, L);
}

template <int TYPE, int NCOLS>
static void launch_gemv_rpw(int rpw, hipStream_t s, const void *W, const void *act, float *dst, int64_t N, int64_t K,
                            int64_t B, int64_t dst_stride) {
    switch (rpw) {
        case 1: launch_gemv<TYPE, NCOLS, 1>(s, W, act, dst, N, K, B, dst_stride); break;
        case 2: launch_gemv<TYPE, NCOLS, 2>(s, W, act, dst, N, K, B, dst_stride); break;
        default: launch_gemv<TYPE, NCOLS, 4>(s, W, act, dst, N, K, B, dst_stride); break;
    }
}

template <int TYPE>
static void launch_gemv_cols(int rpw, hipStream_t s, const void *W, const void *act, float *dst, int64_t N, int64_t K,
                             int64_t B, int64_t dst_stride) {
    switch (B) {
        case 1: launch_gemv_rpw<TYPE, 1>(rpw, s, W, act, dst, N, K, B, dst_stride); break;
        case 2: launch_gemv_rpw<TYPE, 2>(rpw, s, W, act, dst, N, K, B, dst_stride); break;
        case 3: launch_gemv_rpw<TYPE, 3>(rpw, s, W, act, dst, N, K, B, dst_stride); break;
        case 4: launch_gemv_rpw<TYPE, 4>(rpw, s, W, act, dst, N, K, B, dst_stride); break;
        case 5: launch_gemv_rpw<TYPE, 5>(rpw > 2 ? 2 : rpw, s, W, act, dst, N, K, B, dst_stride); break;
        case 6: launch_gemv_rpw<TYPE, 6>(rpw > 2 ? 2 : rpw, s, W, act, dst, N, K, B, dst_stride); break;
        case 7: launch_gemv_rpw<TYPE, 7>(rpw > 2 ? 2 : rpw, s, W, act, dst, N, K, B, dst_stride); break;
        default: launch_gemv_rpw<TYPE, 8>(rpw > 2 ? 2 : rpw, s, W, act, dst, N, K, B, dst_stride); break;
    }
}

// rows per wave: enough waves to cover every SIMD a few times over, then amortise the
// activation reads over more rows.  MI355_GEMV_RPW overrides (tuning aid).
static int pick_rpw(int64_t N) {
    static int forced = -1;
    if (forced < 0) {
        const char *e = getenv("MI355_GEMV_RPW");
        forced = e ? atoi(e) : 0;
    }
    if (forced == 1 || forced == 2 || forced == 4) return forced;
    if (N >= 32768) return 4;
    if (N >= 8192) return 2;
    return 1;
}

}  // namespace mi355

using namespace mi355;

extern "C" {

int mi355_mul_mat_vec_q(void *stream, int type, const void *W, const void *act, float *dst, int64_t N, int64_t K,
                        int64_t B, int64_t dst_stride) {
    MI355_REQUIRE(is_weight_type(type), "mul_mat_vec_q: unsupported weight type %d", type);
    MI355_REQUIRE(N > 0 && K > 0 && B >= 1 && B <= 8, "mul_mat_vec_q: bad shape N=%lld K=%lld B=%lld", (long long)N, (long long)K, (long long)B);
    MI355_REQUIRE(K % type_block_elems(type) == 0, "mul_mat_vec_q: K=%lld is not a multiple of the block size", (long long)K);
    MI355_REQUIRE(dst_stride >= N, "mul_mat_vec_q: dst_stride < N");
    const row_layout L = make_row_layout(type, K);
    MI355_REQUIRE(((uintptr_t)W & 15) == 0 && (L.row_bytes & 15) == 0 && (L.off_b & 15) == 0 && (L.off_c & 15) == 0,
                  "mul_mat_vec_q: weight rows are not 16-byte aligned (K=%lld)", (long long)K);
    MI355_REQUIRE(((uintptr_t)act & 15) == 0, "mul_mat_vec_q: activation workspace is not 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const int rpw = pick_rpw(N);
    switch (type) {
        case MI355_Q4_0: launch_gemv_cols<MI355_Q4_0>(rpw, s, W, act, dst, N, K, B, dst_stride); break;
        case MI355_Q8_0: launch_gemv_cols<MI355_Q8_0>(rpw, s, W, act, dst, N, K, B, dst_stride); break;
        case MI355_Q4_K: launch_gemv_cols<MI355_Q4_K>(rpw, s, W, act, dst, N, K, B, dst_stride); break;
        default: launch_gemv_cols<MI355_Q6_K>(rpw, s, W, act, dst, N, K, B, dst_stride); break;
    }
    return launch_status("k_gemv_q");
}

// act: split layout of nb1*T quantized rows of b.  dst [N, n_used, T] contiguous.
int mi355_mul_mat_id_vec(void *stream, int type, const void *as, const void *act, const int32_t *ids, int64_t ids_stride,
                         float *dst, int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T) {
    MI355_REQUIRE(is_weight_type(type), "mul_mat_id: unsupported weight type %d", type);
    MI355_REQUIRE(N > 0 && K > 0 && n_expert > 0 && n_used > 0 && nb1 > 0 && T > 0, "mul_mat_id: bad shape");
    MI355_REQUIRE(K % type_block_elems(type) == 0, "mul_mat_id: K=%lld is not a multiple of the block size", (long long)K);
    MI355_REQUIRE(n_used * T <= 65535, "mul_mat_id: too many expert slots for one launch");
    const row_layout L = make_row_layout(type, K);
    hipStream_t s = (hipStream_t)stream;
    const int8_t *aq = (const int8_t *)act;
    const act_ds *ads = (const act_ds *)(aq + nb1 * T * K);
    if (!(((uintptr_t)as & 15) == 0 && (L.row_bytes & 15) == 0 && (L.off_b & 15) == 0 && (L.off_c & 15) == 0)) {
        const dim3 ugrid((unsigned)N, (unsigned)(n_used * T));
        switch (type) {
            case MI355_Q4_0: hipLaunchKernelGGL(k_gemv_id_unaligned<MI355_Q4_0>, ugrid, dim3(64), 0, s, (const uint8_t *)as, aq, ads, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, L); break;
            case MI355_Q8_0: hipLaunchKernelGGL(k_gemv_id_unaligned<MI355_Q8_0>, ugrid, dim3(64), 0, s, (const uint8_t *)as, aq, ads, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, L); break;
            case MI355_Q4_K: hipLaunchKernelGGL(k_gemv_id_unaligned<MI355_Q4_K>, ugrid, dim3(64), 0, s, (const uint8_t *)as, aq, ads, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, L); break;
            default: hipLaunchKernelGGL(k_gemv_id_unaligned<MI355_Q6_K>, ugrid, dim3(64), 0, s, (const uint8_t *)as, aq, ads, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, L); break;
        }
        return launch_status("k_gemv_id_unaligned");
    }
    const int rpw = pick_rpw(N) > 2 ? 2 : pick_rpw(N);
    const dim3 grid((unsigned)((N + 4 * rpw - 1) / (4 * rpw)), (unsigned)(n_used * T));
#define MI355_ID_LAUNCH(TY)                                                                                           \
    if (rpw == 1) hipLaunchKernelGGL((k_gemv_id<TY, 1>), grid, dim3(256), 0, s, (const uint8_t *)as, aq, ads, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, L); \
    else hipLaunchKernelGGL((k_gemv_id<TY, 2>), grid, dim3(256), 0, s, (const uint8_t *)as, aq, ads, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, L);
    switch (type) {
        case MI355_Q4_0: MI355_ID_LAUNCH(MI355_Q4_0) break;
        case MI355_Q8_0: MI355_ID_LAUNCH(MI355_Q8_0) break;
        case MI355_Q4_K: MI355_ID_LAUNCH(MI355_Q4_K) break;
        default: MI355_ID_LAUNCH(MI355_Q6_K) break;
    }
#undef MI355_ID_LAUNCH
    return launch_status("k_gemv_id");
}

int mi355_block_dots_q8_1(void *stream, int type, const void *W, const void *a, int32_t *out, int64_t N, int64_t K) {
    // `a` is the split activation layout of mi355_quantize_act for ONE row
    MI355_REQUIRE(is_weight_type(type), "block_dots: unsupported weight type %d", type);
    MI355_REQUIRE(N > 0 && K > 0 && K % type_block_elems(type) == 0, "block_dots: bad shape");
    const row_layout L = make_row_layout(type, K);
    MI355_REQUIRE(((uintptr_t)W & 15) == 0 && (L.row_bytes & 15) == 0 && (L.off_b & 15) == 0 && (L.off_c & 15) == 0,
                  "block_dots: weight rows are not 16-byte aligned (K=%lld)", (long long)K);
    hipStream_t s = (hipStream_t)stream;
    const int8_t *aq = (const int8_t *)a;
    const act_ds *ads = (const act_ds *)(aq + K);
    const dim3 grid((unsigned)N);
    switch (type) {
        case MI355_Q4_0: hipLaunchKernelGGL(k_block_dots<MI355_Q4_0>, grid, dim3(64), 0, s, (const uint8_t *)W, aq, ads, out, N, K, L); break;
        case MI355_Q8_0: hipLaunchKernelGGL(k_block_dots<MI355_Q8_0>, grid, dim3(64), 0, s, (const uint8_t *)W, aq, ads, out, N, K, L); break;
        case MI355_Q4_K: hipLaunchKernelGGL(k_block_dots<MI355_Q4_K>, grid, dim3(64), 0, s, (const uint8_t *)W, aq, ads, out, N, K, L); break;
        default: hipLaunchKernelGGL(k_block_dots<MI355_Q6_K>, grid, dim3(64), 0, s, (const uint8_t *)W, aq, ads, out, N, K, L); break;
    }
    return launch_status("k_block_dots");
}

}  // extern "C"
