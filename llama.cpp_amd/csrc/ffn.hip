// The feed-forward half of a decoded token (llm_build_ffn with LLM_FFN_SILU / LLM_FFN_PAR, src/llama.cpp:280-320):
//   k_gemv_gate_up_blk   ffn_gate, ffn_up, SiLU(gate) * up and the Q8_1 quantization of the product in one launch with no step
//                        between groups: a group owns the 32 output rows of one Q8_1 block in BOTH matrices.
// Measured and not adopted: the same launch continued, past a grid-wide step (per-group flags polled with device-scope loads, the
// wait bounded by the wall clock), with ffn_down + residual, every wave requesting its ffn_down rows before it waits - bit-identical
// to the two launches, but 33.1 / 34.9 us (Q4_K / Q6_K ffn_down) against 15.3 + 10.6 / 11.5 us on the 8B shape: a compute unit's
// vector memory requests complete in order, so the flag polls queue behind the unit's own weight requests and the step costs as
// much as the stream it was meant to hide.
// Row sums are formed exactly as in gemv_body (gemv.hip): same lane-to-chunk mapping, same step order, same wave reduction, so
// every result holds the bits of the separate launches (ggml_compute_forward_mul_mat, ggml-cpu.c:7443-7635, with
// ggml_vec_dot_q*_q8_*; UNARY(SILU) and MUL :6646-6683, 5142-5211; quantize_row_q8_1_ref, ggml-quants.c:220-253).
#include "common.hpp"
#include "qdot.hpp"
#include "norm_quant.hpp"
#include "ffn.hpp"

namespace mi355 {

extern __shared__ __attribute__((aligned(16))) uint8_t s_ffn_dyn[];

// eight waves per group; rows of each matrix a wave has in flight (the types with the largest chunks walk their four rows in two
// rounds, or their registers would not leave room for two groups per compute unit)
constexpr int GU_WAVES = 8;
constexpr int gu_rows_in_flight(int type) { return (type == MI355_Q5_K || type == MI355_Q6_K) ? 2 : 4; }

// Wave w of the group: rows 32 b + RPM w .. + RPM - 1 of gate and of up (RPM = 32 / WAVES), R rows of each in flight; the
// block's 32 values of every activation row meet in s_g / s_u and are quantized by the group's first lanes.  The first round's
// weights are requested before the activation is copied to LDS.  COH: the quantized block is stored with device scope.
template <int TYPE, int NCOLS, int WAVES, int R, bool COH>
__device__ __forceinline__ void gate_up_blk_phase(const uint8_t *__restrict__ Wg, const uint8_t *__restrict__ Wu, const int8_t *__restrict__ aq,
                                                  const act_ds *__restrict__ ads, int K, float *__restrict__ gate, float *__restrict__ up,
                                                  int64_t out_stride, int8_t *__restrict__ act_q, act_ds *__restrict__ act_s, int n,
                                                  uint8_t *s_act, float (*s_g)[32], float (*s_u)[32]) {
    typedef wq<TYPE> T;
    constexpr int RPM = 32 / WAVES;            // rows of each matrix per wave
    static_assert(RPM % R == 0, "rows per wave are walked in rounds of R");
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t blk = blockIdx.x;
    const row_layout L = make_row_layout(TYPE, K);
    const int nchunks = K / T::CHUNK;
    const int nblk = K >> 5;
    const int64_t row0 = blk * 32 + wave * RPM;
    // first round's weights of step 0 are requested before the activation is copied to LDS
    const uint8_t *rows[2 * R];
    typename T::chunk w_first[2 * R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        rows[r] = Wg + (row0 + r) * L.row_bytes;
        rows[R + r] = Wu + (row0 + r) * L.row_bytes;
    }
    const int c_first = lane < nchunks ? lane : nchunks - 1;
    int8_t *s_q = (int8_t *)s_act;
    act_ds *s_ds = (act_ds *)(s_act + NCOLS * K);
    {
#pragma unroll
        for (int r = 0; r < 2 * R; r++) w_first[r] = T::load_w(rows[r], L, c_first);
        for (int i = threadIdx.x * 16; i < NCOLS * K; i += 64 * WAVES * 16) *(u32x4 *)(s_q + i) = load16(aq + i);
        for (int i = threadIdx.x; i < NCOLS * nblk; i += 64 * WAVES) s_ds[i] = ads[i];
    }
    __syncthreads();
#pragma unroll
    for (int round = 0; round < RPM / R; round++) {
        if (round > 0) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                rows[r] = Wg + (row0 + round * R + r) * L.row_bytes;
                rows[R + r] = Wu + (row0 + round * R + r) * L.row_bytes;
            }
        }
        float acc[2 * R][NCOLS];
#pragma unroll
        for (int r = 0; r < 2 * R; r++)
#pragma unroll
            for (int c = 0; c < NCOLS; c++) acc[r][c] = 0.0f;
        for (int c0 = 0; c0 < nchunks; c0 += 64) {
            const int c = c0 + lane;
            if (c < nchunks) {
                typename T::chunk w[2 * R];
#pragma unroll
                for (int r = 0; r < 2 * R; r++) {
                    if (round == 0 && c0 == 0) w[r] = w_first[r];
                    else w[r] = T::load_w(rows[r], L, c);
                }
#pragma unroll
                for (int col = 0; col < NCOLS; col++) {
                    const typename T::act A = T::load_a(s_q + (int64_t)col * K, s_ds + col * nblk, c);
#pragma unroll
                    for (int r = 0; r < 2 * R; r++) {
                        const chunk_dots d = T::dots(w[r], A);
                        acc[r][col] = T::accumulate(acc[r][col], w[r], A, d);
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < 2 * R; r++)
#pragma unroll
            for (int c = 0; c < NCOLS; c++) {
                const float sum = wave_sum_dpp(acc[r][c]);
                if (lane == 0) {
                    const int j = wave * RPM + round * R + (r < R ? r : r - R);    // row inside the block
                    if (r < R) { s_g[c][j] = sum; gate[c * out_stride + blk * 32 + j] = sum; }
                    else { s_u[c][j] = sum; up[c * out_stride + blk * 32 + j] = sum; }
                }
            }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < 32 * NCOLS; idx += 64 * WAVES) {   // whole aligned groups of 32 lanes
        const int col = idx >> 5, j = idx & 31;
        const float h = silu_fast(s_g[col][j]) * s_u[col][j];
        quantize_lane32<COH>(h, act_q + (int64_t)col * n, act_s + (int64_t)col * (n >> 5), blk * 32 + j);
    }
}

template <int TYPE, int NCOLS, int WAVES, int R>
__global__ void __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(NCOLS == 1 ? 4 : 1, 8)))
k_gemv_gate_up_blk(const uint8_t *__restrict__ Wg, const uint8_t *__restrict__ Wu, const int8_t *__restrict__ aq, const act_ds *__restrict__ ads, int K,
                   float *__restrict__ gate, float *__restrict__ up, int64_t out_stride, int8_t *__restrict__ act_q, act_ds *__restrict__ act_s, int n) {
    __shared__ float s_g[NCOLS][32], s_u[NCOLS][32];
    gate_up_blk_phase<TYPE, NCOLS, WAVES, R, false>(Wg, Wu, aq, ads, K, gate, up, out_stride, act_q, act_s, n, s_ffn_dyn, s_g, s_u);
}

int launch_gate_up_blk(hipStream_t s, int type, const void *w_gate, const void *w_up, const int8_t *aq, const act_ds *ads, int64_t K, int64_t B,
                       float *gate, float *up, int64_t out_stride, void *act_out, int64_t N) {
    const size_t lds = (size_t)(B * (K + K / 4));
    int8_t *oq = (int8_t *)act_out;
    act_ds *os = (act_ds *)(oq + B * N);
    const dim3 grid((unsigned)(N / 32));
#define MI355_BLK_ARGS grid, dim3(64 * GU_WAVES), lds, s, (const uint8_t *)w_gate, (const uint8_t *)w_up, aq, ads, (int)K, gate, up, out_stride, oq, os, (int)N
#define MI355_BLK_LAUNCH(TY)                                                                                        \
    switch (B) {                                                                                                    \
        case 1: MI355_LAUNCH((k_gemv_gate_up_blk<TY, 1, GU_WAVES, gu_rows_in_flight(TY)>), MI355_BLK_ARGS); break;  \
        case 2: MI355_LAUNCH((k_gemv_gate_up_blk<TY, 2, GU_WAVES, gu_rows_in_flight(TY)>), MI355_BLK_ARGS); break;  \
        case 3: MI355_LAUNCH((k_gemv_gate_up_blk<TY, 3, GU_WAVES, gu_rows_in_flight(TY)>), MI355_BLK_ARGS); break;  \
        default: MI355_LAUNCH((k_gemv_gate_up_blk<TY, 4, GU_WAVES, gu_rows_in_flight(TY)>), MI355_BLK_ARGS); break; \
    }
    MI355_WEIGHT_TYPE_SWITCH(type, MI355_BLK_LAUNCH)
#undef MI355_BLK_LAUNCH
#undef MI355_BLK_ARGS
    return launch_status("k_gemv_gate_up_blk");
}

// The same launch for the experts of a mixture-of-experts layer (llm_build_moe_ffn, src/llama.cpp:417-538: MUL_MAT_ID(up),
// MUL_MAT_ID(gate), SILU, MUL): blockIdx.y = slot = t * n_used + e, the expert read on the device as k_gemv_id does, one activation
// row per slot.  gate / up: f32 [slots][N]; the quantized product: rows of N per slot.
template <int TYPE, int WAVES, int R>
__global__ void __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(4, 8)))
k_gemv_gate_up_blk_id(const uint8_t *__restrict__ as_gate, const uint8_t *__restrict__ as_up, const int8_t *__restrict__ aq, const act_ds *__restrict__ ads,
                      const int32_t *__restrict__ ids, int64_t ids_stride, int K, float *__restrict__ gate, float *__restrict__ up,
                      int8_t *__restrict__ act_q, act_ds *__restrict__ act_s, int n, int64_t n_expert, int64_t n_used, int64_t nb1) {
    __shared__ float s_g[1][32], s_u[1][32];
    const int64_t slot = blockIdx.y, t = slot / n_used, e = slot % n_used;
    int64_t ex = ids[t * ids_stride + e];
    ex = ex < 0 ? 0 : (ex >= n_expert ? n_expert - 1 : ex);   // never index outside the expert stack
    const int64_t arow = t * nb1 + e % nb1;
    const row_layout L = make_row_layout(TYPE, K);
    const int64_t expert_bytes = (int64_t)n * L.row_bytes;
    gate_up_blk_phase<TYPE, 1, WAVES, R, false>(as_gate + ex * expert_bytes, as_up + ex * expert_bytes, aq + arow * K, ads + arow * (K >> 5), K,
                                                gate + slot * n, up + slot * n, n, act_q + slot * n, act_s + slot * (n >> 5), n, s_ffn_dyn, s_g, s_u);
}

int launch_gate_up_blk_id(hipStream_t s, int type, const void *as_gate, const void *as_up, const int8_t *aq, const act_ds *ads, const int32_t *ids,
                          int64_t ids_stride, int64_t K, float *gate, float *up, void *act_out, int64_t N, int64_t n_expert, int64_t n_used, int64_t nb1,
                          int64_t T) {
    const size_t lds = (size_t)(K + K / 4);
    const int64_t slots = n_used * T;
    int8_t *oq = (int8_t *)act_out;
    act_ds *os = (act_ds *)(oq + slots * N);
    const dim3 grid((unsigned)(N / 32), (unsigned)slots);
#define MI355_BLK_ID_LAUNCH(TY)                                                                                                                          \
    MI355_LAUNCH((k_gemv_gate_up_blk_id<TY, GU_WAVES, gu_rows_in_flight(TY)>), grid, dim3(64 * GU_WAVES), lds, s, (const uint8_t *)as_gate,              \
                 (const uint8_t *)as_up, aq, ads, ids, ids_stride, (int)K, gate, up, oq, os, (int)N, n_expert, n_used, nb1);
    MI355_WEIGHT_TYPE_SWITCH(type, MI355_BLK_ID_LAUNCH)
#undef MI355_BLK_ID_LAUNCH
    return launch_status("k_gemv_gate_up_blk_id");
}

}  // namespace mi355
