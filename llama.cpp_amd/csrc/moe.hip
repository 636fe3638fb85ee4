// Mixture-of-experts glue of llm_build_moe_ffn (src/llama.cpp:417-530) in three launches instead of eight:
//   SOFT_MAX -> ARGSORT                          k_moe_route      (expert probabilities and their descending order)
//   GET_ROWS -> SUM_ROWS -> DIV                  k_moe_weights    (weights of the selected experts, normalised)
//   MUL(weights) -> ADD ... [-> ADD(residual)]   k_moe_combine    (weighted sum of the selected experts' outputs)
// and, for a few tokens, the last two in one (k_moe_weights_combine).
// Measured and not adopted: the router product, its soft-max and the order in one launch of one group per token - 18 us for the
// 8 x 4096 f32 router of one token (a single compute unit pulling 128 KB) against 4.0 + 2.1 us for the product on eight groups and
// k_moe_route.
// Each kernel writes every tensor the separate nodes would have written, with the same arithmetic (same reduction
// order, no fused multiply-adds), so the fused and the node-by-node execution of a graph agree bit for bit.
#include "common.hpp"
#include "moe.hpp"

namespace mi355 {

// One wave per token (moe_route_lane, moe.hpp): probs = softmax(logits), order[rank] = expert.
__global__ void __launch_bounds__(64) k_moe_route(const float *__restrict__ logits, float *__restrict__ probs, int32_t *__restrict__ order,
                                                  int n_expert) {
    const int64_t t = blockIdx.x;
    const int e = threadIdx.x;
    const bool live = e < n_expert;
    float p;
    const int rank = moe_route_lane(live ? logits[t * n_expert + e] : -INFINITY, e, n_expert, p);
    if (live) {
        probs[t * n_expert + e] = p;
        order[t * n_expert + rank] = e;
    }
}

// One wave per token; n_used <= 64.  raw[t][e] = probs[t][ids[t][e]], sum[t] = sum_e raw, norm = raw / sum
// (ggml_compute_forward_get_rows_f32 ggml-cpu.c:8590, sum_rows :5678, div :5236-5305).  Lane e holds v = the probability of the e-th
// selected expert (0 beyond n_used).
__device__ __forceinline__ void moe_weights_lane(float v, int e, int n_used, float *__restrict__ raw, float *__restrict__ sum, float *__restrict__ norm) {
    const bool live = e < n_used;
    if (live) raw[e] = v;
    const float s = wave_sum(live ? v : 0.0f);
    if (e == 0) sum[0] = s;
    if (live) norm[e] = v / s;
}

__global__ void __launch_bounds__(64) k_moe_weights(const float *__restrict__ probs, const int32_t *__restrict__ ids, int64_t ids_stride,
                                                    float *__restrict__ raw, float *__restrict__ sum, float *__restrict__ norm, int n_expert,
                                                    int n_used) {
    const int64_t t = blockIdx.x;
    const int e = threadIdx.x;
    float v = 0.0f;
    if (e < n_used) v = probs[t * n_expert + ids[t * ids_stride + e]];
    moe_weights_lane(v, e, n_used, raw + t * n_used, sum + t, norm + t * n_used);
}

// One lane per 4 elements of a token's row.  scaled[t][e][:] = experts[t][e][:] * weights[t][e];
// out[t][:] = ((scaled[t][0] + scaled[t][1]) + scaled[t][2]) ... (+ residual[t][:])
__global__ void __launch_bounds__(256) k_moe_combine(const float *__restrict__ experts, const float *__restrict__ weights, float *__restrict__ scaled,
                                                     const float *__restrict__ residual, float *__restrict__ out, int64_t n_embd, int n_used) {
    const int64_t t = blockIdx.y;
    const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i0 >= n_embd) return;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int e = 0; e < n_used; e++) {
        const float wt = weights[t * n_used + e];
        const f32x4 x = *(const f32x4 *)(experts + (t * n_used + e) * n_embd + i0);
        f32x4 y;
#pragma unroll
        for (int i = 0; i < 4; i++) y[i] = mul_rn(x[i], wt);
        if (scaled) *(f32x4 *)(scaled + (t * n_used + e) * n_embd + i0) = y;
        if (e == 0) acc = y;
        else {
#pragma unroll
            for (int i = 0; i < 4; i++) acc[i] = add_rn(acc[i], y[i]);
        }
    }
    if (residual) {
        const f32x4 r = *(const f32x4 *)(residual + t * n_embd + i0);
#pragma unroll
        for (int i = 0; i < 4; i++) acc[i] = add_rn(acc[i], r[i]);
    }
    *(f32x4 *)(out + t * n_embd + i0) = acc;
}

// k_moe_weights and k_moe_combine in one launch for a few tokens: every wave works out the token's weights for itself (the same
// reduction as k_moe_weights, so the same bits); the first wave of the token's first group writes them where the caller wants them.
__global__ void __launch_bounds__(256) k_moe_weights_combine(const float *__restrict__ probs, const int32_t *__restrict__ ids, int64_t ids_stride,
                                                             float *__restrict__ raw, float *__restrict__ sum, float *__restrict__ norm, int n_expert,
                                                             const float *__restrict__ experts, float *__restrict__ scaled,
                                                             const float *__restrict__ residual, float *__restrict__ out, int64_t n_embd, int n_used) {
    const int64_t t = blockIdx.y;
    const int lane = threadIdx.x & 63;
    float v = 0.0f;
    if (lane < n_used) v = probs[t * n_expert + ids[t * ids_stride + lane]];
    const float s = wave_sum(v);
    const float wn = v / s;
    if (raw != nullptr && blockIdx.x == 0 && threadIdx.x < 64) {
        if (lane < n_used) {
            raw[t * n_used + lane] = v;
            norm[t * n_used + lane] = wn;
        }
        if (lane == 0) sum[t] = s;
    }
    const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    const bool live = i0 < n_embd;   // every lane takes part in the broadcasts of the weights
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int e = 0; e < n_used; e++) {
        const float wt = __shfl(wn, e, 64);
        if (!live) continue;
        const f32x4 x = *(const f32x4 *)(experts + (t * n_used + e) * n_embd + i0);
        f32x4 y;
#pragma unroll
        for (int i = 0; i < 4; i++) y[i] = mul_rn(x[i], wt);
        if (scaled) *(f32x4 *)(scaled + (t * n_used + e) * n_embd + i0) = y;
        if (e == 0) acc = y;
        else {
#pragma unroll
            for (int i = 0; i < 4; i++) acc[i] = add_rn(acc[i], y[i]);
        }
    }
    if (!live) return;
    if (residual) {
        const f32x4 r = *(const f32x4 *)(residual + t * n_embd + i0);
#pragma unroll
        for (int i = 0; i < 4; i++) acc[i] = add_rn(acc[i], r[i]);
    }
    *(f32x4 *)(out + t * n_embd + i0) = acc;
}

}  // namespace mi355

using namespace mi355;

extern "C" {

int mi355_moe_route(void *stream, const float *logits, float *probs, int32_t *order, int64_t n_expert, int64_t T) {
    MI355_REQUIRE(n_expert >= 1 && n_expert <= 64, "moe_route: %lld experts (1..64 supported)", (long long)n_expert);
    MI355_REQUIRE(T >= 0 && T < 0x7fffffff, "moe_route: bad token count");
    MI355_REQUIRE(logits && probs && order, "moe_route: null operand");
    if (T == 0) return MI355_OK;
    MI355_LAUNCH(k_moe_route, dim3((unsigned)T), dim3(64), 0, (hipStream_t)stream, logits, probs, order, (int)n_expert);
    return launch_status("k_moe_route");
}

int mi355_moe_weights(void *stream, const float *probs, const int32_t *ids, int64_t ids_stride, float *raw, float *sum, float *norm,
                      int64_t n_expert, int64_t n_used, int64_t T) {
    MI355_REQUIRE(n_expert >= 1 && n_used >= 1 && n_used <= 64 && n_used <= n_expert, "moe_weights: bad expert counts");
    MI355_REQUIRE(ids_stride >= n_used, "moe_weights: ids_stride < n_used");
    MI355_REQUIRE(T >= 0 && T < 0x7fffffff, "moe_weights: bad token count");
    MI355_REQUIRE(probs && ids && raw && sum && norm, "moe_weights: null operand");
    if (T == 0) return MI355_OK;
    MI355_LAUNCH(k_moe_weights, dim3((unsigned)T), dim3(64), 0, (hipStream_t)stream, probs, ids, ids_stride, raw, sum, norm, (int)n_expert,
                       (int)n_used);
    return launch_status("k_moe_weights");
}

int mi355_moe_combine(void *stream, const float *experts, const float *weights, float *scaled, const float *residual, float *out,
                      int64_t n_embd, int64_t n_used, int64_t T) {
    MI355_REQUIRE(n_embd > 0 && n_embd % 4 == 0 && n_used >= 1 && n_used <= 64, "moe_combine: bad shape");
    MI355_REQUIRE(T >= 0 && T <= 65535, "moe_combine: bad token count");
    MI355_REQUIRE(experts && weights && out, "moe_combine: null operand");
    MI355_REQUIRE((((uintptr_t)experts | (uintptr_t)scaled | (uintptr_t)residual | (uintptr_t)out) & 15) == 0, "moe_combine: operands must be 16-byte aligned");
    if (T == 0) return MI355_OK;
    const dim3 grid((unsigned)((n_embd / 4 + 255) / 256), (unsigned)T);
    MI355_LAUNCH(k_moe_combine, grid, dim3(256), 0, (hipStream_t)stream, experts, weights, scaled, residual, out, n_embd, (int)n_used);
    return launch_status("k_moe_combine");
}

int mi355_moe_weights_combine(void *stream, const float *probs, const int32_t *ids, int64_t ids_stride, float *raw, float *sum, float *norm,
                              int64_t n_expert, const float *experts, float *scaled, const float *residual, float *out, int64_t n_embd, int64_t n_used,
                              int64_t T) {
    MI355_REQUIRE(n_expert >= 1 && n_used >= 1 && n_used <= 64 && n_used <= n_expert && ids_stride >= n_used, "moe_weights_combine: bad expert counts");
    MI355_REQUIRE(n_embd > 0 && n_embd % 4 == 0 && T >= 0 && T <= 65535, "moe_weights_combine: bad shape");
    MI355_REQUIRE(probs && ids && experts && out, "moe_weights_combine: null operand");
    MI355_REQUIRE((raw != nullptr) == (sum != nullptr) && (raw != nullptr) == (norm != nullptr), "moe_weights_combine: the weights' outputs are given all three or not at all");
    MI355_REQUIRE((((uintptr_t)experts | (uintptr_t)scaled | (uintptr_t)residual | (uintptr_t)out) & 15) == 0, "moe_weights_combine: operands must be 16-byte aligned");
    if (T == 0) return MI355_OK;
    const dim3 grid((unsigned)((n_embd / 4 + 255) / 256), (unsigned)T);
    MI355_LAUNCH(k_moe_weights_combine, grid, dim3(256), 0, (hipStream_t)stream, probs, ids, ids_stride, raw, sum, norm, (int)n_expert, experts, scaled, residual,
                 out, n_embd, (int)n_used);
    return launch_status("k_moe_weights_combine");
}

}  // extern "C"
