// The expert routing of a mixture-of-experts layer by the 64 lanes of one wave, shared by k_moe_route (moe.hip) and the FFN norm
// launch that continues with the router (fused.hip).
#pragma once

#include "common.hpp"

namespace mi355 {

// n_expert <= 64.  p = softmax(logits) as k_soft_max computes it for a 64-thread group (ggml_compute_forward_soft_max_f32,
// ggml-cpu.c:8959-9055); returns the rank of lane e's expert, descending by probability, ties by index
// (ggml_compute_forward_argsort_f32, ggml-cpu.c:10857, leaves ties unspecified).
__device__ __forceinline__ int moe_route_lane(float x, int e, int n_expert, float &p) {
    const bool live = e < n_expert;
    if (!live) x = -INFINITY;
    const float mx = wave_max(x);
    const float ex = live ? expf(x - mx) : 0.0f;
    const float sum = wave_sum(ex);
    const float inv = 1.0f / sum;
    p = ex * inv;
    int rank = 0;
    for (int j = 0; j < n_expert; j++) {
        const float pj = __shfl(p, j, 64);
        rank += (pj > p || (pj == p && j < e)) ? 1 : 0;
    }
    return rank;
}

}  // namespace mi355
