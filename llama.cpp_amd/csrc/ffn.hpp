// Launches of ffn.hip that other translation units call.
#pragma once
#include "common.hpp"

namespace mi355 {

// gate + up + SiLU * up + Q8_1 by groups that own whole 32-row blocks of both matrices (both of type `type`); act_out in the
// mi355_quantize_act layout of B rows of N.  B <= 4, N % 32 == 0, B * 1.25 K bytes of LDS.
int launch_gate_up_blk(hipStream_t s, int type, const void *w_gate, const void *w_up, const int8_t *aq, const act_ds *ads, int64_t K, int64_t B,
                       float *gate, float *up, int64_t out_stride, void *act_out, int64_t N);

// the same for the experts of a mixture-of-experts layer: slot t * n_used + e reads expert ids[t * ids_stride + e] of both stacks and
// activation row t * nb1 + e % nb1; gate / up f32 [slots][N], act_out rows of N per slot.  N % 32 == 0, K % 16 == 0.
int launch_gate_up_blk_id(hipStream_t s, int type, const void *as_gate, const void *as_up, const int8_t *aq, const act_ds *ads, const int32_t *ids,
                          int64_t ids_stride, int64_t K, float *gate, float *up, void *act_out, int64_t N, int64_t n_expert, int64_t n_used, int64_t nb1,
                          int64_t T);

}  // namespace mi355
