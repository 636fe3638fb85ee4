// Arguments shared by the flash-attention kernels (vector kernel for decode, matrix-core kernel for prefill).
#pragma once

#include "common.hpp"

namespace mi355 {

// A Q8_0 / Q4_0 operand read block by block where it lies (no f16 copy).  Block g of the owning tensor sits at g * block bytes
// (row_blocks == 0: plain ggml blocks, the f16 scale in front of the levels) or, for a tensor in the device row layout, in row
// g / row_blocks at position g % row_blocks (the levels of a row first, its scales behind them).  The (cell 0, head) row starts at
// block first_block + head * head_blocks, and in the device row layout base is the owner's row that holds all of cell 0's blocks
// (first_block + head * head_blocks + D / 32 <= row_blocks for every head); a cell further on, the levels lie cell_lv bytes and the scales cell_sc bytes further on:
// both nb1 for plain blocks and where a cell's stride is a whole number of the owner's rows; (blocks per cell) * 32 or 16 and
// (blocks per cell) * 2 where all cells lie in ONE row of the owner (llama.cpp's cache tensors are 1-D: one row of all cells).
struct kv_src {
    const uint8_t *base;
    int64_t first_block, row_blocks, head_blocks;
    int64_t cell_lv, cell_sc;
};

struct fattn_args {
    const uint8_t *q, *k, *v, *mask;
    int type_k = MI355_F16, type_v = MI355_F16;   // k_fattn_vec only: MI355_Q8_0 / MI355_Q4_0 operands are described by kq / vq
    kv_src kq = {nullptr, 0, 0, 0, 0, 0}, vq = {nullptr, 0, 0, 0, 0, 0};
    float *dst;      // [D, Hq, Nq]
    int8_t *act_q;   // optional: Q8_1 of dst rows (Hq*D elements per query) in the split activation layout
    act_ds *act_s;
    float *ws;       // partial results when n_splits > 1: [Nq][Hq][n_splits][D + 2]
    const int32_t *kv_extent;   // prefill, optional: per tile of 32 queries, the number of leading cells after which every
                                // mask entry of the tile's rows is -inf (see k_mask_extent); null = all Nkv cells
    int64_t Nq, Nkv, Hq, Hkv;
    size_t q_nb1, q_nb2, k_nb1, k_nb2, v_nb1, v_nb2, mask_nb1;
    float scale, max_bias, softcap;
    float m0, m1;
    unsigned n_head_log2;
    int n_splits;
    int groups;      // head groups of R per kv head: Hq / Hkv == R * groups
    int64_t cells_per_split;
};

// Q8_1 of one value per lane, 32 consecutive lanes = one block (quantize_row_q8_1_ref,
// ggml/src/ggml-quants.c:220-253); e = element index inside the query row of k elements
__device__ __forceinline__ void quantize_lane32(float v, int8_t *__restrict__ qrow, act_ds *__restrict__ srow, int64_t e) {
    const float amax = lanes_max<32>(fabsf(v));
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const int q = (int)roundf(v * id);
    const int sum = lanes_sum_i<32>(q);
    qrow[e] = (int8_t)q;
    if ((e & 31) == 0) {
        act_ds o;
        o.d = half_bits_to_float(float_to_half_bits(d));
        o.sum = sum;
        srow[e >> 5] = o;
    }
}

// f16 matrix-core kernel for many query rows; returns MI355_OK, an error, or 1 when the shape is not served
int launch_fattn_mma(hipStream_t s, fattn_args &a, int64_t D, size_t ws_bytes);
// the same for a few query rows (decode): one kv split per group, partials merged by k_fattn_combine
int launch_fattn_mma_dec(hipStream_t s, fattn_args &a, int64_t D);

// the vector kernel on f16 / Q8_0 / Q4_0 operands in any mix (a.type_k, a.type_v, a.kq, a.vq filled in), splits merged by
// k_fattn_combine; for the shapes the matrix-core kernels do not take, and for every quantized cache read in place
int launch_fattn_vec_any(hipStream_t s, fattn_args &a, int64_t D);
// mi355_flash_attn_ext_quant's arguments with typed K / V, served by the vector kernel alone (k, v: the f16 operands' data; a
// quantized operand is described by kq / vq and its k_nb1 / v_nb1)
int fattn_vec_kv(hipStream_t s, const float *q, const void *k, int type_k, const kv_src &kq, const void *v, int type_v, const kv_src &vq,
                 const void *mask, float *dst, int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv, size_t q_nb1, size_t q_nb2, size_t k_nb1,
                 size_t k_nb2, size_t v_nb1, size_t v_nb2, size_t mask_nb1, float scale, float max_bias, float logit_softcap, void *ws,
                 size_t ws_bytes, void *act);

// one query token over at most 512 cells of an f16 cache, head size 128, up to four query heads per kv head: one launch, one wave
// per 64 cells, states merged in LDS (fattn_stream.hip); returns 1 when the shape is not served
int launch_fattn_dec_short(hipStream_t s, fattn_args &a, int64_t D);
// one query token over a long f16 cache, head size 128, up to four query heads per kv head: per-wave streaming through LDS
// (fattn_stream.hip); sets a.n_splits for k_fattn_combine; returns 1 when the shape is not served
int launch_fattn_dec_stream(hipStream_t s, fattn_args &a, int64_t D, size_t ws_bytes);

// the same over a Q8_0 / Q4_0 cache in the device row layout, read in place (a.type_k, a.type_v, a.kq, a.vq filled in)
int launch_fattn_dec_stream_q(hipStream_t s, fattn_args &a, int64_t D, size_t ws_bytes);

}  // namespace mi355
