// Tile images: the operand format of the wide-tile K-quant GEMM (mmq_w.hip).
//
// An int8 matrix of R rows x K columns (K a multiple of 256) is stored as tiles of 16 rows x 64 columns = 1 KiB, ordered
// [row block][k block]; inside a tile, the 16-byte chunk c (0..3) of row r (0..15) sits at r * 64 + ((c ^ ((r >> 2) & 3)) << 4):
// the image of the tile in LDS, so that one wave-wide 16-byte-per-lane transfer moves a tile and ds_read_b128 of 32
// consecutive rows is conflict-free.  Rows are padded to a multiple of 16.
//
//   activations (mi355_quantize_act_q8k_tiled):   int8 q image [B16 x K]
//                                                 aux [K/256][cb_pad][576]: per 16 rows { float d8[16]; fp16 bs[16][16] }
//                                                 bs = {bsum_j & 63 (j = 0..7), bsum_j >> 6 (j = 0..7)}; cb_pad = B16/16 rounded up to 16
//   weights (mi355_kq_unpack_tiles):              int8 hi image [N16 x K], int8 lo image [N16 x K]   (value = R * hi + lo;
//                                                 Q4_K: sc * n with R = 8, Q5_K: sc * n with R = 16, Q6_K: sc * (l - 32) with R = 64)
//                                                 aux [K/256][rb_pad][640]: per 16 rows
//                                                 { fp16 m[16][16] = {min_j, 64 * min_j}; float d[16]; float dmin[16] }
//                                                 (Q6_K has no minima: zeros there, so that its images can ride in a launch of the
//                                                 kernel that handles them); rb_pad = N16/16 rounded up to 8
// Levels, scales and sums are those of quantize_row_q8_K_ref (ggml/src/ggml-quants.c:2479-2516) and of the Q4_K / Q6_K
// dequantizers (ggml/src/ggml-quants.c:1280-1302, 1690-1719).
#pragma once
#include "common.hpp"
#include "q8k.hpp"

namespace mi355 {

constexpr int WT_TILE = 1024;
constexpr int WT_A_AUX = 576;

__host__ __device__ constexpr int wt_w_aux_bytes(int) { return 640; }
__host__ __device__ inline int64_t wt_rb_pad(int64_t N) { return (((N + 15) >> 4) + 7) & ~(int64_t)7; }
__host__ __device__ inline int64_t wt_cb_pad(int64_t B) { return (((B + 15) >> 4) + 15) & ~(int64_t)15; }

// byte offset of element (row, k) of an image with K columns; k a multiple of 16 addresses a whole chunk
__host__ __device__ inline int64_t wt_tile_off(int64_t row, int64_t k, int64_t K) {
    const int r = (int)(row & 15), c = (int)((k >> 4) & 3);
    return ((row >> 4) * (K >> 6) + (k >> 6)) * WT_TILE + r * 64 + ((c ^ ((r >> 2) & 3)) << 4) + (k & 15);
}

__host__ __device__ inline size_t wt_act_bytes(int64_t K, int64_t B) {
    const size_t b16 = (size_t)((B + 15) & ~(int64_t)15);
    // + 1 KiB: the scale entries of a 128-row tile (4608 bytes) are fetched as five 1 KiB transfers
    return b16 * (size_t)K + (size_t)(K >> 8) * (size_t)wt_cb_pad(B) * WT_A_AUX + 1024;
}
// offset of the per-super-block entries behind the two images
__host__ __device__ inline size_t wt_w_aux_offset(int64_t N, int64_t K) { return 2 * (size_t)((N + 15) & ~(int64_t)15) * (size_t)K; }
__host__ __device__ inline size_t wt_weight_bytes(int type, int64_t N, int64_t K) {
    return wt_w_aux_offset(N, K) + (size_t)(K >> 8) * (size_t)wt_rb_pad(N) * (size_t)wt_w_aux_bytes(type);
}

// q8k_quantize_wave writing the tiled form: one wave quantizes super-block sb of activation row `row` (lane l holds elements
// 4l .. 4l+3; rows >= B must be given zeros and come out as zeros).  act: base of the tiled activation buffer of B rows.
__device__ __forceinline__ void q8k_quantize_wave_tiled(const f32x4 &v, int lane, uint8_t *__restrict__ act, int64_t K, int64_t B, int64_t row, int64_t sb) {
    u32 packed;
    float d;
    int sum;
    q8k_quantize_values(v, lane, packed, d, sum);
    const int64_t b16 = (B + 15) & ~(int64_t)15;
    *(u32 *)(act + wt_tile_off(row, sb * QKK + lane * 4, K)) = packed;
    uint8_t *e = act + b16 * K + (sb * wt_cb_pad(B) + (row >> 4)) * WT_A_AUX;
    const int r = (int)(row & 15);
    if (lane == 0) *(float *)(e + r * 4) = d;
    if ((lane & 7) == 0) {
        _Float16 *bs = (_Float16 *)(e + 64 + r * 32);
        bs[lane >> 3] = (_Float16)(float)(sum & 63);
        bs[8 + (lane >> 3)] = (_Float16)(float)(sum >> 6);
    }
}

// Sum of a product's K slices (partial sums [slice][B][N]) + residual -> dst rows, each row then RMS-normalised, multiplied by w and
// written as y (optional) and as its part of the tile image act_out: one launch, the bits of the slice sum followed by the norm
// launch (mmq_w.hip).  N <= 4096, a multiple of 256; 16-byte aligned operands.
void launch_split_sum_norm(hipStream_t s, const float *part, float *dst, const float *residual, int64_t N, int64_t B, int64_t dst_stride, int n_slices,
                           const float *w, float eps, float *y, int64_t y_stride, void *act_out);

// MUL_MAT_ID: the (token, expert slot) pairs sorted by expert (k_route_slots, mmq_k.hip).  Column c of the sorted list reads
// activation row act_row[c] and writes dst row dst_row[c]; tiles[4 i] = {expert, first column, end column of the expert, 0} for
// column tiles of at most bn columns; *n_tiles tiles are in use.  At most 256 experts.
void launch_route_slots(hipStream_t s, const int32_t *ids, int64_t ids_stride, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T, int bn,
                        int32_t *act_row, int32_t *dst_row, int32_t *tiles, int32_t *n_tiles);

}  // namespace mi355
