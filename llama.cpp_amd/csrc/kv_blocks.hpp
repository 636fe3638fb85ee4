// Where the Q8_0 / Q4_0 blocks of a quantized KV cache lie, and the quantization of one block by 32 lanes of a wave: shared by
// the cache copies (kv_quant.hip) and by the Q/K/V launch whose epilogue stores K and V into such a cache (gemv.hip).
#pragma once

#include "common.hpp"

namespace mi355 {

struct kv_place {
    int64_t first_block;   // block index, within the owning tensor, of the first block addressed
    int64_t row_blocks;    // blocks per row of the owning tensor in the device row layout; 0 = plain ggml blocks
};

// byte offsets (from the owning tensor's data) of the levels and of the f16 scale of block g
template <int TYPE>
__device__ __forceinline__ void kv_block_offsets(const kv_place &p, int64_t g, int64_t &levels, int64_t &scale) {
    constexpr int BB = TYPE == MI355_Q8_0 ? Q8_0_BYTES : Q4_0_BYTES;   // block bytes
    constexpr int LB = TYPE == MI355_Q8_0 ? 32 : 16;                   // bytes of levels per block
    if (p.row_blocks == 0) {
        scale = g * BB;
        levels = scale + 2;
    } else {
        int64_t row = 0, b = g;
        if (g >= p.row_blocks) {   // (a 1-D cache tensor is one row: no 64-bit division on the common path)
            row = g / p.row_blocks;
            b = g % p.row_blocks;
        }
        const int64_t base = row * p.row_blocks * BB;
        levels = base + b * LB;
        scale = base + p.row_blocks * LB + b * 2;
    }
}

// One block by the 32 lanes j = 0..31 of a half wave, lane j holding element j (both halves of the wave must run this with their
// own 32 values: the exchanges stay inside a half).  quantize_row_q8_0_ref (ggml/src/ggml-quants.c:194-218) bit for bit.
__device__ __forceinline__ void kv_store_q8_0_lane32(float v, int j, uint8_t *__restrict__ y, int64_t lv, int64_t sc, bool live) {
    const float amax = lanes_max<32>(fabsf(v));
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const int q = (int)roundf(v * id);
    if (!live) return;
    y[lv + j] = (uint8_t)(q & 0xFF);
    if (j == 0) *(unsigned short *)(y + sc) = float_to_half_bits(d);
}

// quantize_row_q4_0_ref (ggml/src/ggml-quants.c:39-72): the scale comes from the value of largest magnitude, the first one among
// equals; byte j of the block pairs element j (low nibble) with element j + 16 (high nibble)
__device__ __forceinline__ void kv_store_q4_0_lane32(float v, int j, uint8_t *__restrict__ y, int64_t lv, int64_t sc, bool live) {
    float amax = fabsf(v), vmax = v;
    int imax = amax == 0.0f ? 32 : j;   // "no element yet": loses every tie
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) {
        const float oa = __shfl_xor(amax, off, 64), ov = __shfl_xor(vmax, off, 64);
        const int oi = __shfl_xor(imax, off, 64);
        if (oa > amax || (oa == amax && oi < imax)) {
            amax = oa;
            vmax = ov;
            imax = oi;
        }
    }
    // d = vmax / -8, exact as an eighth with the sign flipped; the stored half takes its sign flip in the half's bits, so that a
    // zero block keeps the reference's -0.0
    const float eighth = vmax * 0.125f;
    const float d = -eighth;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const int8_t qi = (int8_t)(v * id + 8.5f);
    const unsigned u = (unsigned)(qi < 15 ? qi : 15) & 0xFu;
    const unsigned hi = (unsigned)__shfl_down((int)u, 16, 32);
    if (!live) return;
    if (j < 16) y[lv + j] = (uint8_t)(u | (hi << 4));
    if (j == 0) *(unsigned short *)(y + sc) = (unsigned short)(float_to_half_bits(eighth) ^ 0x8000u);
}

// The same two quantizations with TWO adjacent elements per lane, 16 lanes per block: lane l16 of the block holds elements
// 2 * l16 and 2 * l16 + 1 (the rotation pairs of the adjacent-pair rope mode).
__device__ __forceinline__ void kv_store_q8_0_pair16(float y0, float y1, int l16, uint8_t *__restrict__ y, int64_t lv, int64_t sc) {
    const float amax = lanes_max<16>(fmaxf(fabsf(y0), fabsf(y1)));
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const int q0 = (int)roundf(y0 * id), q1 = (int)roundf(y1 * id);
    *(unsigned short *)(y + lv + 2 * l16) = (unsigned short)((q0 & 0xFF) | ((q1 & 0xFF) << 8));
    if (l16 == 0) *(unsigned short *)(y + sc) = float_to_half_bits(d);
}
__device__ __forceinline__ void kv_store_q4_0_pair16(float y0, float y1, int l16, uint8_t *__restrict__ y, int64_t lv, int64_t sc) {
    float amax = fabsf(y0), vmax = y0;
    int imax = amax == 0.0f ? 32 : 2 * l16;
    if (fabsf(y1) > amax) {
        amax = fabsf(y1);
        vmax = y1;
        imax = 2 * l16 + 1;
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) {
        const float oa = __shfl_xor(amax, off, 64), ov = __shfl_xor(vmax, off, 64);
        const int oi = __shfl_xor(imax, off, 64);
        if (oa > amax || (oa == amax && oi < imax)) {
            amax = oa;
            vmax = ov;
            imax = oi;
        }
    }
    const float eighth = vmax * 0.125f;
    const float d = -eighth;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const int8_t a0 = (int8_t)(y0 * id + 8.5f), a1 = (int8_t)(y1 * id + 8.5f);
    const unsigned u = ((unsigned)(a0 < 15 ? a0 : 15) & 0xFu) | (((unsigned)(a1 < 15 ? a1 : 15) & 0xFu) << 8);
    const unsigned hi = (unsigned)__shfl_down((int)u, 8, 16);   // lanes 0..7 take the nibbles of elements + 16 from lanes 8..15
    if (l16 < 8) *(unsigned short *)(y + lv + 2 * l16) = (unsigned short)(u | (hi << 4));
    if (l16 == 0) *(unsigned short *)(y + sc) = (unsigned short)(float_to_half_bits(eighth) ^ 0x8000u);
}

}  // namespace mi355
