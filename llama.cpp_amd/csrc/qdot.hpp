// Per-lane integer dot products of quantized weight chunks against Q8_1 activations.
//
// Work unit ("chunk"): what one lane consumes per step.  Chunk c of a row is taken by lane
// c % 64 at step c / 64, so a wave walks a row in consecutive 16-byte, 16-byte-aligned loads.
//   Q4_0 / Q8_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL : chunk = one 32-element block.
//   IQ4_XS      : chunk = one 32-element block of its super-block; 8 chunks share the 8-byte header.
//   Q4_K        : chunk = 32 bytes of qs = sub-blocks 2g (low nibbles) and 2g+1 (high nibbles),
//                 64 elements; 4 chunks per super-block share its 16-byte header.
//   Q5_K        : as Q4_K, plus the 32 bytes of qh that carry the fifth bit of all eight sub-blocks.
//   Q6_K        : chunk = 16 bytes of ql + the matching 16 bytes of qh = two 16-element
//                 scale groups, 32 elements; 8 chunks per super-block.
// The same functions feed the GEMV kernels and the parity entry point that dumps the
// integer dots, so what is checked bit-for-bit is what ships.
#pragma once

#include "common.hpp"

namespace mi355 {

// Device layout of one weight row (see mi355_kernels.h): byte offsets of the per-row regions.
struct row_layout {
    int64_t row_bytes;
    int off_b;   // IQ4_XS: {fp16 d, scales_h, scales_l[4]} array.  Q4_0/Q8_0/IQ4_NL: fp16 d array.  Q4_1: {fp16 d, fp16 m} array.  Q5_0/Q5_1: fifth-bit words.  Q6_K: qh array
    int off_c;   // Q5_0: fp16 d array.  Q5_1: {fp16 d, fp16 m} array.  Q6_K: scales array
    int off_d;   // Q6_K: fp16 d array
};

__host__ __device__ inline row_layout make_row_layout(int type, int64_t k) {
    row_layout L = {0, 0, 0, 0};
    const int64_t nb = k / type_block_elems(type);
    L.row_bytes = nb * type_block_bytes(type);
    switch (type) {
        case MI355_Q4_0: case MI355_IQ4_NL: case MI355_Q4_1: L.off_b = (int)(nb * 16); break;
        case MI355_Q5_0: case MI355_Q5_1: L.off_b = (int)(nb * 16); L.off_c = (int)(nb * 20); break;
        case MI355_Q8_0: L.off_b = (int)(nb * 32); break;
        case MI355_IQ4_XS: L.off_b = (int)(nb * 128); break;
        case MI355_Q6_K: L.off_b = (int)(nb * 128); L.off_c = (int)(nb * 192); L.off_d = (int)(nb * 208); break;
        default: break;
    }
    return L;
}
__host__ inline bool layout_aligned(const void *W, const row_layout &L) {
    return ((uintptr_t)W & 15) == 0 && (L.row_bytes & 15) == 0 && (L.off_b & 15) == 0 && (L.off_c & 15) == 0;
}

// Byte-load GEMV for weight rows that are not 16-byte aligned, any batch (mul_mat.hip).
// act: split activation layout holding B rows of K; residual may be null or alias dst.
int gemv_unaligned(hipStream_t s, int type, const void *W, const void *act, float *dst, const float *residual, int64_t N,
                   int64_t K, int64_t B, int64_t dst_stride);

// 6-bit (scale, min) of sub-block j from the 12 packed bytes held in three dwords
// (get_scale_min_k4, ggml/src/ggml-quants.c:631-638); u0 = b[0..3], u1 = b[4..7], u2 = b[8..11]
__device__ __forceinline__ void q4k_scale_min(u32 u0, u32 u1, u32 u2, int j, int &sc, int &mn) {
    const int sh = 8 * (j & 3);
    const u32 b_lo = (u0 >> sh) & 0xFFu, b_mid = (u1 >> sh) & 0xFFu, b_hi = (u2 >> sh) & 0xFFu;
    if (j < 4) {
        sc = (int)(b_lo & 63u);
        mn = (int)(b_mid & 63u);
    } else {
        sc = (int)((b_hi & 0x0Fu) | ((b_lo >> 6) << 4));
        mn = (int)((b_hi >> 4) | ((b_mid >> 6) << 4));
    }
}

// Integer results of one weight chunk against one activation chunk.
struct chunk_dots {
    int i0, i1;
};

// wq<TYPE>::accumulate adds one chunk's contribution to a running sum.  Every multiply, add and fused
// multiply-add is spelled out: left to the compiler, the choice of which product of a sum gets fused
// differs between kernel instantiations, and launches that must agree bit for bit would not.
template <int TYPE> struct wq;

// ---------------------------------------------------------------- Q4_0
template <> struct wq<MI355_Q4_0> {
    static constexpr int CHUNK = 32;
    struct chunk { u32x4 qs; float d; };
    struct act { u32x4 a0, a1; float d; int sum; };
    static __device__ __forceinline__ chunk load_w(const uint8_t *__restrict__ row, const row_layout &L, int c) {
        chunk w;
        w.qs = load_stream16(row + c * 16);
        w.d = half_bits_to_float(*(const unsigned short *)(row + L.off_b + c * 2));
        return w;
    }
    static __device__ __forceinline__ act load_a(const int8_t *__restrict__ q, const act_ds *__restrict__ ds, int c) {
        act A;
        A.a0 = load16(q + c * 32);
        A.a1 = load16(q + c * 32 + 16);
        const act_ds s = ds[c];
        A.d = s.d;
        A.sum = s.sum;
        return A;
    }
    // i0 = sum (nibble-8)*q over the block (ggml-cpu-quants.c:2496-2505)
    static __device__ __forceinline__ chunk_dots dots(const chunk &w, const act &A) {
        int s = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            s = dot4((int)(w.qs[i] & 0x0F0F0F0Fu), (int)A.a0[i], s);
            s = dot4((int)((w.qs[i] >> 4) & 0x0F0F0F0Fu), (int)A.a1[i], s);
        }
        chunk_dots r = {s - 8 * A.sum, 0};
        return r;
    }
    static __device__ __forceinline__ float accumulate(float acc, const chunk &w, const act &A, const chunk_dots &r) {
        return __builtin_fmaf(w.d, mul_rn(A.d, (float)r.i0), acc);
    }
};

// ---------------------------------------------------------------- Q8_0
template <> struct wq<MI355_Q8_0> {
    static constexpr int CHUNK = 32;
    struct chunk { u32x4 q0, q1; float d; };
    struct act { u32x4 a0, a1; float d; };
    static __device__ __forceinline__ chunk load_w(const uint8_t *__restrict__ row, const row_layout &L, int c) {
        chunk w;
        // the two loads of a wave interleave 16-byte pieces of the same 128-byte lines: a streaming
        // (non-temporal) hint would fetch each line from HBM twice, so these stay ordinary loads
        w.q0 = load16(row + c * 32);
        w.q1 = load16(row + c * 32 + 16);
        w.d = half_bits_to_float(*(const unsigned short *)(row + L.off_b + c * 2));
        return w;
    }
    static __device__ __forceinline__ act load_a(const int8_t *__restrict__ q, const act_ds *__restrict__ ds, int c) {
        act A;
        A.a0 = load16(q + c * 32);
        A.a1 = load16(q + c * 32 + 16);
        A.d = ds[c].d;
        return A;
    }
    static __device__ __forceinline__ chunk_dots dots(const chunk &w, const act &A) {   // ggml-cpu-quants.c:3919-3927
        int s = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            s = dot4((int)w.q0[i], (int)A.a0[i], s);
            s = dot4((int)w.q1[i], (int)A.a1[i], s);
        }
        chunk_dots r = {s, 0};
        return r;
    }
    static __device__ __forceinline__ float accumulate(float acc, const chunk &w, const act &A, const chunk_dots &r) {
        return __builtin_fmaf(w.d, mul_rn(A.d, (float)r.i0), acc);
    }
};

// ---------------------------------------------------------------- IQ4_NL
// block_iq4_nl (ggml/src/ggml-common.h:399-404): the Q4_0 bytes, but nibble n stands for kvalues_iq4nl[n]
// (ggml/src/ggml-cpu/ggml-cpu-quants.c:1672); ggml_vec_dot_iq4_nl_q8_0 (:11188, scalar tail :11368-11377).
// The sixteen table bytes sit in four dwords; two byte permutes pick among the lower and the upper eight by the low three bits
// of each nibble, bit 3 then chooses between the two results.
__device__ __forceinline__ u32 iq4nl_lookup4(u32 nibbles) {   // four nibbles, one per byte -> four table entries
    constexpr u32 T0 = 0xBFAD9881u, T1 = 0xF6EADDCFu, T2 = 0x26190D01u, T3 = 0x71594535u;   // -127 -104 -83 -65 | -49 -35 -22 -10 | 1 13 25 38 | 53 69 89 113
    const u32 sel = nibbles & 0x07070707u;
    const u32 lo = __builtin_amdgcn_perm(T1, T0, sel);
    const u32 hi = __builtin_amdgcn_perm(T3, T2, sel);
    const u32 m = ((nibbles >> 3) & 0x01010101u) * 0xFFu;
    return (lo & ~m) | (hi & m);
}
template <> struct wq<MI355_IQ4_NL> {
    static constexpr int CHUNK = 32;
    typedef wq<MI355_Q4_0>::chunk chunk;
    typedef wq<MI355_Q8_0>::act act;
    static __device__ __forceinline__ chunk load_w(const uint8_t *__restrict__ row, const row_layout &L, int c) { return wq<MI355_Q4_0>::load_w(row, L, c); }
    static __device__ __forceinline__ act load_a(const int8_t *__restrict__ q, const act_ds *__restrict__ ds, int c) { return wq<MI355_Q8_0>::load_a(q, ds, c); }
    static __device__ __forceinline__ chunk_dots dots(const chunk &w, const act &A) {
        int s = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            s = dot4((int)iq4nl_lookup4(w.qs[i] & 0x0F0F0F0Fu), (int)A.a0[i], s);
            s = dot4((int)iq4nl_lookup4((w.qs[i] >> 4) & 0x0F0F0F0Fu), (int)A.a1[i], s);
        }
        chunk_dots r = {s, 0};
        return r;
    }
    static __device__ __forceinline__ float accumulate(float acc, const chunk &w, const act &A, const chunk_dots &r) {
        return __builtin_fmaf(w.d, mul_rn(A.d, (float)r.i0), acc);
    }
};

// ---------------------------------------------------------------- IQ4_XS
// block_iq4_xs (ggml/src/ggml-common.h:406-412): eight blocks of IQ4_NL levels under one fp16 d; block ib is scaled by
// d * (ls - 32), ls = scales_l nibble ib | two bits of scales_h << 4 (dequantize_row_iq4_xs, ggml/src/ggml-quants.c:2454-2475;
// ggml_vec_dot_iq4_xs_q8_K, ggml/src/ggml-cpu/ggml-cpu-quants.c:11381, scalar tail :11647-11676).
// hdr = the header's two dwords: {d | scales_h << 16, scales_l[0..3]}
__device__ __forceinline__ float iq4xs_block_scale(u32 h0, u32 h1, int ib) {
    const int ls = (int)(((h1 >> (4 * ib)) & 0xFu) | (((h0 >> (16 + 2 * ib)) & 3u) << 4));
    return mul_rn(half_bits_to_float((unsigned short)(h0 & 0xFFFFu)), (float)(ls - 32));
}
template <> struct wq<MI355_IQ4_XS> {
    static constexpr int CHUNK = 32;
    typedef wq<MI355_Q4_0>::chunk chunk;
    typedef wq<MI355_Q8_0>::act act;
    static __device__ __forceinline__ chunk load_w(const uint8_t *__restrict__ row, const row_layout &L, int c) {
        chunk w;
        w.qs = load_stream16(row + c * 16);
        const uint2 h = *(const uint2 *)(row + L.off_b + (c >> 3) * 8);   // the same eight bytes for the eight lanes of a super-block
        w.d = iq4xs_block_scale(h.x, h.y, c & 7);
        return w;
    }
    static __device__ __forceinline__ act load_a(const int8_t *__restrict__ q, const act_ds *__restrict__ ds, int c) { return wq<MI355_Q8_0>::load_a(q, ds, c); }
    static __device__ __forceinline__ chunk_dots dots(const chunk &w, const act &A) { return wq<MI355_IQ4_NL>::dots(w, A); }
    static __device__ __forceinline__ float accumulate(float acc, const chunk &w, const act &A, const chunk_dots &r) {
        return __builtin_fmaf(w.d, mul_rn(A.d, (float)r.i0), acc);
    }
};

// ---------------------------------------------------------------- Q4_1, Q5_0, Q5_1
// block_q4_1 / q5_0 / q5_1 (ggml/src/ggml-common.h:168-201): value = d * level (+ m), level = nibble (| fifth bit << 4)
// (- 16 for Q5_0); ggml_vec_dot_q4_1_q8_1, _q5_0_q8_0, _q5_1_q8_1 (ggml/src/ggml-cpu/ggml-cpu-quants.c:2511, 2804, 3159; scalar
// tails :2784-2799, :3131-3153, :3504-3526).  The block minimum meets the activation through d_a * sum of its levels.
__device__ __forceinline__ u32 spread4(u32 bits) {   // bits 0..3 -> bit 4 of bytes 0..3
    return (((bits & 0xFu) * 0x00204081u) & 0x01010101u) << 4;
}
template <> struct wq<MI355_Q4_1> {
    static constexpr int CHUNK = 32;
    struct chunk { u32x4 qs; float d, m; };
    typedef wq<MI355_Q4_0>::act act;
    static __device__ __forceinline__ chunk load_w(const uint8_t *__restrict__ row, const row_layout &L, int c) {
        chunk w;
        w.qs = load_stream16(row + c * 16);
        const u32 dm = *(const u32 *)(row + L.off_b + c * 4);
        w.d = half_bits_to_float((unsigned short)(dm & 0xFFFFu));
        w.m = half_bits_to_float((unsigned short)(dm >> 16));
        return w;
    }
    static __device__ __forceinline__ act load_a(const int8_t *__restrict__ q, const act_ds *__restrict__ ds, int c) { return wq<MI355_Q4_0>::load_a(q, ds, c); }
    static __device__ __forceinline__ chunk_dots dots(const chunk &w, const act &A) {
        int s = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            s = dot4((int)(w.qs[i] & 0x0F0F0F0Fu), (int)A.a0[i], s);
            s = dot4((int)((w.qs[i] >> 4) & 0x0F0F0F0Fu), (int)A.a1[i], s);
        }
        chunk_dots r = {s, 0};
        return r;
    }
    static __device__ __forceinline__ float accumulate(float acc, const chunk &w, const act &A, const chunk_dots &r) {
        const float t = __builtin_fmaf(w.d, mul_rn(A.d, (float)r.i0), mul_rn(w.m, mul_rn(A.d, (float)A.sum)));
        return add_rn(acc, t);
    }
};
template <> struct wq<MI355_Q5_0> {
    static constexpr int CHUNK = 32;
    struct chunk { u32x4 qs; u32 qh; float d; };
    typedef wq<MI355_Q4_0>::act act;
    static __device__ __forceinline__ chunk load_w(const uint8_t *__restrict__ row, const row_layout &L, int c) {
        chunk w;
        w.qs = load_stream16(row + c * 16);
        w.qh = *(const u32 *)(row + L.off_b + c * 4);
        w.d = half_bits_to_float(*(const unsigned short *)(row + L.off_c + c * 2));
        return w;
    }
    static __device__ __forceinline__ act load_a(const int8_t *__restrict__ q, const act_ds *__restrict__ ds, int c) { return wq<MI355_Q4_0>::load_a(q, ds, c); }
    // sum (level - 16) * q: bit j of qh belongs to element j; elements 4i..4i+3 are the low nibbles of dword i, 16+4i.. the high ones
    static __device__ __forceinline__ int level_dot(const u32x4 &qs, u32 qh, const u32x4 &a0, const u32x4 &a1) {
        int s = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            s = dot4((int)((qs[i] & 0x0F0F0F0Fu) | spread4(qh >> (4 * i))), (int)a0[i], s);
            s = dot4((int)(((qs[i] >> 4) & 0x0F0F0F0Fu) | spread4(qh >> (16 + 4 * i))), (int)a1[i], s);
        }
        return s;
    }
    static __device__ __forceinline__ chunk_dots dots(const chunk &w, const act &A) {
        chunk_dots r = {level_dot(w.qs, w.qh, A.a0, A.a1) - 16 * A.sum, 0};
        return r;
    }
    static __device__ __forceinline__ float accumulate(float acc, const chunk &w, const act &A, const chunk_dots &r) {
        return __builtin_fmaf(w.d, mul_rn(A.d, (float)r.i0), acc);
    }
};
template <> struct wq<MI355_Q5_1> {
    static constexpr int CHUNK = 32;
    struct chunk { u32x4 qs; u32 qh; float d, m; };
    typedef wq<MI355_Q4_0>::act act;
    static __device__ __forceinline__ chunk load_w(const uint8_t *__restrict__ row, const row_layout &L, int c) {
        chunk w;
        w.qs = load_stream16(row + c * 16);
        w.qh = *(const u32 *)(row + L.off_b + c * 4);
        const u32 dm = *(const u32 *)(row + L.off_c + c * 4);
        w.d = half_bits_to_float((unsigned short)(dm & 0xFFFFu));
        w.m = half_bits_to_float((unsigned short)(dm >> 16));
        return w;
    }
    static __device__ __forceinline__ act load_a(const int8_t *__restrict__ q, const act_ds *__restrict__ ds, int c) { return wq<MI355_Q4_0>::load_a(q, ds, c); }
    static __device__ __forceinline__ chunk_dots dots(const chunk &w, const act &A) {
        chunk_dots r = {wq<MI355_Q5_0>::level_dot(w.qs, w.qh, A.a0, A.a1), 0};
        return r;
    }
    static __device__ __forceinline__ float accumulate(float acc, const chunk &w, const act &A, const chunk_dots &r) {
        const float t = __builtin_fmaf(w.d, mul_rn(A.d, (float)r.i0), mul_rn(w.m, mul_rn(A.d, (float)A.sum)));
        return add_rn(acc, t);
    }
};

// ---------------------------------------------------------------- Q4_K
template <> struct wq<MI355_Q4_K> {
    static constexpr int CHUNK = 64;
    struct chunk { u32x4 q0, q1; float d, dmin, scA, mA, scB, mB; };
    struct act { u32x4 a0lo, a0hi, a1lo, a1hi; float d0, d1, ds0, ds1; };
    static __device__ __forceinline__ chunk load_w(const uint8_t *__restrict__ row, const row_layout &, int c) {
        chunk w;
        const int sb = c >> 2, g = c & 3;
        const uint8_t *blk = row + sb * Q4_K_BYTES;
        // header and both qs loads touch the same 128-byte lines from three instructions: ordinary
        // (temporal) loads, so the line is fetched from HBM once and the other two hit in cache
        const u32x4 hdr = load16(blk);   // d, dmin, 12 scale bytes: same address for the 4 lanes of a super-block
        w.q0 = load16(blk + 16 + g * 32);
        w.q1 = load16(blk + 32 + g * 32);
        w.d = half_bits_to_float((unsigned short)(hdr[0] & 0xFFFFu));
        w.dmin = half_bits_to_float((unsigned short)(hdr[0] >> 16));
        // all eight 6-bit (scale, min) pairs at once, branch-free (get_scale_min_k4, ggml-quants.c:631-638)
        const u32 s_lo = hdr[1] & 0x3F3F3F3Fu, m_lo = hdr[2] & 0x3F3F3F3Fu;
        const u32 s_hi = (hdr[3] & 0x0F0F0F0Fu) | (((hdr[1] >> 6) & 0x03030303u) << 4);
        const u32 m_hi = ((hdr[3] >> 4) & 0x0F0F0F0Fu) | (((hdr[2] >> 6) & 0x03030303u) << 4);
        const u32 S = g < 2 ? s_lo : s_hi, M = g < 2 ? m_lo : m_hi;
        const int sh = 16 * (g & 1);
        w.scA = (float)((S >> sh) & 0xFFu);
        w.scB = (float)((S >> (sh + 8)) & 0xFFu);
        w.mA = (float)((M >> sh) & 0xFFu);
        w.mB = (float)((M >> (sh + 8)) & 0xFFu);
        return w;
    }
    static __device__ __forceinline__ act load_a(const int8_t *__restrict__ q, const act_ds *__restrict__ ds, int c) {
        act A;
        const int8_t *p = q + c * 64;      // activation blocks 2c (sub-block 2g) and 2c+1 (sub-block 2g+1)
        A.a0lo = load16(p);
        A.a0hi = load16(p + 16);
        A.a1lo = load16(p + 32);
        A.a1hi = load16(p + 48);
        const u32x4 s = load16(ds + 2 * c);   // {d, sum} of both blocks
        const u32 d0b = s[0], sum0 = s[1], d1b = s[2], sum1 = s[3];   // copy the lanes out before bit-casting
        A.d0 = __builtin_bit_cast(float, d0b);
        A.d1 = __builtin_bit_cast(float, d1b);
        A.ds0 = A.d0 * (float)(int)sum0;
        A.ds1 = A.d1 * (float)(int)sum1;
        return A;
    }
    // i0 / i1 = sum nibble*q over sub-blocks 2g / 2g+1 (ggml-cpu-quants.c:6817-6848)
    static __device__ __forceinline__ chunk_dots dots(const chunk &w, const act &A) {
        int sA = 0, sB = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            sA = dot4((int)(w.q0[i] & 0x0F0F0F0Fu), (int)A.a0lo[i], sA);
            sA = dot4((int)(w.q1[i] & 0x0F0F0F0Fu), (int)A.a0hi[i], sA);
            sB = dot4((int)((w.q0[i] >> 4) & 0x0F0F0F0Fu), (int)A.a1lo[i], sB);
            sB = dot4((int)((w.q1[i] >> 4) & 0x0F0F0F0Fu), (int)A.a1hi[i], sB);
        }
        chunk_dots r = {sA, sB};
        return r;
    }
    static __device__ __forceinline__ float accumulate(float acc, const chunk &w, const act &A, const chunk_dots &r) {
        const float pos = __builtin_fmaf(w.scA, mul_rn(A.d0, (float)r.i0), mul_rn(w.scB, mul_rn(A.d1, (float)r.i1)));
        const float neg = __builtin_fmaf(w.mA, A.ds0, mul_rn(w.mB, A.ds1));
        return add_rn(acc, __builtin_fmaf(w.d, pos, -mul_rn(w.dmin, neg)));
    }
};

// ---------------------------------------------------------------- Q6_K
// Q5_K (block_q5_K, ggml/src/ggml-common.h:296-308: d, dmin, 12 scale bytes, qh[32], qs[128]): the Q4_K arithmetic on levels
// 0..31 - low nibble from qs, bit 4 of sub-block j from bit j of qh[l] (dequantize_row_q5_K, ggml/src/ggml-quants.c:1482-1507;
// ggml_vec_dot_q5_K_q8_K, ggml/src/ggml-cpu/ggml-cpu-quants.c:7539-7592)
template <> struct wq<MI355_Q5_K> {
    static constexpr int CHUNK = 64;
    struct chunk { u32x4 q0, q1, h0, h1; float d, dmin, scA, mA, scB, mB; int g; };
    typedef wq<MI355_Q4_K>::act act;
    static __device__ __forceinline__ chunk load_w(const uint8_t *__restrict__ row, const row_layout &, int c) {
        chunk w;
        const int sb = c >> 2, g = c & 3;
        const uint8_t *blk = row + sb * Q5_K_BYTES;
        const u32x4 hdr = load16(blk);   // d, dmin, 12 scale bytes: same address for the 4 lanes of a super-block
        w.h0 = load16(blk + 16);         // qh: also shared by the 4 lanes
        w.h1 = load16(blk + 32);
        w.q0 = load16(blk + 48 + g * 32);
        w.q1 = load16(blk + 64 + g * 32);
        w.g = g;
        w.d = half_bits_to_float((unsigned short)(hdr[0] & 0xFFFFu));
        w.dmin = half_bits_to_float((unsigned short)(hdr[0] >> 16));
        const u32 s_lo = hdr[1] & 0x3F3F3F3Fu, m_lo = hdr[2] & 0x3F3F3F3Fu;
        const u32 s_hi = (hdr[3] & 0x0F0F0F0Fu) | (((hdr[1] >> 6) & 0x03030303u) << 4);
        const u32 m_hi = ((hdr[3] >> 4) & 0x0F0F0F0Fu) | (((hdr[2] >> 6) & 0x03030303u) << 4);
        const u32 S = g < 2 ? s_lo : s_hi, M = g < 2 ? m_lo : m_hi;
        const int sh = 16 * (g & 1);
        w.scA = (float)((S >> sh) & 0xFFu);
        w.scB = (float)((S >> (sh + 8)) & 0xFFu);
        w.mA = (float)((M >> sh) & 0xFFu);
        w.mB = (float)((M >> (sh + 8)) & 0xFFu);
        return w;
    }
    static __device__ __forceinline__ act load_a(const int8_t *__restrict__ q, const act_ds *__restrict__ ds, int c) { return wq<MI355_Q4_K>::load_a(q, ds, c); }
    // i0 / i1 = sum level*q over sub-blocks 2g / 2g+1
    static __device__ __forceinline__ chunk_dots dots(const chunk &w, const act &A) {
        int sA = 0, sB = 0;
        const int ba = 2 * w.g, bb = 2 * w.g + 1;   // bits of qh that belong to the two sub-blocks
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const u32 la0 = (w.q0[i] & 0x0F0F0F0Fu) | (((w.h0[i] >> ba) & 0x01010101u) << 4);
            const u32 la1 = (w.q1[i] & 0x0F0F0F0Fu) | (((w.h1[i] >> ba) & 0x01010101u) << 4);
            const u32 lb0 = ((w.q0[i] >> 4) & 0x0F0F0F0Fu) | (((w.h0[i] >> bb) & 0x01010101u) << 4);
            const u32 lb1 = ((w.q1[i] >> 4) & 0x0F0F0F0Fu) | (((w.h1[i] >> bb) & 0x01010101u) << 4);
            sA = dot4((int)la0, (int)A.a0lo[i], sA);
            sA = dot4((int)la1, (int)A.a0hi[i], sA);
            sB = dot4((int)lb0, (int)A.a1lo[i], sB);
            sB = dot4((int)lb1, (int)A.a1hi[i], sB);
        }
        chunk_dots r = {sA, sB};
        return r;
    }
    static __device__ __forceinline__ float accumulate(float acc, const chunk &w, const act &A, const chunk_dots &r) {
        const float pos = __builtin_fmaf(w.scA, mul_rn(A.d0, (float)r.i0), mul_rn(w.scB, mul_rn(A.d1, (float)r.i1)));
        const float neg = __builtin_fmaf(w.mA, A.ds0, mul_rn(w.mB, A.ds1));
        return add_rn(acc, __builtin_fmaf(w.d, pos, -mul_rn(w.dmin, neg)));
    }
};

template <> struct wq<MI355_Q6_K> {
    static constexpr int CHUNK = 32;
    struct chunk { u32x4 ql, qh; float d, scA, scB; int shA, shB; };
    struct act { u32x4 a0, a1; float d0, d1; int s0, s1; };
    static __device__ __forceinline__ chunk load_w(const uint8_t *__restrict__ row, const row_layout &L, int c) {
        chunk w;
        const int sb = c >> 3, cc = c & 7, hf = cc >> 2, r = cc & 3;
        const int l0 = 16 * (r & 1), qa = r >> 1;
        w.ql = load_stream16(row + sb * 128 + cc * 16);
        w.qh = load_stream16(row + L.off_b + sb * 64 + hf * 32 + l0);
        const int8_t *sc = (const int8_t *)(row + L.off_c + sb * 16 + hf * 8 + (l0 >> 4));
        w.scA = (float)sc[2 * qa];
        w.scB = (float)sc[2 * qa + 4];
        w.d = half_bits_to_float(*(const unsigned short *)(row + L.off_d + sb * 2));
        w.shA = 2 * qa;
        w.shB = 2 * qa + 4;
        return w;
    }
    static __device__ __forceinline__ act load_a(const int8_t *__restrict__ q, const act_ds *__restrict__ ds, int c) {
        act A;
        const int sb = c >> 3, cc = c & 7, hf = cc >> 2, r = cc & 3;
        const int l0 = 16 * (r & 1), qa = r >> 1;
        const int bA = sb * 8 + 4 * hf + qa;   // quarter qa of this half; quarter qa+2 is two blocks on
        A.a0 = load16(q + bA * 32 + l0);
        A.a1 = load16(q + (bA + 2) * 32 + l0);
        A.d0 = ds[bA].d;
        A.d1 = ds[bA + 2].d;
        int s0 = 0, s1 = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            s0 = dot4(0x01010101, (int)A.a0[i], s0);
            s1 = dot4(0x01010101, (int)A.a1[i], s1);
        }
        A.s0 = s0;
        A.s1 = s1;
        return A;
    }
    // i0 / i1 = sum (q6-32)*q over the two 16-element scale groups of this chunk (ggml-cpu-quants.c:8262-8283)
    static __device__ __forceinline__ chunk_dots dots(const chunk &w, const act &A) {
        int sA = 0, sB = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const u32 vA = (w.ql[i] & 0x0F0F0F0Fu) | (((w.qh[i] >> w.shA) & 0x03030303u) << 4);
            const u32 vB = ((w.ql[i] >> 4) & 0x0F0F0F0Fu) | (((w.qh[i] >> w.shB) & 0x03030303u) << 4);
            sA = dot4((int)vA, (int)A.a0[i], sA);
            sB = dot4((int)vB, (int)A.a1[i], sB);
        }
        chunk_dots r = {sA - 32 * A.s0, sB - 32 * A.s1};
        return r;
    }
    static __device__ __forceinline__ float accumulate(float acc, const chunk &w, const act &A, const chunk_dots &r) {
        const float t = __builtin_fmaf(w.scA, mul_rn(A.d0, (float)r.i0), mul_rn(w.scB, mul_rn(A.d1, (float)r.i1)));
        return __builtin_fmaf(w.d, t, acc);
    }
};

// ---------------------------------------------------------------- scalar element access
// Dequantized weight element e of a row stored in device layout.  Byte loads only, so it
// works for rows that are not 16-byte aligned (K not a multiple of 256 for Q4_0/Q8_0, of
// 2048 for Q6_K).  Semantics: dequantize_row_* of ggml/src/ggml-quants.c:255-347, 349-363,
// 1280-1302, 1482-1507, 1690-1719, 2436-2475.
template <int TYPE>
__device__ __forceinline__ float weight_value(const uint8_t *__restrict__ row, const row_layout &L, int64_t e) {
    if constexpr (TYPE == MI355_Q4_0) {
        const int64_t b = e >> 5;
        const int j = (int)(e & 31);
        const uint8_t byte = row[b * 16 + (j & 15)];
        const int n = j < 16 ? (byte & 0x0F) : (byte >> 4);
        const unsigned short dh = (unsigned short)(row[L.off_b + 2 * b] | (row[L.off_b + 2 * b + 1] << 8));
        return half_bits_to_float(dh) * (float)(n - 8);
    } else if constexpr (TYPE == MI355_IQ4_NL) {
        constexpr int8_t values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
        const int64_t b = e >> 5;
        const int j = (int)(e & 31);
        const uint8_t byte = row[b * 16 + (j & 15)];
        const unsigned short dh = (unsigned short)(row[L.off_b + 2 * b] | (row[L.off_b + 2 * b + 1] << 8));
        return half_bits_to_float(dh) * (float)values[j < 16 ? (byte & 0x0F) : (byte >> 4)];
    } else if constexpr (TYPE == MI355_IQ4_XS) {
        constexpr int8_t values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
        const int64_t b = e >> 5;
        const int j = (int)(e & 31), ib = (int)(b & 7);
        const uint8_t byte = row[b * 16 + (j & 15)];
        const uint8_t *h = row + L.off_b + (b >> 3) * 8;
        const int ls = ((h[4 + ib / 2] >> (4 * (ib & 1))) & 0xF) | (((((int)h[2] | ((int)h[3] << 8)) >> (2 * ib)) & 3) << 4);
        const float dl = half_bits_to_float((unsigned short)(h[0] | (h[1] << 8))) * (float)(ls - 32);
        return dl * (float)values[j < 16 ? (byte & 0x0F) : (byte >> 4)];
    } else if constexpr (TYPE == MI355_Q4_1 || TYPE == MI355_Q5_0 || TYPE == MI355_Q5_1) {
        const int64_t b = e >> 5;
        const int j = (int)(e & 31);
        const uint8_t byte = row[b * 16 + (j & 15)];
        int n = j < 16 ? (byte & 0x0F) : (byte >> 4);
        if constexpr (TYPE != MI355_Q4_1) n |= ((row[L.off_b + 4 * b + (j >> 3)] >> (j & 7)) & 1) << 4;
        const int64_t so = TYPE == MI355_Q4_1 ? L.off_b + 4 * b : TYPE == MI355_Q5_0 ? L.off_c + 2 * b : L.off_c + 4 * b;
        const float d = half_bits_to_float((unsigned short)(row[so] | (row[so + 1] << 8)));
        if constexpr (TYPE == MI355_Q5_0) return d * (float)(n - 16);
        else return add_rn(mul_rn((float)n, d), half_bits_to_float((unsigned short)(row[so + 2] | (row[so + 3] << 8))));
    } else if constexpr (TYPE == MI355_Q8_0) {
        const int64_t b = e >> 5;
        const int8_t q = (int8_t)row[b * 32 + (e & 31)];
        const unsigned short dh = (unsigned short)(row[L.off_b + 2 * b] | (row[L.off_b + 2 * b + 1] << 8));
        return half_bits_to_float(dh) * (float)q;
    } else if constexpr (TYPE == MI355_Q4_K) {
        const int64_t sb = e >> 8;
        const int r = (int)(e & 255), j = r >> 5, l = r & 31;
        const uint8_t *blk = row + sb * Q4_K_BYTES;
        const unsigned short dh = (unsigned short)(blk[0] | (blk[1] << 8)), mh = (unsigned short)(blk[2] | (blk[3] << 8));
        const uint8_t *p = blk + 4;
        int sc, mn;
        if (j < 4) { sc = p[j] & 63; mn = p[j + 4] & 63; }
        else { sc = (p[j + 4] & 0x0F) | ((p[j - 4] >> 6) << 4); mn = (p[j + 4] >> 4) | ((p[j] >> 6) << 4); }
        const uint8_t byte = blk[16 + 32 * (j >> 1) + l];
        const int n = (j & 1) ? (byte >> 4) : (byte & 0x0F);
        return half_bits_to_float(dh) * (float)sc * (float)n - half_bits_to_float(mh) * (float)mn;
    } else if constexpr (TYPE == MI355_Q5_K) {
        const int64_t sb = e >> 8;
        const int r = (int)(e & 255), j = r >> 5, l = r & 31;
        const uint8_t *blk = row + sb * Q5_K_BYTES;
        const unsigned short dh = (unsigned short)(blk[0] | (blk[1] << 8)), mh = (unsigned short)(blk[2] | (blk[3] << 8));
        const uint8_t *p = blk + 4;
        int sc, mn;
        if (j < 4) { sc = p[j] & 63; mn = p[j + 4] & 63; }
        else { sc = (p[j + 4] & 0x0F) | ((p[j - 4] >> 6) << 4); mn = (p[j + 4] >> 4) | ((p[j] >> 6) << 4); }
        const uint8_t byte = blk[48 + 32 * (j >> 1) + l];
        const int n = ((j & 1) ? (byte >> 4) : (byte & 0x0F)) + (((blk[16 + l] >> j) & 1) << 4);
        return half_bits_to_float(dh) * (float)sc * (float)n - half_bits_to_float(mh) * (float)mn;
    } else {
        const int64_t sb = e >> 8;
        const int r = (int)(e & 255), hf = r >> 7, quad = (r & 127) >> 5, l = r & 31;
        const uint8_t lo = row[sb * 128 + 64 * hf + 32 * (quad & 1) + l];
        const int nib = quad < 2 ? (lo & 0x0F) : (lo >> 4);
        const int hi = (row[L.off_b + sb * 64 + 32 * hf + l] >> (2 * quad)) & 3;
        const int8_t sc = (int8_t)row[L.off_c + sb * 16 + (r >> 4)];
        const unsigned short dh = (unsigned short)(row[L.off_d + 2 * sb] | (row[L.off_d + 2 * sb + 1] << 8));
        return half_bits_to_float(dh) * (float)sc * (float)((nib | (hi << 4)) - 32);
    }
}

}  // namespace mi355
