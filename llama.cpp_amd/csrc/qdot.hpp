// Per-lane integer dot products of quantized weight chunks against Q8_1 activations.
//
// Work unit ("chunk"): 32 weight elements.  Chunk c of a row is taken by lane c % 64 at
// step c / 64, so one wave consumes 2048 consecutive elements per step and every lane
// issues 16-byte, 16-byte-aligned loads to consecutive addresses.
//   Q4_0 / Q8_0 : chunk = one block.
//   Q4_K        : chunk = 16 bytes of qs = the 16h..16h+15 elements of sub-blocks 2g
//                 (low nibbles) and 2g+1 (high nibbles); 8 chunks per super-block.
//   Q6_K        : chunk = 16 bytes of ql + the matching 16 bytes of qh = two 16-element
//                 scale groups; 8 chunks per super-block.
// The same functions feed the GEMV kernels and the parity entry point that dumps the
// integer dots, so what is checked bit-for-bit is what ships.
#pragma once

#include "common.hpp"

namespace mi355 {

// Device layout of one weight row (see mi355_kernels.h): byte offsets of the per-row regions.
struct row_layout {
    int64_t row_bytes;
    int64_t off_b;   // Q4_0/Q8_0: fp16 d array.  Q6_K: qh array
    int64_t off_c;   // Q6_K: scales array
    int64_t off_d;   // Q6_K: fp16 d array
};

__host__ __device__ inline row_layout make_row_layout(int type, int64_t k) {
    row_layout L = {0, 0, 0, 0};
    const int64_t nb = k / type_block_elems(type);
    L.row_bytes = nb * type_block_bytes(type);
    switch (type) {
        case MI355_Q4_0: L.off_b = nb * 16; break;
        case MI355_Q8_0: L.off_b = nb * 32; break;
        case MI355_Q6_K: L.off_b = nb * 128; L.off_c = nb * 192; L.off_d = nb * 208; break;
        default: break;
    }
    return L;
}

// Activation operands of one chunk for one activation row (column of the product).
struct act_chunk {
    u32x4 a0, a1;   // 2 x 16 int8 levels
    float d0, d1;   // block scales of the blocks a0 / a1 come from
    int s0, s1;     // integer level sums that pair with a0 / a1 (meaning depends on type)
};

// Integer results of one weight chunk against one act_chunk.
struct chunk_dots {
    int i0, i1;
};

template <int TYPE>
__device__ __forceinline__ act_chunk load_act_chunk(const int8_t *__restrict__ q, const act_ds *__restrict__ ds,
                                                    int64_t c) {
    act_chunk A;
    if constexpr (TYPE == MI355_Q4_0 || TYPE == MI355_Q8_0) {
        A.a0 = load16(q + c * 32);
        A.a1 = load16(q + c * 32 + 16);
        const act_ds s = ds[c];
        A.d0 = A.d1 = s.d;
        A.s0 = A.s1 = s.sum;
    } else if constexpr (TYPE == MI355_Q4_K) {
        const int64_t sb = c >> 3;
        const int cc = (int)(c & 7), g = cc >> 1, h = cc & 1;
        const int64_t bA = sb * 8 + 2 * g;
        A.a0 = load16(q + bA * 32 + 16 * h);
        A.a1 = load16(q + (bA + 1) * 32 + 16 * h);
        const act_ds sA = ds[bA], sB = ds[bA + 1];
        A.d0 = sA.d;
        A.d1 = sB.d;
        // the "- dmin * m * sum(q)" term of a sub-block is applied once, by the lane holding its first half
        A.s0 = h == 0 ? sA.sum : 0;
        A.s1 = h == 0 ? sB.sum : 0;
    } else {   // Q6_K
        const int64_t sb = c >> 3;
        const int cc = (int)(c & 7), hf = cc >> 2, r = cc & 3;
        const int l0 = 16 * (r & 1), qa = r >> 1;
        const int64_t bA = sb * 8 + 4 * hf + qa;   // quarter qa of this half; quarter qa+2 is two blocks on
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
    }
    return A;
}

// ---------------------------------------------------------------- Q4_0
struct wchunk_q4_0 {
    u32x4 qs;
    float d;
};
__device__ __forceinline__ wchunk_q4_0 load_w_q4_0(const uint8_t *__restrict__ row, const row_layout &L, int64_t c) {
    wchunk_q4_0 w;
    w.qs = load_stream16(row + c * 16);
    w.d = half_bits_to_float(*(const unsigned short *)(row + L.off_b + c * 2));
    return w;
}
// i0 = sum (nibble-8)*q over the block (ggml-cpu-quants.c:2496-2505); i1 unused
__device__ __forceinline__ chunk_dots dots_q4_0(const wchunk_q4_0 &w, const act_chunk &A) {
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        s = dot4((int)(w.qs[i] & 0x0F0F0F0Fu), (int)A.a0[i], s);
        s = dot4((int)((w.qs[i] >> 4) & 0x0F0F0F0Fu), (int)A.a1[i], s);
    }
    chunk_dots r = {s - 8 * A.s0, 0};
    return r;
}
__device__ __forceinline__ float combine_q4_0(const wchunk_q4_0 &w, const act_chunk &A, const chunk_dots &r) {
    return w.d * (A.d0 * (float)r.i0);
}

// ---------------------------------------------------------------- Q8_0
struct wchunk_q8_0 {
    u32x4 q0, q1;
    float d;
};
__device__ __forceinline__ wchunk_q8_0 load_w_q8_0(const uint8_t *__restrict__ row, const row_layout &L, int64_t c) {
    wchunk_q8_0 w;
    w.q0 = load_stream16(row + c * 32);
    w.q1 = load_stream16(row + c * 32 + 16);
    w.d = half_bits_to_float(*(const unsigned short *)(row + L.off_b + c * 2));
    return w;
}
__device__ __forceinline__ chunk_dots dots_q8_0(const wchunk_q8_0 &w, const act_chunk &A) {
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        s = dot4((int)w.q0[i], (int)A.a0[i], s);
        s = dot4((int)w.q1[i], (int)A.a1[i], s);
    }
    chunk_dots r = {s, 0};
    return r;
}
__device__ __forceinline__ float combine_q8_0(const wchunk_q8_0 &w, const act_chunk &A, const chunk_dots &r) {
    return w.d * (A.d0 * (float)r.i0);
}

// ---------------------------------------------------------------- Q4_K
struct wchunk_q4_K {
    u32x4 qs;
    float d, dmin;
    float scA, mA, scB, mB;   // 6-bit scale/min of sub-blocks 2g and 2g+1
};
// 6-bit (scale, min) of sub-block j from the 12 packed bytes held in three dwords
// (get_scale_min_k4, ggml/src/ggml-quants.c:631-638)
__device__ __forceinline__ void q4k_scale_min(u32 u0, u32 u1, u32 u2, int j, int &sc, int &mn) {
    // bytes: u0 = b[0..3], u1 = b[4..7], u2 = b[8..11]
    const int jj = j & 3, sh = 8 * jj;
    const u32 b_lo = (u0 >> sh) & 0xFFu;    // b[jj]
    const u32 b_mid = (u1 >> sh) & 0xFFu;   // b[jj+4]
    const u32 b_hi = (u2 >> sh) & 0xFFu;    // b[jj+8]
    if (j < 4) {
        sc = (int)(b_lo & 63u);
        mn = (int)(b_mid & 63u);
    } else {
        sc = (int)((b_hi & 0x0Fu) | ((b_lo >> 6) << 4));
        mn = (int)((b_hi >> 4) | ((b_mid >> 6) << 4));
    }
}
__device__ __forceinline__ wchunk_q4_K load_w_q4_K(const uint8_t *__restrict__ row, const row_layout &, int64_t c) {
    wchunk_q4_K w;
    const int64_t sb = c >> 3;
    const int cc = (int)(c & 7);
    const uint8_t *blk = row + sb * Q4_K_BYTES;
    const u32x4 hdr = load_stream16(blk);   // d, dmin, 12 scale bytes; same address for the 8 lanes of a super-block
    w.qs = load_stream16(blk + 16 + cc * 16);
    w.d = half_bits_to_float((unsigned short)(hdr[0] & 0xFFFFu));
    w.dmin = half_bits_to_float((unsigned short)(hdr[0] >> 16));
    int sc, mn;
    q4k_scale_min(hdr[1], hdr[2], hdr[3], (cc >> 1) * 2, sc, mn);
    w.scA = (float)sc;
    w.mA = (float)mn;
    q4k_scale_min(hdr[1], hdr[2], hdr[3], (cc >> 1) * 2 + 1, sc, mn);
    w.scB = (float)sc;
    w.mB = (float)mn;
    return w;
}
// i0 / i1 = sum nibble*q over this lane's half of sub-block 2g / 2g+1 (ggml-cpu-quants.c:6817-6848)
__device__ __forceinline__ chunk_dots dots_q4_K(const wchunk_q4_K &w, const act_chunk &A) {
    int sA = 0, sB = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        sA = dot4((int)(w.qs[i] & 0x0F0F0F0Fu), (int)A.a0[i], sA);
        sB = dot4((int)((w.qs[i] >> 4) & 0x0F0F0F0Fu), (int)A.a1[i], sB);
    }
    chunk_dots r = {sA, sB};
    return r;
}
__device__ __forceinline__ float combine_q4_K(const wchunk_q4_K &w, const act_chunk &A, const chunk_dots &r) {
    const float pos = w.scA * (A.d0 * (float)r.i0) + w.scB * (A.d1 * (float)r.i1);
    const float neg = w.mA * (A.d0 * (float)A.s0) + w.mB * (A.d1 * (float)A.s1);
    return w.d * pos - w.dmin * neg;
}

// ---------------------------------------------------------------- Q6_K
struct wchunk_q6_K {
    u32x4 ql, qh;
    float d;
    float scA, scB;
    int shA, shB;   // bit offsets of this chunk's two quarters inside qh
};
__device__ __forceinline__ wchunk_q6_K load_w_q6_K(const uint8_t *__restrict__ row, const row_layout &L, int64_t c) {
    wchunk_q6_K w;
    const int64_t sb = c >> 3;
    const int cc = (int)(c & 7), hf = cc >> 2, r = cc & 3;
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
// i0 / i1 = sum (q6-32)*q over the two 16-element scale groups of this chunk (ggml-cpu-quants.c:8262-8283)
__device__ __forceinline__ chunk_dots dots_q6_K(const wchunk_q6_K &w, const act_chunk &A) {
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
__device__ __forceinline__ float combine_q6_K(const wchunk_q6_K &w, const act_chunk &A, const chunk_dots &r) {
    return w.d * (w.scA * (A.d0 * (float)r.i0) + w.scB * (A.d1 * (float)r.i1));
}

// Dequantized weight element e of a row stored in device layout.  Byte loads only, so it
// works for rows that are not 16-byte aligned (K not a multiple of 256 for Q4_0/Q8_0, of
// 2048 for Q6_K).  Semantics: dequantize_row_* of ggml/src/ggml-quants.c:255-273, 349-363,
// 1280-1302, 1690-1719.
template <int TYPE>
__device__ __forceinline__ float weight_value(const uint8_t *__restrict__ row, const row_layout &L, int64_t e) {
    if constexpr (TYPE == MI355_Q4_0) {
        const int64_t b = e >> 5;
        const int j = (int)(e & 31);
        const uint8_t byte = row[b * 16 + (j & 15)];
        const int n = j < 16 ? (byte & 0x0F) : (byte >> 4);
        const unsigned short dh = (unsigned short)(row[L.off_b + 2 * b] | (row[L.off_b + 2 * b + 1] << 8));
        return half_bits_to_float(dh) * (float)(n - 8);
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

// ---------------------------------------------------------------- type dispatch
template <int TYPE> struct wq;
template <> struct wq<MI355_Q4_0> {
    typedef wchunk_q4_0 chunk;
    static __device__ __forceinline__ chunk load(const uint8_t *row, const row_layout &L, int64_t c) { return load_w_q4_0(row, L, c); }
    static __device__ __forceinline__ chunk_dots dots(const chunk &w, const act_chunk &A) { return dots_q4_0(w, A); }
    static __device__ __forceinline__ float combine(const chunk &w, const act_chunk &A, const chunk_dots &r) { return combine_q4_0(w, A, r); }
};
template <> struct wq<MI355_Q8_0> {
    typedef wchunk_q8_0 chunk;
    static __device__ __forceinline__ chunk load(const uint8_t *row, const row_layout &L, int64_t c) { return load_w_q8_0(row, L, c); }
    static __device__ __forceinline__ chunk_dots dots(const chunk &w, const act_chunk &A) { return dots_q8_0(w, A); }
    static __device__ __forceinline__ float combine(const chunk &w, const act_chunk &A, const chunk_dots &r) { return combine_q8_0(w, A, r); }
};
template <> struct wq<MI355_Q4_K> {
    typedef wchunk_q4_K chunk;
    static __device__ __forceinline__ chunk load(const uint8_t *row, const row_layout &L, int64_t c) { return load_w_q4_K(row, L, c); }
    static __device__ __forceinline__ chunk_dots dots(const chunk &w, const act_chunk &A) { return dots_q4_K(w, A); }
    static __device__ __forceinline__ float combine(const chunk &w, const act_chunk &A, const chunk_dots &r) { return combine_q4_K(w, A, r); }
};
template <> struct wq<MI355_Q6_K> {
    typedef wchunk_q6_K chunk;
    static __device__ __forceinline__ chunk load(const uint8_t *row, const row_layout &L, int64_t c) { return load_w_q6_K(row, L, c); }
    static __device__ __forceinline__ chunk_dots dots(const chunk &w, const act_chunk &A) { return dots_q6_K(w, A); }
    static __device__ __forceinline__ float combine(const chunk &w, const act_chunk &A, const chunk_dots &r) { return combine_q6_K(w, A, r); }
};

}  // namespace mi355
