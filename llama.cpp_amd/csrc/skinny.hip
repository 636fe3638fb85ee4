// MUL_MAT for a handful of activation rows (4 .. 32): weight-streaming kernel on the int8 matrix cores.
//
// The batch-1 kernels (gemv.hip) spend eight v_dot4 per weight block and activation row, which binds them to the vector
// ALUs from about five activation rows on; the tile kernels (mmq.hip, mmq_k.hip) are built around 64..128-row activation
// tiles and a K loop with group barriers, and a launch with one tile column is latency-bound.  Here a wave owns 32 weight
// rows and one quarter of K and never waits for another wave until the end:
//   * per step of 256 elements the wave copies its weights (32 rows), activation rows and activation scales to its own
//     part of LDS with fully coalesced 16-byte loads (a lane reads along a row; the loads of the next step are requested
//     as soon as the registers are free, before the current step is contracted), and reads them back in matrix-core
//     operand order.  Nobody else touches that part of LDS, and a wave's LDS accesses complete in program order, so no
//     barrier is involved;
//   * one v_mfma_i32_32x32x32_i8 per weight block: operand A = 16 levels of an activation row per lane (lane % 32 = row,
//     lane / 32 = half of the block), operand B = 16 levels of a weight row per lane;
//   * the result puts ONE weight row (lane % 32) and activation rows 4 (lane / 32) + 8 q + 0..3 (q = 0..3) in a lane:
//     the weight scale is one value per lane and block, the activation scales are 4 consecutive table entries per q,
//     and only the q that hold real activation rows are finished (NI = ceil(rows / 8) of them);
//   * the four K quarters of a group meet in LDS at the end and are added in a fixed order.
// Integer sums are exact, so the result differs from the batch-1 kernels' only in the order of the f32 additions.
// Activations are the Q8_1 workspace of mi355_quantize_act (ggml-cpu quantizes to Q8_0/Q8_1 for Q4_0/Q8_0 weights and to
// Q8_K for Q4_K, ggml-cpu.c:7420-7450; the NMSE bound of the product is what is checked for Q4_K).
#include "qdot.hpp"

namespace mi355 {

namespace {

// What goes through LDS per step (256 elements) and weight row: the 4-bit (Q8_0: 8-bit) plane of the levels - 128 bytes of
// nibbles for every type but Q8_0; Q6_K copies its 64 bytes of high bit pairs beside them.  Everything a lane needs of ITS row
// only (block scales and minima, the K-quants' 16-byte header, the fifth bits of Q5_0 / Q5_1 / Q5_K) goes straight to registers.
template <int TYPE> struct sk_traits {
    static constexpr int ROW_BYTES = TYPE == MI355_Q8_0 ? 256 : 128;
    // per-32-block types whose block is 16 bytes of nibbles, element b low and element 16 + b high in byte b
    static constexpr bool NIB32 = TYPE == MI355_Q4_0 || TYPE == MI355_IQ4_NL || TYPE == MI355_IQ4_XS || TYPE == MI355_Q4_1 || TYPE == MI355_Q5_0 ||
                                  TYPE == MI355_Q5_1;
    static constexpr bool TABLE = TYPE == MI355_IQ4_NL || TYPE == MI355_IQ4_XS;     // a nibble stands for an entry of the sixteen-value table
    static constexpr bool PAIR = TYPE == MI355_Q4_1 || TYPE == MI355_Q5_1;          // {f16 d, f16 m} per block
    static constexpr bool FIFTH32 = TYPE == MI355_Q5_0 || TYPE == MI355_Q5_1;       // one word of fifth bits per block
    static constexpr bool KQ = TYPE == MI355_Q4_K || TYPE == MI355_Q5_K;            // 16-byte header + 6-bit (scale, min) pairs
    static constexpr int STEP_BYTES = TYPE == MI355_Q8_0 ? 256 : TYPE == MI355_Q4_K ? Q4_K_BYTES : TYPE == MI355_Q5_K ? Q5_K_BYTES : 128;
    static constexpr int QS_OFF = TYPE == MI355_Q4_K ? 16 : TYPE == MI355_Q5_K ? 48 : 0;   // where the nibbles start inside a step
    // the activation's block sum enters as x = OFFSET * d * sum (levels stored with an offset) or as d * sum (block minimum)
    static constexpr float OFFSET = TYPE == MI355_Q4_0 ? -8.0f : TYPE == MI355_Q5_0 ? -16.0f : 1.0f;
};

// Orders a wave's own LDS accesses around the point where its lanes exchange data through LDS: the hardware completes
// them in program order, so all that is needed is that neither the compiler nor the instruction scheduler moves an access
// across this point (they may otherwise: the copies and the operand reads go through differently typed pointers).
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

constexpr int SK_APAD = 256 + 16;      // LDS row strides (+16: rows 32 apart in banks do not all collide)

__device__ __forceinline__ float f16_of(const u32x4 &v, int j) {   // j is a compile-time constant after unrolling
    const u32 u = v[j >> 1];
    return half_bits_to_float((unsigned short)((j & 1) ? (u >> 16) : (u & 0xFFFFu)));
}

// registers of one step in flight
template <int TYPE, int NI> struct sk_regs {
    static constexpr int NW = 32 * sk_traits<TYPE>::ROW_BYTES / 1024;   // 16-byte loads per lane for the weights
    static constexpr int NA = 2 * NI;                                   // ... for 8 NI activation rows of 256 bytes
    static constexpr int NT = (NI + 1) / 2;                             // ... for their 8 {d, sum} pairs each
    u32x4 w[NW], a[NA], t[NT], hdr;
    u32x4 hdr2;                             // Q4_1 / Q5_1: the second half of the eight {d, m} pairs
    u32x4 qh[2];                            // Q6_K: the high bit pairs, 32 rows x 64 bytes (on their way to LDS); Q5_0 / Q5_1: the
                                            // eight fifth-bit words of the lane's row; Q5_K ([0] only): qh bytes 16 (lane / 32) .. + 16
    u32 d6;                                 // Q6_K: the f16 super-block scale of the lane's row (hdr holds its 16 int8 scales)
};

// grid.x = 32-row tiles of the weight matrix, grid.y = slices of K (partial sums to `dst` as [slice][B][dst_stride] then).
// The group's four waves split the slice's steps.
template <int TYPE, int NI>
__global__ void __launch_bounds__(256) k_mm_skinny(const uint8_t *__restrict__ W, const int8_t *__restrict__ aq, const act_ds *__restrict__ ads,
                                                   float *__restrict__ dst, const float *__restrict__ residual, int64_t N, int K, int B,
                                                   int64_t dst_stride, int steps_per_slice, int steps_per_wave) {
    typedef sk_traits<TYPE> T;
    typedef sk_regs<TYPE, NI> R;
    constexpr int WPAD = T::ROW_BYTES + 16;
    constexpr int QHPAD = 64 + 16;
    constexpr bool Q6 = TYPE == MI355_Q6_K;
    constexpr int W_BYTES = 32 * WPAD + (Q6 ? 32 * QHPAD : 0), A_BYTES = 8 * NI * SK_APAD, T_BYTES = 8 * 8 * NI * 8;
    constexpr int G_BYTES = Q6 ? 16 * 8 * NI * 4 : 0;   // Q6_K: integer sums of the activation levels per 16 elements
    constexpr int WAVE_BYTES = W_BYTES + A_BYTES + T_BYTES + G_BYTES;
    constexpr int RED_BYTES = 4 * NI * 4 * 64 * 4;
    __shared__ __attribute__((aligned(16))) uint8_t s_mem[4 * WAVE_BYTES > RED_BYTES ? 4 * WAVE_BYTES : RED_BYTES];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 31, kh = lane >> 5;
    uint8_t *s_w = s_mem + wave * WAVE_BYTES;
    uint8_t *s_a = s_w + W_BYTES;
    float2 *s_t = (float2 *)(s_a + A_BYTES);
    int *s_g = (int *)(s_a + A_BYTES + T_BYTES);
    uint8_t *s_qh = s_w + 32 * WPAD;

    const row_layout L = make_row_layout(TYPE, K);
    const int nsteps = K >> 8;
    const int nblk = K >> 5;
    const int64_t row0 = (int64_t)blockIdx.x * 32;

    const int slice_lo = blockIdx.y * steps_per_slice;
    const int slice_hi = slice_lo + steps_per_slice < nsteps ? slice_lo + steps_per_slice : nsteps;
    const int s_lo = slice_lo + wave * steps_per_wave;
    const int s_hi = s_lo + steps_per_wave < slice_hi ? s_lo + steps_per_wave : slice_hi;   // may be <= s_lo: a wave without steps

    // copy assignments: weights: a lane reads 16 bytes along a row, LPR lanes per row; activation rows: 16 lanes per row
    constexpr int LPR = T::ROW_BYTES / 16, RPL = 64 / LPR;   // lanes per row, rows per load
    const int w_piece = lane % LPR, w_row = lane / LPR;
    const uint8_t *w_src[R::NW];
#pragma unroll
    for (int u = 0; u < R::NW; u++) {
        int64_t row = row0 + w_row + u * RPL;
        row = row < N ? row : N - 1;   // clamp: rows past the end repeat the last row and are not stored
        w_src[u] = W + row * L.row_bytes + 16 * w_piece + T::QS_OFF;
    }
    const uint8_t *qh_src[2];   // Q6_K: 4 lanes per row, 16 rows per load
#pragma unroll
    for (int u = 0; u < 2; u++) {
        int64_t row = row0 + (lane >> 2) + 16 * u;
        row = row < N ? row : N - 1;
        qh_src[u] = W + row * L.row_bytes + L.off_b + 16 * (lane & 3);
    }
    const int64_t my_row = row0 + r < N ? row0 + r : N - 1;
    const uint8_t *w_mine = W + my_row * L.row_bytes;   // the row whose results this lane holds: its scales go to registers
    const int a_piece = lane & 15, a_row = lane >> 4;
    const int8_t *a_src[R::NA];
#pragma unroll
    for (int u = 0; u < R::NA; u++) {
        const int c = a_row + 4 * u < B ? a_row + 4 * u : B - 1;   // activation rows past the end repeat the last one
        a_src[u] = aq + (int64_t)c * K + 16 * a_piece;
    }
    const int t_piece = lane & 3, t_row = lane >> 2;   // {d, sum} pairs: 4 lanes x 16 bytes per activation row and step
    const act_ds *t_src[R::NT];
#pragma unroll
    for (int u = 0; u < R::NT; u++) {
        const int c = t_row + 16 * u < B ? t_row + 16 * u : B - 1;
        t_src[u] = ads + (int64_t)c * nblk + 2 * t_piece;
    }

    // loads of one step into the register set `g`
    auto fetch = [&](int step, R &g) {
        const int s = step < nsteps ? step : nsteps - 1;
        const int w_off = s * T::STEP_BYTES;   // < 2^31: rows are shorter than that
#pragma unroll
        for (int u = 0; u < R::NW; u++) g.w[u] = load16(w_src[u] + w_off);
        if constexpr (T::KQ) {
            g.hdr = load16(w_mine + w_off);
            if constexpr (TYPE == MI355_Q5_K) g.qh[0] = load16(w_mine + w_off + 16 + 16 * kh);
        } else if constexpr (T::FIFTH32) {
            g.qh[0] = load16(w_mine + L.off_b + s * 32);
            g.qh[1] = load16(w_mine + L.off_b + s * 32 + 16);
            if constexpr (T::PAIR) {
                g.hdr = load16(w_mine + L.off_c + s * 32);
                g.hdr2 = load16(w_mine + L.off_c + s * 32 + 16);
            } else {
                g.hdr = load16(w_mine + L.off_c + s * 16);
            }
        } else if constexpr (T::PAIR) {
            g.hdr = load16(w_mine + L.off_b + s * 32);
            g.hdr2 = load16(w_mine + L.off_b + s * 32 + 16);
        } else if constexpr (TYPE == MI355_IQ4_XS) {
            const uint2 h = *(const uint2 *)(w_mine + L.off_b + s * 8);   // the super-block's d, scales_h, scales_l
            g.hdr[0] = h.x;
            g.hdr[1] = h.y;
        } else if constexpr (Q6) {
#pragma unroll
            for (int u = 0; u < 2; u++) g.qh[u] = load16(qh_src[u] + s * 64);
            g.hdr = load16(w_mine + L.off_c + s * 16);                            // sixteen int8 scales
            g.d6 = *(const unsigned short *)(w_mine + L.off_d + s * 2);
        } else {
            g.hdr = load16(w_mine + L.off_b + s * 16);   // eight f16 block scales
        }
#pragma unroll
        for (int u = 0; u < R::NA; u++) g.a[u] = load16(a_src[u] + s * 256);
#pragma unroll
        for (int u = 0; u < R::NT; u++) g.t[u] = load16(t_src[u] + s * 8);
    };

    float acc[NI][4];
#pragma unroll
    for (int q = 0; q < NI; q++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[q][i] = 0.0f;

    // One set of load registers: as soon as a step's loads have been copied to LDS, the same registers take the next step's
    // loads, which are then in flight while this step is contracted.  Only the weight scales of the lane's row stay behind.
    R cur = {};
    fetch(s_lo, cur);
    for (int step = s_lo; step < s_hi; step++) {
        // ---- registers -> the wave's LDS
#pragma unroll
        for (int u = 0; u < R::NW; u++) *(u32x4 *)(s_w + (w_row + u * RPL) * WPAD + 16 * w_piece) = cur.w[u];
        if constexpr (Q6) {
#pragma unroll
            for (int u = 0; u < 2; u++) *(u32x4 *)(s_qh + ((lane >> 2) + 16 * u) * QHPAD + 16 * (lane & 3)) = cur.qh[u];
        }
#pragma unroll
        for (int u = 0; u < R::NA; u++) {
            *(u32x4 *)(s_a + (a_row + 4 * u) * SK_APAD + 16 * a_piece) = cur.a[u];
            if constexpr (Q6) {   // the lane's 16 bytes are one 16-element group of its activation row
                int sum = 0;
#pragma unroll
                for (int i = 0; i < 4; i++) sum = dot4(0x01010101, (int)cur.a[u][i], sum);
                s_g[a_piece * (8 * NI) + a_row + 4 * u] = sum;
            }
        }
#pragma unroll
        for (int u = 0; u < R::NT; u++) {
            if (t_row + 16 * u < 8 * NI) {
#pragma unroll
                for (int h = 0; h < 2; h++) {   // blocks 2 t_piece + h of activation row t_row + 16 u
                    const u32 d_bits = cur.t[u][2 * h], sum_bits = cur.t[u][2 * h + 1];   // copy the lanes out before bit-casting
                    const float d = __builtin_bit_cast(float, d_bits);
                    const float sum = (float)(int)sum_bits;
                    float2 v;
                    v.x = d;
                    v.y = T::OFFSET * d * sum;
                    s_t[(2 * t_piece + h) * (8 * NI) + t_row + 16 * u] = v;
                }
            }
        }
        const u32x4 hdr = cur.hdr, hdr2 = cur.hdr2;
        const u32x4 fifth[2] = {cur.qh[0], cur.qh[1]};   // (Q6_K's went to LDS above)
        const u32 d6 = cur.d6;
        wave_lds_sync();
        if (step + 1 < s_hi) fetch(step + 1, cur);

        const int am = r < 8 * NI ? r : r & 7;   // operand rows past the copied ones repeat copied ones; their results are not used
        if constexpr (Q6) {
            // 16 groups of 16 levels, each with its own int8 scale: one v_mfma_i32_32x32x16_i8 per group (8 levels per lane).
            // Group (hf, q, is): levels 128 hf + 32 q + 16 is .. + 16; level l of it = nibble q / 2 of ql byte 64 hf + 32 (q % 2) + 16 is + l
            // plus bits 2q, 2q + 1 of qh byte 32 hf + 16 is + l, minus 32 (dequantize_row_q6_K, ggml/src/ggml-quants.c:1690-1719).
            const float d = half_bits_to_float((unsigned short)d6);
#pragma unroll
            for (int hf = 0; hf < 2; hf++)
#pragma unroll
                for (int is = 0; is < 2; is++) {
                    const u32x2 qh8 = *(const u32x2 *)(s_qh + r * QHPAD + 32 * hf + 16 * is + 8 * kh);
#pragma unroll
                    for (int qlo = 0; qlo < 2; qlo++) {
                        const u32x2 ql8 = *(const u32x2 *)(s_w + r * WPAD + 64 * hf + 32 * qlo + 16 * is + 8 * kh);
#pragma unroll
                        for (int qhi = 0; qhi < 2; qhi++) {
                            const int q = qlo + 2 * qhi;
                            const int g = 8 * hf + 2 * q + is;   // scale index = position of the group in the super-block
                            u32x2 lv;
#pragma unroll
                            for (int i = 0; i < 2; i++) lv[i] = ((ql8[i] >> (4 * qhi)) & 0x0F0F0F0Fu) | (((qh8[i] >> (2 * q)) & 0x03030303u) << 4);
                            const u32x2 a8 = *(const u32x2 *)(s_a + am * SK_APAD + 128 * hf + 32 * q + 16 * is + 8 * kh);
                            i32x16 z;
#pragma unroll
                            for (int i = 0; i < 16; i++) z[i] = 0;
                            const i32x16 D = __builtin_amdgcn_mfma_i32_32x32x16_i8(__builtin_bit_cast(long, a8), __builtin_bit_cast(long, lv), z, 0, 0, 0);
                            const u32 sc_word = hdr[g >> 2];
                            const float wsg = d * (float)(int)(signed char)((sc_word >> (8 * (g & 3))) & 0xFFu);
#pragma unroll
                            for (int qq = 0; qq < NI; qq++) {
                                const float4 *e = (const float4 *)(s_t + (4 * hf + q) * (8 * NI) + 8 * qq + 4 * kh);
                                const float4 e01 = e[0], e23 = e[1];
                                const float dd[4] = {e01.x, e01.z, e23.x, e23.z};
                                const i32x4 gs = *(const i32x4 *)(s_g + g * (8 * NI) + 8 * qq + 4 * kh);
#pragma unroll
                                for (int i = 0; i < 4; i++) acc[qq][i] = __builtin_fmaf(wsg, dd[i] * (float)(D[4 * qq + i] - 32 * gs[i]), acc[qq][i]);
                            }
                        }
                    }
                }
        } else {
            // ---- per-block weight scales of this lane's row
            float ws[8], wm[8];
            if constexpr (T::KQ) {
                const float d = half_bits_to_float((unsigned short)(hdr[0] & 0xFFFFu));
                const float dmin = half_bits_to_float((unsigned short)(hdr[0] >> 16));
                    // all eight 6-bit (scale, min) pairs at once, as the bytes of four words (get_scale_min_k4, ggml-quants.c:631-638)
                const u32 u0 = hdr[1], u1 = hdr[2], u2 = hdr[3];
                const u32 s_lo = u0 & 0x3F3F3F3Fu, m_lo = u1 & 0x3F3F3F3Fu;
                const u32 s_hi = (u2 & 0x0F0F0F0Fu) | (((u0 >> 6) & 0x03030303u) << 4);
                const u32 m_hi = ((u2 >> 4) & 0x0F0F0F0Fu) | (((u1 >> 6) & 0x03030303u) << 4);
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const u32 S = j < 4 ? s_lo : s_hi, M = j < 4 ? m_lo : m_hi;
                    ws[j] = d * (float)((S >> (8 * (j & 3))) & 0xFFu);
                    wm[j] = -(dmin * (float)((M >> (8 * (j & 3))) & 0xFFu));
                }
            } else if constexpr (T::PAIR) {
    #pragma unroll
                for (int j = 0; j < 8; j++) {
                    const u32 dm = j < 4 ? hdr[j & 3] : hdr2[j & 3];
                    ws[j] = half_bits_to_float((unsigned short)(dm & 0xFFFFu));
                    wm[j] = half_bits_to_float((unsigned short)(dm >> 16));
                }
            } else if constexpr (TYPE == MI355_IQ4_XS) {
    #pragma unroll
                for (int j = 0; j < 8; j++) ws[j] = iq4xs_block_scale(hdr[0], hdr[1], j);
            } else {
    #pragma unroll
                for (int j = 0; j < 8; j++) ws[j] = f16_of(hdr, j);
            }
    #pragma unroll
            for (int j = 0; j < 8; j++) {
                // operand B: levels 16 kh .. + 16 of block j of weight row r
                i32x4 wop;
                if constexpr (TYPE == MI355_Q8_0) {
                    wop = *(const i32x4 *)(s_w + r * WPAD + 32 * j + 16 * kh);
                } else if constexpr (T::NIB32) {   // byte b of the block's 16: level b in the low nibble, level 16 + b in the high one
                    const u32x4 v = *(const u32x4 *)(s_w + r * WPAD + 16 * j);
                    const u32 fw = j < 4 ? fifth[0][j & 3] : fifth[1][j & 3];   // Q5_0 / Q5_1: bit e = fifth bit of element e
    #pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const u32 nib = (v[i] >> (4 * kh)) & 0x0F0F0F0Fu;   // elements 16 kh + 4 i .. + 4
                        if constexpr (T::TABLE) wop[i] = (int)iq4nl_lookup4(nib);
                        else if constexpr (T::FIFTH32) wop[i] = (int)(nib | spread4(fw >> (16 * kh + 4 * i)));
                        else wop[i] = (int)nib;
                    }
                } else {   // chunk j / 2: byte b of its 32: level b of sub-block 2 (j / 2) in the low nibble, of the next one in the high nibble
                    const u32x4 v = *(const u32x4 *)(s_w + r * WPAD + 32 * (j >> 1) + 16 * kh);
    #pragma unroll
                    for (int i = 0; i < 4; i++) {
                        wop[i] = (int)((v[i] >> (4 * (j & 1))) & 0x0F0F0F0Fu);
                        // Q5_K: bit j of qh byte l is the fifth bit of level l of sub-block j (dequantize_row_q5_K, ggml/src/ggml-quants.c:1482-1507)
                        if constexpr (TYPE == MI355_Q5_K) wop[i] |= (int)(((fifth[0][i] >> j) & 0x01010101u) << 4);
                    }
                }
                const i32x4 aop = *(const i32x4 *)(s_a + am * SK_APAD + 32 * j + 16 * kh);
                i32x16 z;
    #pragma unroll
                for (int i = 0; i < 16; i++) z[i] = 0;
                const i32x16 D = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, wop, z, 0, 0, 0);
    #pragma unroll
                for (int q = 0; q < NI; q++) {
                    const float4 *e = (const float4 *)(s_t + j * (8 * NI) + 8 * q + 4 * kh);
                    const float4 e01 = e[0], e23 = e[1];
                    const float dd[4] = {e01.x, e01.z, e23.x, e23.z};
                    const float xx[4] = {e01.y, e01.w, e23.y, e23.w};
    #pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float Df = (float)D[4 * q + i];
                        if constexpr (TYPE == MI355_Q4_0 || TYPE == MI355_Q5_0) {
                            acc[q][i] = __builtin_fmaf(ws[j], __builtin_fmaf(dd[i], Df, xx[i]), acc[q][i]);   // x = -8 (-16) d sum
                        } else if constexpr (TYPE == MI355_Q8_0 || T::TABLE) {
                            acc[q][i] = __builtin_fmaf(ws[j], dd[i] * Df, acc[q][i]);
                        } else {   // block minimum: + m (Q4_1, Q5_1), - dmin * 6-bit minimum (Q4_K, Q5_K)
                            acc[q][i] = __builtin_fmaf(ws[j], dd[i] * Df, acc[q][i]);
                            acc[q][i] = __builtin_fmaf(wm[j], xx[i], acc[q][i]);                              // x = d sum
                        }
                    }
                }
            }
        }
        wave_lds_sync();   // the next step's copies come after this step's reads
    }

    // the four quarters of K: fixed order 0, 1, 2, 3
    __syncthreads();   // everybody is done with the copies; the same memory now holds the partial sums
    float *s_red = (float *)s_mem;   // [wave][NI * 4][64]
#pragma unroll
    for (int q = 0; q < NI; q++)
#pragma unroll
        for (int i = 0; i < 4; i++) s_red[(wave * NI * 4 + q * 4 + i) * 64 + lane] = acc[q][i];
    __syncthreads();
    // wave w finishes the values v = w, w + 4, ...; lane (r, kh) of value (q, i) is activation row 8 q + 4 kh + i, weight row row0 + r
    for (int v = wave; v < NI * 4; v += 4) {
        const float sum = ((s_red[(0 * NI * 4 + v) * 64 + lane] + s_red[(1 * NI * 4 + v) * 64 + lane]) + s_red[(2 * NI * 4 + v) * 64 + lane]) +
                          s_red[(3 * NI * 4 + v) * 64 + lane];
        const int q = v >> 2, i = v & 3;
        const int c = 8 * q + 4 * kh + i;
        if (c < B && row0 + r < N) {
            const int64_t o = ((int64_t)blockIdx.y * B + c) * dst_stride + row0 + r;
            dst[o] = residual ? sum + residual[o] : sum;
        }
    }
}

// sum of the K slices: dst[c][n] = sum_s part[s][c][n] (+ residual), slices in ascending order
__global__ void __launch_bounds__(256) k_skinny_slices(const float *__restrict__ part, float *__restrict__ dst, const float *__restrict__ residual,
                                                       int64_t N, int B, int64_t dst_stride, int slices) {
    const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int c = blockIdx.y;
    if (n >= N) return;
    float sum = part[(int64_t)c * N + n];
    for (int s = 1; s < slices; s++) sum += part[((int64_t)s * B + c) * N + n];
    const int64_t o = c * dst_stride + n;
    dst[o] = residual ? sum + residual[o] : sum;
}

template <int TYPE, int NI>
void launch_skinny(hipStream_t s, const void *W, const int8_t *aq, const act_ds *ads, float *dst, const float *residual, int64_t N, int K, int B,
                   int64_t dst_stride, int slices, float *part) {
    const int nsteps = K >> 8;
    const int steps_per_slice = (nsteps + slices - 1) / slices;
    const int steps_per_wave = (steps_per_slice + 3) / 4;
    const dim3 grid((unsigned)((N + 31) / 32), (unsigned)slices);
    if (slices == 1) {
        MI355_LAUNCH((k_mm_skinny<TYPE, NI>), grid, dim3(256), 0, s, (const uint8_t *)W, aq, ads, dst, residual, N, K, B, dst_stride, steps_per_slice,
                           steps_per_wave);
    } else {
        MI355_LAUNCH((k_mm_skinny<TYPE, NI>), grid, dim3(256), 0, s, (const uint8_t *)W, aq, ads, part, (const float *)nullptr, N, K, B, N, steps_per_slice,
                           steps_per_wave);
        MI355_LAUNCH(k_skinny_slices, dim3((unsigned)((N + 255) / 256), (unsigned)B), dim3(256), 0, s, part, dst, residual, N, B, dst_stride, slices);
    }
}

template <int TYPE>
void launch_skinny_nt(hipStream_t s, const void *W, const int8_t *aq, const act_ds *ads, float *dst, const float *residual, int64_t N, int K, int B,
                      int64_t dst_stride, int slices, float *part) {
    if (B <= 8) launch_skinny<TYPE, 1>(s, W, aq, ads, dst, residual, N, K, B, dst_stride, slices, part);
    else if (B <= 16) launch_skinny<TYPE, 2>(s, W, aq, ads, dst, residual, N, K, B, dst_stride, slices, part);
    else if (B <= 24) launch_skinny<TYPE, 3>(s, W, aq, ads, dst, residual, N, K, B, dst_stride, slices, part);
    else launch_skinny<TYPE, 4>(s, W, aq, ads, dst, residual, N, K, B, dst_stride, slices, part);
}

// slices of K: launches with fewer than ~1.5 groups per compute unit split K over several groups (and pay a second launch
// that adds the slices), as long as a slice keeps 4 steps; a short K with at most 8 activation rows is quicker in one go.
int skinny_slices(int64_t N, int64_t K, int64_t B) {
    const int64_t tiles = (N + 31) / 32, nsteps = K >> 8;
    if (tiles >= 384 || (B <= 8 && nsteps <= 16)) return 1;
    int s = 1;
    while (s < 8 && tiles * s < 512 && nsteps / (s * 2) >= 4) s *= 2;
    return s;
}

}  // namespace

}  // namespace mi355

using namespace mi355;

extern "C" {

int mi355_mul_mat_skinny_supported(int type, const void *W, int64_t K, int64_t B) {
    return is_weight_type(type) && B >= 1 && B <= 32 && K > 0 && K % 256 == 0 && K < (int64_t(1) << 30) &&
           layout_aligned(W, make_row_layout(type, K));
}

size_t mi355_mul_mat_skinny_ws_bytes(int64_t N, int64_t K, int64_t B) {
    const int s = skinny_slices(N, K, B);
    return s > 1 ? (size_t)s * B * N * sizeof(float) : 0;
}

int mi355_mul_mat_skinny(void *stream, int type, const void *W, const void *act, float *dst, const float *residual, int64_t N, int64_t K, int64_t B,
                         int64_t dst_stride, void *ws, size_t ws_bytes) {
    MI355_REQUIRE(mi355_mul_mat_skinny_supported(type, W, K, B), "mul_mat_skinny: type %d, K=%lld, B=%lld or the weight alignment is not supported", type,
                  (long long)K, (long long)B);
    MI355_REQUIRE(N > 0 && dst_stride >= N, "mul_mat_skinny: bad shape N=%lld dst_stride=%lld", (long long)N, (long long)dst_stride);
    MI355_REQUIRE(((uintptr_t)act & 15) == 0, "mul_mat_skinny: activation workspace is not 16-byte aligned");
    int slices = skinny_slices(N, K, B);
    if (slices > 1 && (ws == nullptr || ws_bytes < (size_t)slices * B * N * sizeof(float))) slices = 1;   // no room for partial sums: one slice
    hipStream_t s = (hipStream_t)stream;
    const int8_t *aq = (const int8_t *)act;
    const act_ds *ads = (const act_ds *)(aq + B * K);
#define X(T) launch_skinny_nt<T>(s, W, aq, ads, dst, residual, N, (int)K, (int)B, dst_stride, slices, (float *)ws);
    MI355_WEIGHT_TYPE_SWITCH(type, X)
#undef X
    return launch_status("k_mm_skinny");
}

}  // extern "C"
