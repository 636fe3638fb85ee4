// Batched quantized GEMM on the int8 matrix cores (B > 8):
//   dst[b][n] = sum_k W[n][k] * x[b][k],  W block-quantized, x quantized to Q8_1 on the device.
//
// A 256-thread group (4 waves, 2 x 2) owns a 128 (weight rows) x BN (activation rows)
// tile of dst and walks K in stages of 128 elements.  Per stage the weight rows are
// unpacked from their 4/6/8-bit blocks to int8 in LDS (16-byte streaming loads from HBM,
// each weight byte is unpacked once per group and reused for BN activation rows), the
// activation int8 rows are copied to LDS, and each wave contracts its 64 x (BN/2)
// sub-tile with v_mfma_i32_32x32x32_i8, one instruction per 32-element quantization block,
// so every MFMA result is an exact per-block integer dot.  Block results are scaled by
// (weight block scale) x (activation block scale) and accumulated in f32 registers.
//
//   Q4_0 : level - 8 as int8, scale d                    (one MFMA per block)
//   Q8_0 : level as int8, scale d
//   Q5_0 : level - 16 as int8, scale d;  IQ4_NL : the table value of the nibble as int8, scale d
//   IQ4_XS : as IQ4_NL, scale d * (ls - 32) from the super-block's header
//   Q4_1, Q5_1 : level 0..15 / 0..31 as int8, scale d; the "+ m * d_x * sum(q)" term of the stage's four blocks is added with one
//          v_mfma_f32_32x32x16_f16 on (fp16 dx*sum(q), the reference's `s` field of block_q8_1) x (fp16 m)
//   Q4_K, Q5_K : level 0..15 / 0..31 as int8, scale d*sc; the "- dmin*m*sum(q)" term of all blocks is
//          added with one v_mfma_f32_32x32x16_f16 per stage on (fp16 dx*sum(q)) x (fp16 dmin*m)
//   Q6_K : level - 32 as int8, scale d*sc per 16 elements (v_mfma_i32_32x32x16_i8, two per block)
//
// MFMA operand mapping used here (A = activations, B = weights, D[i][j], i = activation
// row, j = weight row): lane l supplies row/column l % 32 and the k bytes
// [16*(l/32), 16*(l/32)+16) of the 32-wide step (8-byte halves for the 16-wide step);
// D register r of lane l is element i = 8*(r/4) + 4*(l/32) + r%4, j = l % 32.  Both
// operands use the same k split, so the contraction is independent of how the hardware
// numbers k internally.
//
// Group ids are remapped so that the groups sharing one weight panel run on the same XCD
// (ids are dealt round-robin over the 8 XCDs) and hit its L2 instead of HBM.
#include "common.hpp"
#include "qdot.hpp"
#include "tiles.hpp"

namespace mi355 {

constexpr int MMQ_BM = 128;          // weight rows per group
constexpr int MMQ_BK = 128;          // K elements per stage
constexpr int MMQ_LDK = MMQ_BK + 16; // LDS row pitch in bytes (pad to spread banks)

template <int TYPE> struct mmq_cfg {
    static constexpr int G = TYPE == MI355_Q6_K ? 16 : 32;   // elements per weight scale
    static constexpr int NG = MMQ_BK / G;                    // weight scales per row per stage
    // a per-block offset rides on the sums of the activation levels: - dmin * m (Q4_K), + m (Q4_1, Q5_1)
    static constexpr bool MIN = TYPE == MI355_Q4_K || TYPE == MI355_Q5_K || TYPE == MI355_Q4_1 || TYPE == MI355_Q5_1;
    // 16 bytes of nibbles per block with a per-block scale: one request / commit form serves them all
    static constexpr bool NIBBLE32 = TYPE == MI355_Q4_0 || TYPE == MI355_Q4_1 || TYPE == MI355_Q5_0 || TYPE == MI355_Q5_1 || TYPE == MI355_IQ4_NL ||
                                     TYPE == MI355_IQ4_XS;
    static constexpr bool PREFETCH = NIBBLE32 || TYPE == MI355_Q8_0;
};

// ---- stage loaders: global (device layout) -> int8 rows + scales in LDS ----------------
// sW  : int8 [MMQ_BM][MMQ_LDK]
// sWs : float [NG][MMQ_BM]   (scale g of row r at sWs[g*MMQ_BM + r])
// sWo : fp16  [MMQ_BM][4]    (Q4_K only: dmin*m of the 4 sub-blocks of the stage)
template <int TYPE>
__device__ __forceinline__ void load_weight_stage(const uint8_t *__restrict__ W, const row_layout &L, int64_t row0,
                                                  int64_t N, int64_t k0, int8_t *sW, float *sWs, _Float16 *sWo) {
    const int tid = threadIdx.x;
    if constexpr (TYPE == MI355_Q4_0) {
        // 128 rows x 4 blocks of 16 B
#pragma unroll
        for (int it = 0; it < 2; it++) {
            const int idx = tid + it * 256;
            const int r = idx >> 2, b = idx & 3;
            const int64_t row = row0 + r < N ? row0 + r : N - 1;
            const uint8_t *wrow = W + row * L.row_bytes;
            const int64_t blk = (k0 >> 5) + b;
            const u32x4 q = load16(wrow + blk * 16);
            u32x4 lo, hi;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                // nibble - 8 per byte without cross-byte borrow
                lo[i] = (((q[i] & 0x0F0F0F0Fu) | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
                hi[i] = ((((q[i] >> 4) & 0x0F0F0F0Fu) | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
            }
            *(u32x4 *)(sW + r * MMQ_LDK + b * 32) = lo;
            *(u32x4 *)(sW + r * MMQ_LDK + b * 32 + 16) = hi;
            sWs[b * MMQ_BM + r] = half_bits_to_float(*(const unsigned short *)(wrow + L.off_b + blk * 2));
        }
    } else if constexpr (TYPE == MI355_Q8_0) {
        // 128 rows x 4 blocks x 2 halves of 16 B
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const int idx = tid + it * 256;
            const int r = idx >> 3, c = idx & 7;   // c: 16-byte piece of the stage
            const int64_t row = row0 + r < N ? row0 + r : N - 1;
            const uint8_t *wrow = W + row * L.row_bytes;
            const u32x4 q = load16(wrow + k0 + c * 16);
            *(u32x4 *)(sW + r * MMQ_LDK + c * 16) = q;
            if ((c & 1) == 0) {
                const int b = c >> 1;
                sWs[b * MMQ_BM + r] = half_bits_to_float(*(const unsigned short *)(wrow + L.off_b + ((k0 >> 5) + b) * 2));
            }
        }
    } else if constexpr (TYPE == MI355_Q4_K || TYPE == MI355_Q5_K) {
        // stage = half a super-block: sub-blocks j0..j0+3, 64 B of qs per row = 4 pieces of 16 B (Q5_K: bit j of qh[l] is the fifth
        // bit of element l of sub-block j, dequantize_row_q5_K, ggml/src/ggml-quants.c:1482-1507)
        constexpr int BB = TYPE == MI355_Q4_K ? Q4_K_BYTES : Q5_K_BYTES, QS = TYPE == MI355_Q4_K ? 16 : 48;
        const int64_t sb = k0 >> 8;
        const int half = (int)((k0 >> 7) & 1);
#pragma unroll
        for (int it = 0; it < 2; it++) {
            const int idx = tid + it * 256;
            const int r = idx >> 2, p = idx & 3;          // p: piece -> group gl = p>>1 of the stage, half h = p&1
            const int gl = p >> 1, h = p & 1;
            const int64_t row = row0 + r < N ? row0 + r : N - 1;
            const uint8_t *blk = W + row * L.row_bytes + sb * BB;
            const u32x4 q = load16(blk + QS + (half * 2 + gl) * 32 + h * 16);
            u32x4 lo, hi;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                lo[i] = q[i] & 0x0F0F0F0Fu;
                hi[i] = (q[i] >> 4) & 0x0F0F0F0Fu;
            }
            if constexpr (TYPE == MI355_Q5_K) {
                const u32x4 qh = load16(blk + 16 + h * 16);
                const int ja = half * 4 + 2 * gl;         // sub-block of the low nibbles; the high nibbles are the next one
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    lo[i] |= ((qh[i] >> ja) & 0x01010101u) << 4;
                    hi[i] |= ((qh[i] >> (ja + 1)) & 0x01010101u) << 4;
                }
            }
            *(u32x4 *)(sW + r * MMQ_LDK + (2 * gl) * 32 + h * 16) = lo;
            *(u32x4 *)(sW + r * MMQ_LDK + (2 * gl + 1) * 32 + h * 16) = hi;
            // this thread also owns the (scale, min) of sub-block p of the stage
            const u32x4 hdr = load16(blk);
            const float d = half_bits_to_float((unsigned short)(hdr[0] & 0xFFFFu));
            const float dmin = half_bits_to_float((unsigned short)(hdr[0] >> 16));
            int sc, mn;
            q4k_scale_min(hdr[1], hdr[2], hdr[3], half * 4 + p, sc, mn);
            sWs[p * MMQ_BM + r] = d * (float)sc;
            sWo[r * 4 + p] = (_Float16)(dmin * (float)mn);
        }
    } else {   // Q6_K: stage = half hf of a super-block: 64 B ql + 32 B qh, 8 scales
        const int64_t sb = k0 >> 8;
        const int hf = (int)((k0 >> 7) & 1);
#pragma unroll
        for (int it = 0; it < 2; it++) {
            const int idx = tid + it * 256;
            const int r = idx >> 2, p = idx & 3;          // p: 16-byte piece of this half's ql
            const int l0 = 16 * (p & 1), qa = p >> 1;
            const int64_t row = row0 + r < N ? row0 + r : N - 1;
            const uint8_t *wrow = W + row * L.row_bytes;
            const u32x4 ql = load16(wrow + sb * 128 + hf * 64 + p * 16);
            const u32x4 qh = load16(wrow + L.off_b + sb * 64 + hf * 32 + l0);
            u32x4 vA, vB;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const u32 a = (ql[i] & 0x0F0F0F0Fu) | (((qh[i] >> (2 * qa)) & 0x03030303u) << 4);
                const u32 b = ((ql[i] >> 4) & 0x0F0F0F0Fu) | (((qh[i] >> (2 * qa + 4)) & 0x03030303u) << 4);
                // level - 32 per byte: flip bit 5, then sign-extend it into bits 6..7
                const u32 ta = a ^ 0x20202020u, tb = b ^ 0x20202020u;
                const u32 ma = ta & 0x20202020u, mb = tb & 0x20202020u;
                vA[i] = ta | (ma << 1) | (ma << 2);
                vB[i] = tb | (mb << 1) | (mb << 2);
            }
            *(u32x4 *)(sW + r * MMQ_LDK + qa * 32 + l0) = vA;
            *(u32x4 *)(sW + r * MMQ_LDK + (qa + 2) * 32 + l0) = vB;
            // scales of 16-element groups 2p and 2p+1 of the stage
            const float d = half_bits_to_float(*(const unsigned short *)(wrow + L.off_d + sb * 2));
            const int8_t *sc = (const int8_t *)(wrow + L.off_c + sb * 16 + hf * 8);
            sWs[(2 * p) * MMQ_BM + r] = d * (float)sc[2 * p];
            sWs[(2 * p + 1) * MMQ_BM + r] = d * (float)sc[2 * p + 1];
        }
    }
}

// sA  : int8 [BN][MMQ_LDK];  sAd : float [4][BN] block scales;  sAs : fp16 [BN][4]  dx*sum(q) (Q4_K)
template <int TYPE, int BN>
__device__ __forceinline__ void load_act_stage(const int8_t *__restrict__ aq, const act_ds *__restrict__ ads,
                                               int64_t col0, int64_t B, int64_t K, int64_t k0, int8_t *sA, float *sAd,
                                               _Float16 *sAs) {
    const int tid = threadIdx.x;
    const int64_t nblk = K >> 5;
    // BN rows x 8 pieces of 16 B
#pragma unroll
    for (int it = 0; it < BN * 8 / 256; it++) {
        const int idx = tid + it * 256;
        const int r = idx >> 3, c = idx & 7;
        const int64_t col = col0 + r < B ? col0 + r : B - 1;
        *(u32x4 *)(sA + r * MMQ_LDK + c * 16) = load16(aq + col * K + k0 + c * 16);
    }
    // BN rows x 4 block scales
#pragma unroll
    for (int it = 0; it < (BN * 4 + 255) / 256; it++) {
        const int idx = tid + it * 256;
        if (idx < BN * 4) {
            const int r = idx >> 2, b = idx & 3;
            const int64_t col = col0 + r < B ? col0 + r : B - 1;
            const act_ds s = ads[col * nblk + (k0 >> 5) + b];
            sAd[b * BN + r] = s.d;
            if constexpr (TYPE == MI355_Q4_K || TYPE == MI355_Q5_K) sAs[r * 4 + b] = (_Float16)(s.d * (float)s.sum);
        }
    }
}

// ---- the same stages split into "request" (global -> registers) and "commit" (unpack -> LDS), so that the next stage's bytes
// travel while the current stage is contracted (Q4_0 / Q8_0, whose per-32 scales keep them on this kernel)
template <int TYPE, bool NIB = mmq_cfg<TYPE>::NIBBLE32> struct mmq_wregs {};
// Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL, IQ4_XS: thread t owns blocks (row, b) = (idx >> 2, idx & 3), idx = t and t + 256
template <int TYPE> struct mmq_wregs<TYPE, true> {
    static constexpr bool HAS_QH = TYPE == MI355_Q5_0 || TYPE == MI355_Q5_1;
    static constexpr bool HAS_MIN = TYPE == MI355_Q4_1 || TYPE == MI355_Q5_1;
    u32x4 q[2];
    u32 qh[2];
    u32 dm[2];   // fp16 d in the low half, fp16 m above it (HAS_MIN); IQ4_XS: the bits of the f32 block scale
    __device__ __forceinline__ void fetch(const uint8_t *__restrict__ W, const row_layout &L, int64_t row0, int64_t N, int64_t k0, int tid) {
#pragma unroll
        for (int it = 0; it < 2; it++) {
            const int idx = tid + it * 256;
            const int r = idx >> 2, b = idx & 3;
            const int64_t row = row0 + r < N ? row0 + r : N - 1;
            const uint8_t *wrow = W + row * L.row_bytes;
            const int64_t blk = (k0 >> 5) + b;
            q[it] = load16(wrow + blk * 16);
            if constexpr (HAS_QH) qh[it] = *(const u32 *)(wrow + L.off_b + blk * 4);
            const int so = HAS_QH ? L.off_c : L.off_b;   // the scales follow the fifth bits where there are any
            if constexpr (TYPE == MI355_IQ4_XS) {
                const uint2 h = *(const uint2 *)(wrow + L.off_b + (blk >> 3) * 8);
                dm[it] = __builtin_bit_cast(u32, iq4xs_block_scale(h.x, h.y, (int)(blk & 7)));
            } else if constexpr (HAS_MIN) dm[it] = *(const u32 *)(wrow + so + blk * 4);
            else dm[it] = *(const unsigned short *)(wrow + so + blk * 2);
        }
    }
    __device__ __forceinline__ void commit(int8_t *sW, float *sWs, _Float16 *sWo, int tid) const {
#pragma unroll
        for (int it = 0; it < 2; it++) {
            const int idx = tid + it * 256;
            const int r = idx >> 2, b = idx & 3;
            u32x4 lo, hi;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                u32 a = q[it][i] & 0x0F0F0F0Fu, c = (q[it][i] >> 4) & 0x0F0F0F0Fu;
                if constexpr (HAS_QH) {   // bit j of qh: element j; dword i holds elements 4i.. (low nibbles) and 16 + 4i.. (high)
                    a |= spread4(qh[it] >> (4 * i));
                    c |= spread4(qh[it] >> (16 + 4 * i));
                }
                if constexpr (TYPE == MI355_Q4_0) {          // nibble - 8 per byte without cross-byte borrow
                    a = ((a | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
                    c = ((c | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
                } else if constexpr (TYPE == MI355_Q5_0) {   // level - 16
                    a = ((a | 0x80808080u) - 0x10101010u) ^ 0x80808080u;
                    c = ((c | 0x80808080u) - 0x10101010u) ^ 0x80808080u;
                } else if constexpr (TYPE == MI355_IQ4_NL || TYPE == MI355_IQ4_XS) {
                    a = iq4nl_lookup4(a);
                    c = iq4nl_lookup4(c);
                }
                lo[i] = a;
                hi[i] = c;
            }
            *(u32x4 *)(sW + r * MMQ_LDK + b * 32) = lo;
            *(u32x4 *)(sW + r * MMQ_LDK + b * 32 + 16) = hi;
            if constexpr (TYPE == MI355_IQ4_XS) sWs[b * MMQ_BM + r] = __builtin_bit_cast(float, dm[it]);
            else sWs[b * MMQ_BM + r] = half_bits_to_float((unsigned short)(dm[it] & 0xFFFFu));
            if constexpr (HAS_MIN) {
                union { unsigned short u; _Float16 f; } m;
                m.u = (unsigned short)(dm[it] >> 16);
                sWo[r * 4 + b] = m.f;
            }
        }
    }
};
template <> struct mmq_wregs<MI355_Q8_0, false> {
    u32x4 q[4];
    unsigned short d[4];
    __device__ __forceinline__ void fetch(const uint8_t *__restrict__ W, const row_layout &L, int64_t row0, int64_t N, int64_t k0, int tid) {
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const int idx = tid + it * 256;
            const int r = idx >> 3, c = idx & 7;   // c: 16-byte piece of the stage
            const int64_t row = row0 + r < N ? row0 + r : N - 1;
            const uint8_t *wrow = W + row * L.row_bytes;
            q[it] = load16(wrow + k0 + c * 16);
            d[it] = *(const unsigned short *)(wrow + L.off_b + ((k0 >> 5) + (c >> 1)) * 2);   // both pieces of a block read its scale
        }
    }
    __device__ __forceinline__ void commit(int8_t *sW, float *sWs, _Float16 *, int tid) const {
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const int idx = tid + it * 256;
            const int r = idx >> 3, c = idx & 7;
            *(u32x4 *)(sW + r * MMQ_LDK + c * 16) = q[it];
            if ((c & 1) == 0) sWs[(c >> 1) * MMQ_BM + r] = half_bits_to_float(d[it]);
        }
    }
};
template <int BN, bool WITH_SUM> struct mmq_aregs {
    static constexpr int NQ = BN * 8 / 256, NS = (BN * 4 + 255) / 256;
    u32x4 q[NQ];
    float d[NS];
    int sum[NS];
    // row_of: null, or the activation row of every column (the routed form: columns are (token, expert slot) pairs sorted by expert)
    __device__ __forceinline__ void fetch(const int8_t *__restrict__ aq, const act_ds *__restrict__ ads, int64_t col0, int64_t B, int64_t K, int64_t k0,
                                          int tid, const int32_t *__restrict__ row_of = nullptr) {
        const int64_t nblk = K >> 5;
#pragma unroll
        for (int it = 0; it < NQ; it++) {
            const int idx = tid + it * 256;
            const int r = idx >> 3, c = idx & 7;
            int64_t col = col0 + r < B ? col0 + r : B - 1;
            if (row_of) col = row_of[col];
            q[it] = load16(aq + col * K + k0 + c * 16);
        }
#pragma unroll
        for (int it = 0; it < NS; it++) {
            const int idx = tid + it * 256;
            const int r = (idx >> 2) < BN ? (idx >> 2) : BN - 1, b = idx & 3;
            int64_t col = col0 + r < B ? col0 + r : B - 1;
            if (row_of) col = row_of[col];
            const act_ds e = ads[col * nblk + (k0 >> 5) + b];
            d[it] = e.d;
            if constexpr (WITH_SUM) sum[it] = e.sum;
        }
    }
    __device__ __forceinline__ void commit(int8_t *sA, float *sAd, _Float16 *sAs, int tid) const {
#pragma unroll
        for (int it = 0; it < NQ; it++) {
            const int idx = tid + it * 256;
            const int r = idx >> 3, c = idx & 7;
            *(u32x4 *)(sA + r * MMQ_LDK + c * 16) = q[it];
        }
#pragma unroll
        for (int it = 0; it < NS; it++) {
            const int idx = tid + it * 256;
            if (idx < BN * 4) {
                sAd[(idx & 3) * BN + (idx >> 2)] = d[it];
                if constexpr (WITH_SUM) sAs[idx] = (_Float16)(d[it] * (float)sum[it]);   // [row][block of the stage]
            }
        }
    }
};

// MUL_MAT_ID with many slots (ID): column tile ct of the slot list sorted by expert (k_route_slots) holds slots [first, end) of one
// expert; their activation rows are gathered through act_row and their results go to the dst rows of dst_row.
struct mmq32_route {
    const int32_t *act_row;
    const int32_t *dst_row;
    const int32_t *tiles;      // per column tile: expert, first slot, end slot, -
    const int32_t *n_tiles;    // column tiles in use (device value)
    int64_t expert_bytes;      // from one expert's matrix to the next
};

template <int TYPE, int TN, bool ID = false>
__global__ void __launch_bounds__(256) k_mmq(const uint8_t *__restrict__ W, const int8_t *__restrict__ aq,
                                             const act_ds *__restrict__ ads, float *__restrict__ dst, int64_t N,
                                             int64_t K, int64_t B, int64_t dst_stride, row_layout L, int n_col_tiles,
                                             int n_groups, int n_groups_padded, mmq32_route route) {
    typedef mmq_cfg<TYPE> C;
    static_assert(!ID || C::PREFETCH, "the routed form exists for the per-32-block types");
    constexpr int BN = 64 * TN;
    __shared__ __attribute__((aligned(16))) int8_t sW[MMQ_BM * MMQ_LDK];
    __shared__ __attribute__((aligned(16))) int8_t sA[BN * MMQ_LDK];
    __shared__ __attribute__((aligned(16))) float sWs[C::NG * MMQ_BM];
    __shared__ __attribute__((aligned(16))) float sAd[4 * BN];
    __shared__ __attribute__((aligned(16))) _Float16 sWo[C::MIN ? MMQ_BM * 4 : 4];
    __shared__ __attribute__((aligned(16))) _Float16 sAs[C::MIN ? BN * 4 : 4];

    // XCD-aware id: hardware deals group ids round-robin over 8 XCDs; make logical neighbours share an XCD
    const int per_xcd = n_groups_padded >> 3;
    const int lid = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (lid >= n_groups) return;   // uniform for the whole group
    const int64_t row0 = (int64_t)(lid / n_col_tiles) * MMQ_BM;
    int64_t col0 = (int64_t)(lid % n_col_tiles) * BN;
    const int32_t *row_of = nullptr;
    if constexpr (ID) {
        const int ct = lid % n_col_tiles;
        if (ct >= *route.n_tiles) return;   // uniform for the whole group
        W += (int64_t)route.tiles[4 * ct] * route.expert_bytes;
        col0 = route.tiles[4 * ct + 1];
        B = route.tiles[4 * ct + 2];
        row_of = route.act_row;
    }

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    const int wrow0 = (wave & 1) * 64;           // weight rows of this wave inside the tile
    const int wcol0 = (wave >> 1) * (32 * TN);   // activation rows of this wave inside the tile

    f32x16 acc[TN][2];
#pragma unroll
    for (int tb = 0; tb < TN; tb++)
#pragma unroll
        for (int tw = 0; tw < 2; tw++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[tb][tw][r] = 0.0f;

    // split K: grid row y walks stages [k_lo, k_hi) and writes its sums to slice y of `dst` (a workspace then, see launch_mmq)
    const int64_t stages = K / MMQ_BK, st_per = (stages + gridDim.y - 1) / gridDim.y;
    const int64_t k_lo = (int64_t)blockIdx.y * st_per * MMQ_BK;
    const int64_t k_hi = k_lo + st_per * MMQ_BK < K ? k_lo + st_per * MMQ_BK : K;
    if (gridDim.y > 1) dst += (int64_t)blockIdx.y * B * dst_stride;

    constexpr bool PREFETCH = C::PREFETCH;
    mmq_wregs<TYPE> wregs;
    mmq_aregs<BN, C::MIN> aregs;
    if constexpr (PREFETCH) {
        wregs.fetch(W, L, row0, N, k_lo, threadIdx.x);
        aregs.fetch(aq, ads, col0, B, K, k_lo, threadIdx.x, row_of);
    }
    for (int64_t k0 = k_lo; k0 < k_hi; k0 += MMQ_BK) {
        __syncthreads();
        if constexpr (PREFETCH) {
            wregs.commit(sW, sWs, sWo, threadIdx.x);
            aregs.commit(sA, sAd, sAs, threadIdx.x);
        } else {
            load_weight_stage<TYPE>(W, L, row0, N, k0, sW, sWs, sWo);
            load_act_stage<TYPE, BN>(aq, ads, col0, B, K, k0, sA, sAd, sAs);
        }
        __syncthreads();
        if constexpr (PREFETCH) {
            // past the end the last stage is requested again and never committed: no branch, the loads stay here
            const int64_t k1 = k0 + MMQ_BK < k_hi ? k0 + MMQ_BK : k0;
            wregs.fetch(W, L, row0, N, k1, threadIdx.x);
            aregs.fetch(aq, ads, col0, B, K, k1, threadIdx.x, row_of);
            __builtin_amdgcn_sched_barrier(0);   // requested now, a whole stage ahead of their commit
        }

#pragma unroll
        for (int ks = 0; ks < 4; ks++) {   // one Q8_1 block per step
            // activation block scales for this lane's 16 D rows: i = 8*(r/4) + 4*lhi + r%4
            f32x4 dx[TN][4];
#pragma unroll
            for (int tb = 0; tb < TN; tb++)
#pragma unroll
                for (int q = 0; q < 4; q++) dx[tb][q] = *(const f32x4 *)(sAd + ks * BN + wcol0 + tb * 32 + 8 * q + 4 * lhi);

            if constexpr (C::G == 32) {
                i32x4 af[TN], bf[2];
#pragma unroll
                for (int tb = 0; tb < TN; tb++) af[tb] = *(const i32x4 *)(sA + (wcol0 + tb * 32 + l32) * MMQ_LDK + ks * 32 + 16 * lhi);
#pragma unroll
                for (int tw = 0; tw < 2; tw++) bf[tw] = *(const i32x4 *)(sW + (wrow0 + tw * 32 + l32) * MMQ_LDK + ks * 32 + 16 * lhi);
#pragma unroll
                for (int tw = 0; tw < 2; tw++) {
                    const float dw = sWs[ks * MMQ_BM + wrow0 + tw * 32 + l32];
#pragma unroll
                    for (int tb = 0; tb < TN; tb++) {
                        i32x16 z;
#pragma unroll
                        for (int r = 0; r < 16; r++) z[r] = 0;
                        const i32x16 I = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[tb], bf[tw], z, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 16; r++) acc[tb][tw][r] += (float)I[r] * (dw * dx[tb][r >> 2][r & 3]);
                    }
                }
            } else {
#pragma unroll
                for (int hs = 0; hs < 2; hs++) {   // two 16-element scale groups per block
                    long af[TN], bf[2];
#pragma unroll
                    for (int tb = 0; tb < TN; tb++) af[tb] = *(const long *)(sA + (wcol0 + tb * 32 + l32) * MMQ_LDK + ks * 32 + hs * 16 + 8 * lhi);
#pragma unroll
                    for (int tw = 0; tw < 2; tw++) bf[tw] = *(const long *)(sW + (wrow0 + tw * 32 + l32) * MMQ_LDK + ks * 32 + hs * 16 + 8 * lhi);
#pragma unroll
                    for (int tw = 0; tw < 2; tw++) {
                        const float dw = sWs[(ks * 2 + hs) * MMQ_BM + wrow0 + tw * 32 + l32];
#pragma unroll
                        for (int tb = 0; tb < TN; tb++) {
                            i32x16 z;
#pragma unroll
                            for (int r = 0; r < 16; r++) z[r] = 0;
                            const i32x16 I = __builtin_amdgcn_mfma_i32_32x32x16_i8(af[tb], bf[tw], z, 0, 0, 0);
#pragma unroll
                            for (int r = 0; r < 16; r++) acc[tb][tw][r] += (float)I[r] * (dw * dx[tb][r >> 2][r & 3]);
                        }
                    }
                }
            }
        }

        if constexpr (C::MIN) {
            // acc -= sum_b (dx*sum q)[i][b] * (dmin*m)[j][b] over the 4 blocks of the stage (Q4_K; Q4_1 and Q5_1: acc += ... * m[j][b]):
            // a 32x32x16 f16 MFMA whose k slots 0..3 hold the blocks (lanes 32..63 and slots 4..7 are zero)
            f16x8 af[TN], bf[2];
#pragma unroll
            for (int tb = 0; tb < TN; tb++) {
                const f16x4 v = *(const f16x4 *)(sAs + (wcol0 + tb * 32 + l32) * 4);
#pragma unroll
                for (int i = 0; i < 8; i++) af[tb][i] = (i < 4 && lhi == 0) ? (TYPE == MI355_Q4_K || TYPE == MI355_Q5_K ? (_Float16)(-(float)v[i & 3]) : v[i & 3]) : (_Float16)0.0f;
            }
#pragma unroll
            for (int tw = 0; tw < 2; tw++) {
                const f16x4 v = *(const f16x4 *)(sWo + (wrow0 + tw * 32 + l32) * 4);
#pragma unroll
                for (int i = 0; i < 8; i++) bf[tw][i] = (i < 4 && lhi == 0) ? v[i & 3] : (_Float16)0.0f;
            }
#pragma unroll
            for (int tb = 0; tb < TN; tb++)
#pragma unroll
                for (int tw = 0; tw < 2; tw++) acc[tb][tw] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[tb], bf[tw], acc[tb][tw], 0, 0, 0);
        }
    }

    // store: lane holds weight row j = l32 of each 32-wide tile, 16 activation rows
#pragma unroll
    for (int tb = 0; tb < TN; tb++)
#pragma unroll
        for (int tw = 0; tw < 2; tw++) {
            const int64_t n = row0 + wrow0 + tw * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t b = col0 + wcol0 + tb * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
                if (n < N && b < B) dst[(ID ? (int64_t)route.dst_row[b] : b) * dst_stride + n] = acc[tb][tw][r];
            }
        }
}

// A product with few tiles leaves most of the chip idle while each group walks all of K: such launches are cut along K into
// slices that run side by side and a second launch adds the slices in fixed order.  At least four stages per slice, at most
// eight slices, at most two groups per compute unit.
static int mmq_slices(int64_t N, int64_t K, int64_t B) {
    const int64_t bn = B <= 64 ? 64 : 128;
    const int64_t groups = ((N + MMQ_BM - 1) / MMQ_BM) * ((B + bn - 1) / bn), stages = K / MMQ_BK;
    int64_t n = 512 / groups;
    if (n > stages / 4) n = stages / 4;
    if (n > 8) n = 8;
    if (n < 2) return 1;
    const int64_t per = (stages + n - 1) / n;
    return (int)((stages + per - 1) / per);   // no empty slice
}

__global__ void __launch_bounds__(256) k_mmq_split_sum(const float *__restrict__ part, float *__restrict__ dst, int64_t N, int64_t B, int64_t dst_stride,
                                                       int n_slices) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N * B) return;
    float acc = part[i];
    for (int sl = 1; sl < n_slices; sl++) acc = add_rn(acc, part[(int64_t)sl * N * B + i]);
    dst[(i / N) * dst_stride + i % N] = acc;
}

template <int TYPE, int TN>
static void launch_mmq(hipStream_t s, const void *W, const void *act, float *dst, int64_t N, int64_t K, int64_t B,
                       int64_t dst_stride, void *ws, size_t ws_bytes) {
    constexpr int BN = 64 * TN;
    const row_layout L = make_row_layout(TYPE, K);
    const int8_t *aq = (const int8_t *)act;
    const act_ds *ads = (const act_ds *)(aq + B * K);
    const int n_row_tiles = (int)((N + MMQ_BM - 1) / MMQ_BM);
    const int n_col_tiles = (int)((B + BN - 1) / BN);
    const int n_groups = n_row_tiles * n_col_tiles;
    const int n_groups_padded = (n_groups + 7) & ~7;
    int n_slices = mmq_slices(N, K, B);
    if (n_slices > 1 && (ws == nullptr || ((uintptr_t)ws & 15) != 0 || ws_bytes < (size_t)n_slices * (size_t)N * (size_t)B * sizeof(float))) n_slices = 1;
    if (n_slices > 1) {
        MI355_LAUNCH((k_mmq<TYPE, TN>), dim3((unsigned)n_groups_padded, (unsigned)n_slices), dim3(256), 0, s, (const uint8_t *)W, aq, ads,
                           (float *)ws, N, K, B, N, L, n_col_tiles, n_groups, n_groups_padded, mmq32_route{});
        MI355_LAUNCH(k_mmq_split_sum, dim3((unsigned)((N * B + 255) / 256)), dim3(256), 0, s, (const float *)ws, dst, N, B, dst_stride, n_slices);
        return;
    }
    MI355_LAUNCH((k_mmq<TYPE, TN>), dim3((unsigned)n_groups_padded), dim3(256), 0, s, (const uint8_t *)W, aq, ads,
                       dst, N, K, B, dst_stride, L, n_col_tiles, n_groups, n_groups_padded, mmq32_route{});
}

template <int TYPE>
static void launch_mmq_tn(hipStream_t s, const void *W, const void *act, float *dst, int64_t N, int64_t K, int64_t B,
                          int64_t dst_stride, void *ws, size_t ws_bytes) {
    if (B <= 64) launch_mmq<TYPE, 1>(s, W, act, dst, N, K, B, dst_stride, ws, ws_bytes);
    else launch_mmq<TYPE, 2>(s, W, act, dst, N, K, B, dst_stride, ws, ws_bytes);
}

// the routed launch: 128-column tiles over the slot list sorted by expert; the routing workspace is laid out as for the
// super-block kernel's routed form (act_row[S], dst_row[S], tiles[4 x ((S + 63) / 64 + n_expert)], n_tiles)
template <int TYPE>
static void launch_mmq_id(hipStream_t s, const void *as, const void *act, int64_t act_rows, const int32_t *ids, int64_t ids_stride, float *dst, int64_t N,
                          int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T, void *route_ws) {
    constexpr int BN = 128;
    const int64_t S = T * n_used;
    const int max_tiles = (int)((S + BN - 1) / BN + n_expert);
    int32_t *act_row = (int32_t *)route_ws, *dst_row = act_row + S, *tiles = dst_row + S, *n_tiles = tiles + 4 * ((S + 63) / 64 + n_expert);
    launch_route_slots(s, ids, ids_stride, n_expert, n_used, nb1, T, BN, act_row, dst_row, tiles, n_tiles);
    const row_layout L = make_row_layout(TYPE, K);
    const int8_t *aq = (const int8_t *)act;
    const act_ds *ads = (const act_ds *)(aq + act_rows * K);
    const int n_row_tiles = (int)((N + MMQ_BM - 1) / MMQ_BM);
    const int n_groups = n_row_tiles * max_tiles;
    const int n_groups_padded = (n_groups + 7) & ~7;
    const mmq32_route route = {act_row, dst_row, tiles, n_tiles, N * L.row_bytes};
    MI355_LAUNCH((k_mmq<TYPE, 2, true>), dim3((unsigned)n_groups_padded), dim3(256), 0, s, (const uint8_t *)as, aq, ads, dst, N, K, S, N, L, max_tiles,
                 n_groups, n_groups_padded, route);
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_mul_mat_id_q_supported(int type, const void *as, int64_t N, int64_t K, int64_t n_expert) {
    const bool typed = type == MI355_Q4_0 || type == MI355_Q4_1 || type == MI355_Q5_0 || type == MI355_Q5_1 || type == MI355_IQ4_NL || type == MI355_Q8_0;
    if (!typed || N <= 0 || K <= 0 || K % MMQ_BK != 0 || n_expert <= 0 || n_expert > 256) return 0;
    const row_layout L = make_row_layout(type, K);
    return layout_aligned(as, L) && (N * L.row_bytes) % 16 == 0 ? 1 : 0;
}

extern "C" int mi355_mul_mat_id_q(void *stream, int type, const void *as, const void *act, const int32_t *ids, int64_t ids_stride, float *dst, int64_t N,
                                  int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T, void *route_ws, size_t route_ws_bytes) {
    MI355_REQUIRE(mi355_mul_mat_id_q_supported(type, as, N, K, n_expert), "mul_mat_id_q: type %d, K=%lld, %lld experts or the weight alignment is not supported",
                  type, (long long)K, (long long)n_expert);
    MI355_REQUIRE(n_used > 0 && nb1 > 0 && T > 0 && ids_stride >= n_used, "mul_mat_id_q: bad shape");
    MI355_REQUIRE(T * n_used < (1 << 24) && nb1 * T < (1 << 24), "mul_mat_id_q: too many slots");
    MI355_REQUIRE(((uintptr_t)act & 15) == 0, "mul_mat_id_q: activation workspace is not 16-byte aligned");
    const size_t need = mi355_mul_mat_id_q8k_route_bytes(n_expert, n_used, T);
    if (route_ws == nullptr || route_ws_bytes < need || ((uintptr_t)route_ws & 15) != 0) {
        set_error("mul_mat_id_q: routing workspace of %zu bytes, need %zu (16-byte aligned)", route_ws_bytes, need);
        return MI355_ERR_WORKSPACE;
    }
    hipStream_t s = (hipStream_t)stream;
    const int64_t rows = nb1 * T;
    switch (type) {
        case MI355_Q4_0: launch_mmq_id<MI355_Q4_0>(s, as, act, rows, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, T, route_ws); break;
        case MI355_Q4_1: launch_mmq_id<MI355_Q4_1>(s, as, act, rows, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, T, route_ws); break;
        case MI355_Q5_0: launch_mmq_id<MI355_Q5_0>(s, as, act, rows, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, T, route_ws); break;
        case MI355_Q5_1: launch_mmq_id<MI355_Q5_1>(s, as, act, rows, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, T, route_ws); break;
        case MI355_IQ4_NL: launch_mmq_id<MI355_IQ4_NL>(s, as, act, rows, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, T, route_ws); break;
        default: launch_mmq_id<MI355_Q8_0>(s, as, act, rows, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, T, route_ws); break;
    }
    return launch_status("k_mmq (routed)");
}

extern "C" size_t mi355_mul_mat_q_ws_bytes(int64_t N, int64_t K, int64_t B) {
    if (N <= 0 || K <= 0 || B <= 0 || K % MMQ_BK != 0) return 0;
    const int n = mmq_slices(N, K, B);
    return n > 1 ? (size_t)n * (size_t)N * (size_t)B * sizeof(float) : 0;
}

extern "C" int mi355_mul_mat_q(void *stream, int type, const void *W, const void *act, float *dst, int64_t N, int64_t K,
                               int64_t B, int64_t dst_stride) {
    return mi355_mul_mat_q_ws(stream, type, W, act, dst, N, K, B, dst_stride, nullptr, 0);
}

extern "C" int mi355_mul_mat_q_ws(void *stream, int type, const void *W, const void *act, float *dst, int64_t N, int64_t K,
                                  int64_t B, int64_t dst_stride, void *ws, size_t ws_bytes) {
    MI355_REQUIRE(is_weight_type(type), "mul_mat_q: unsupported weight type %d", type);
    MI355_REQUIRE(N > 0 && K > 0 && B > 0, "mul_mat_q: bad shape N=%lld K=%lld B=%lld", (long long)N, (long long)K, (long long)B);
    MI355_REQUIRE(K % type_block_elems(type) == 0, "mul_mat_q: K=%lld is not a multiple of the block size", (long long)K);
    MI355_REQUIRE(dst_stride >= N, "mul_mat_q: dst_stride < N");
    const row_layout L = make_row_layout(type, K);
    if (!layout_aligned(W, L) || K % MMQ_BK != 0)   // tiny / odd shapes only
        return gemv_unaligned((hipStream_t)stream, type, W, act, dst, nullptr, N, K, B, dst_stride);
    MI355_REQUIRE(((uintptr_t)act & 15) == 0, "mul_mat_q: activation workspace is not 16-byte aligned");
    MI355_REQUIRE((N + MMQ_BM - 1) / MMQ_BM * ((B + 63) / 64) < (1 << 30), "mul_mat_q: too many tiles");
    hipStream_t s = (hipStream_t)stream;
    switch (type) {
        case MI355_Q4_0: launch_mmq_tn<MI355_Q4_0>(s, W, act, dst, N, K, B, dst_stride, ws, ws_bytes); break;
        case MI355_Q8_0: launch_mmq_tn<MI355_Q8_0>(s, W, act, dst, N, K, B, dst_stride, ws, ws_bytes); break;
        case MI355_Q4_K: launch_mmq_tn<MI355_Q4_K>(s, W, act, dst, N, K, B, dst_stride, ws, ws_bytes); break;
        case MI355_Q5_K: launch_mmq_tn<MI355_Q5_K>(s, W, act, dst, N, K, B, dst_stride, ws, ws_bytes); break;
        case MI355_Q4_1: launch_mmq_tn<MI355_Q4_1>(s, W, act, dst, N, K, B, dst_stride, ws, ws_bytes); break;
        case MI355_Q5_0: launch_mmq_tn<MI355_Q5_0>(s, W, act, dst, N, K, B, dst_stride, ws, ws_bytes); break;
        case MI355_Q5_1: launch_mmq_tn<MI355_Q5_1>(s, W, act, dst, N, K, B, dst_stride, ws, ws_bytes); break;
        case MI355_IQ4_NL: launch_mmq_tn<MI355_IQ4_NL>(s, W, act, dst, N, K, B, dst_stride, ws, ws_bytes); break;
        case MI355_IQ4_XS: launch_mmq_tn<MI355_IQ4_XS>(s, W, act, dst, N, K, B, dst_stride, ws, ws_bytes); break;
        default: launch_mmq_tn<MI355_Q6_K>(s, W, act, dst, N, K, B, dst_stride, ws, ws_bytes); break;
    }
    return launch_status("k_mmq");
}
