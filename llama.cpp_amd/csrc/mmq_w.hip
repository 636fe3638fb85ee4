// Wide-tile K-quant GEMM on the int8 matrix cores: 128 weight rows x 128 activation rows per 512-thread group, one group per
// compute unit, both operands streamed from pre-tiled images in HBM straight into LDS (no vector-ALU work on the way).
//
// Arithmetic is that of mmq_k.hip (ggml_vec_dot_q4_K_q8_K / ggml_vec_dot_q6_K_q8_K, ggml/src/ggml-cpu/ggml-cpu-quants.c:6817-6848,
// 8262-8283, on activations quantized by quantize_row_q8_K_ref, ggml/src/ggml-quants.c:2479-2516): the integer sub-scales are
// folded into two int8 operands per weight (value = R*hi + lo, R = 8 for Q4_K, 64 for Q6_K), v_mfma_i32_32x32x32_i8 sums whole
// super-blocks in int32, the Q4_K min term is one v_mfma_f32_32x32x16_f16 per super-block on exact small integers, and the
// vector ALU touches a result once per 256 elements.
//
// What differs is the data path and the schedule.  Measured on this part: about 52 bytes per clock and compute unit from L2 into LDS;
// one wave per SIMD issues a matrix instruction (32x32x32 i8) every 15.8 ns alone and every 18.2 / 23.7 / 30.5 ns with 4 / 8 / 12
// independent vector instructions behind each, two waves per SIMD every 14.6 / 15.2 / 19.2 / 23.3 ns: a wave overlaps its own
// vector and matrix instructions as long as both are there to issue, and two waves issue vector instructions at twice the rate of
// one (1.3-1.5 ns against 2.3-2.8 ns each).  Keeping one byte per Q4_K weight in LDS and multiplying by the sub-block scale on the
// way into the matrix instruction was measured 35 % slower than the two planes.
// A 128 x 256 tile (64 x 64 per wave: 0.75 KiB of operand reads per matrix instruction instead of 1, same arithmetic bit for bit) was
// built and measured on 14336 x 4096 at batch 512: Q6_K 76.8 us against 76-80 us here, Q4_K 99 us against 82-86 us.  At that wave
// tile the registers hold one set of integer sums, so a finished super-block is scaled in one burst at the start of the next; both
// waves of a SIMD reach it together and the matrix pipe waits (all 68.1 us, without the scaling 52.1, matrix instructions alone
// 41.5, empty loop 11.8).  The second set of sums below is what lets the scaling hide; it fits only at 32 x 64 per wave.
//  * Both operands live in HBM as *tile images* (tiles.hpp): tiles of 16 rows x 64 elements = 1 KiB, each byte for byte what
//    LDS holds, so one wave-wide global_load_lds moves a tile and nobody computes an address per element: 384 bytes from L2 per
//    matrix instruction where a 64 x 128 tile needs 512.
//  * K is walked in stages of 64 elements through a ring of four LDS buffers = one super-block; transfers run three stages
//    ahead of their use, one barrier per stage.  Every LDS read (operands, scales) is issued one 32-element step ahead of its use
//    and waited for once per step; the operand reads are inline assembly, because for reads it can see the compiler waits for
//    every transfer in flight whose target it cannot tell from the array being read.
//  * A wave owns 32 weight rows x 64 activation rows.  That leaves registers for a second set of integer accumulators: the sums
//    of super-block s are scaled into the f32 accumulators in eight pieces placed between the matrix instructions of
//    super-block s + 1, so the vector ALU of one wave works in the shadow of the other wave's matrix instructions.
//
// MFMA operand mapping (A = activations, B = weights, D[i][j]): lane l supplies row l % 32 and k bytes [16*(l/32), +16)
// (f16: k slots [8*(l/32), +8)); D register r of lane l is i = 8*(r/4) + 4*(l/32) + r%4, j = l % 32.
#include "common.hpp"
#include "norm_quant.hpp"
#include "q8k.hpp"
#include "qdot.hpp"
#include "tiles.hpp"

#include <type_traits>

namespace mi355 {

// unpack one 16-byte piece of packed weights into its two planes (same arithmetic as k_unpack_planes of mmq_k.hip) and store
// the chunks into the tile images; one thread per piece: row, super-block, half, piece
typedef unsigned short wt_u16x2 __attribute__((ext_vector_type(2)));
typedef short wt_i16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32 wt_mul_bytes(u32 x, u32 f) {
    const wt_u16x2 v = __builtin_bit_cast(wt_u16x2, x);
    const wt_u16x2 m = {(unsigned short)f, (unsigned short)f};
    const wt_u16x2 p = v * m;
    return __builtin_bit_cast(u32, p);
}
__device__ __forceinline__ void wt_q6k_planes(u32 a, int sc, u32 &hi, u32 &lo) {
    const wt_i16x2 s = {(short)sc, (short)sc};
    const wt_i16x2 off = {(short)(-32 * sc), (short)(-32 * sc)};
    const wt_i16x2 e = __builtin_bit_cast(wt_i16x2, a & 0x00FF00FFu);
    const wt_i16x2 o = __builtin_bit_cast(wt_i16x2, (a >> 8) & 0x00FF00FFu);
    const wt_i16x2 pe = e * s + off, po = o * s + off;
    const wt_i16x2 six = {6, 6};
    const u32 he = __builtin_bit_cast(u32, pe >> six), ho = __builtin_bit_cast(u32, po >> six);
    const u32 le = __builtin_bit_cast(u32, pe) & 0x003F003Fu, lo_ = __builtin_bit_cast(u32, po) & 0x003F003Fu;
    hi = (he & 0x00FF00FFu) | ((ho & 0x00FF00FFu) << 8);
    lo = le | (lo_ << 8);
}

// IQ4_XS: the four table values (int8) in the bytes of `a` times the block scale -32..31 -> P = 64 * hi + lo, hi -64..63, lo 0..63:
// the Q6_K form
__device__ __forceinline__ void wt_iq4xs_planes(u32 a, int sc, u32 &hi, u32 &lo) {
    const wt_i16x2 s = {(short)sc, (short)sc};
    const wt_i16x2 eight = {8, 8}, six = {6, 6};
    const wt_i16x2 e = (__builtin_bit_cast(wt_i16x2, a << 8) & (wt_i16x2){(short)0xFF00, (short)0xFF00}) >> eight;   // sign-extended even bytes
    const wt_i16x2 o = (__builtin_bit_cast(wt_i16x2, a) & (wt_i16x2){(short)0xFF00, (short)0xFF00}) >> eight;        // ... odd bytes
    const wt_i16x2 pe = e * s, po = o * s;
    const u32 he = __builtin_bit_cast(u32, pe >> six), ho = __builtin_bit_cast(u32, po >> six);
    const u32 le = __builtin_bit_cast(u32, pe) & 0x003F003Fu, lo_ = __builtin_bit_cast(u32, po) & 0x003F003Fu;
    hi = (he & 0x00FF00FFu) | ((ho & 0x00FF00FFu) << 8);
    lo = le | (lo_ << 8);
}

// Q5_K: the four levels 0..31 in the bytes of `a` times the sub-block scale 0..63 -> P = 16 * hi + lo with hi <= 122, lo <= 15
__device__ __forceinline__ void wt_q5k_planes(u32 a, int sc, u32 &hi, u32 &lo) {
    const wt_u16x2 s = {(unsigned short)sc, (unsigned short)sc};
    const wt_u16x2 e = __builtin_bit_cast(wt_u16x2, a & 0x00FF00FFu);
    const wt_u16x2 o = __builtin_bit_cast(wt_u16x2, (a >> 8) & 0x00FF00FFu);
    const wt_u16x2 pe = e * s, po = o * s;
    const wt_u16x2 four = {4, 4};
    const u32 he = __builtin_bit_cast(u32, pe >> four), ho = __builtin_bit_cast(u32, po >> four);
    const u32 le = __builtin_bit_cast(u32, pe) & 0x000F000Fu, lo_ = __builtin_bit_cast(u32, po) & 0x000F000Fu;
    hi = (he & 0x00FF00FFu) | ((ho & 0x00FF00FFu) << 8);
    lo = le | (lo_ << 8);
}

// weight types with tile images: the K-quants of the Q4_K form (minima, radix 8 / 16) and those of the Q6_K form (signed levels
// times signed scales, radix 64, no minima: Q6_K and IQ4_XS)
static bool wt_has_images(int type) { return type == MI355_Q4_K || type == MI355_Q5_K || type == MI355_Q6_K || type == MI355_IQ4_XS; }

template <int TYPE>
__global__ void __launch_bounds__(256) k_unpack_tiles(const uint8_t *__restrict__ W, int8_t *__restrict__ img, int64_t N, int64_t K, row_layout L) {
    const int64_t per_row = (K >> 8) * 8;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t n16 = (N + 15) & ~(int64_t)15;
    if (idx >= n16 * per_row) return;
    const int64_t row = idx / per_row, rem = idx % per_row, sb = rem >> 3;
    const int half = (int)((rem >> 2) & 1), p = (int)(rem & 3);
    uint8_t *aux = (uint8_t *)img + wt_w_aux_offset(N, K);
    const int64_t n_rb_pad = wt_rb_pad(N);
    constexpr int W_AUX = wt_w_aux_bytes(TYPE);
    const bool live = row < N;   // rows that pad the last 16-row block hold zeros
    const uint8_t *wrow = W + (live ? row : 0) * L.row_bytes;
    const int64_t k0 = sb * QKK + half * 128;
    int8_t *hi_img = img, *lo_img = img + n16 * K;
    u32x4 a1 = {0, 0, 0, 0}, a0 = a1, b1 = a1, b0 = a1;
    int c0, c1;   // 16-byte chunk index inside the 128-element half
    if constexpr (TYPE == MI355_Q4_K) {
        const uint8_t *blk = wrow + sb * Q4_K_BYTES;
        const u32x4 q = load16(blk + 16 + (half * 2 + (p >> 1)) * 32 + (p & 1) * 16);
        const u32x4 hdr = load16(blk);
        const int gl = p >> 1;
        int scl, mnl, sch, mnh;
        q4k_scale_min(hdr[1], hdr[2], hdr[3], half * 4 + 2 * gl, scl, mnl);
        q4k_scale_min(hdr[1], hdr[2], hdr[3], half * 4 + 2 * gl + 1, sch, mnh);
        if (live) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const u32 nl = q[i] & 0x0F0F0F0Fu, nh = (q[i] >> 4) & 0x0F0F0F0Fu;
                a1[i] = wt_mul_bytes(nl, (u32)scl >> 3);
                a0[i] = wt_mul_bytes(nl, (u32)scl & 7u);
                b1[i] = wt_mul_bytes(nh, (u32)sch >> 3);
                b0[i] = wt_mul_bytes(nh, (u32)sch & 7u);
            }
        }
        c0 = 4 * gl + (p & 1);
        c1 = c0 + 2;
        if (half == 0 && p == 0) {
            uint8_t *e = aux + (sb * n_rb_pad + (row >> 4)) * W_AUX;
            const int r = (int)(row & 15);
            f16x8 m1, m64;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                int sc, mn;
                q4k_scale_min(hdr[1], hdr[2], hdr[3], j, sc, mn);
                if (!live) mn = 0;
                m1[j] = (_Float16)(float)mn;
                m64[j] = (_Float16)(float)(64 * mn);
            }
            *(f16x8 *)(e + r * 32) = m1;
            *(f16x8 *)(e + r * 32 + 16) = m64;
            *(float *)(e + 512 + r * 4) = live ? half_bits_to_float((unsigned short)(hdr[0] & 0xFFFFu)) : 0.0f;
            *(float *)(e + 576 + r * 4) = live ? half_bits_to_float((unsigned short)(hdr[0] >> 16)) : 0.0f;
        }
    } else if constexpr (TYPE == MI355_Q5_K) {
        // the Q4_K geometry (block_q5_K, ggml/src/ggml-common.h:296-308: header, qh[32] at 16, qs[128] at 48); the fifth bit of sub-block j
        // is bit j of qh[l]; planes at radix 16
        const uint8_t *blk = wrow + sb * Q5_K_BYTES;
        const u32x4 q = load16(blk + 48 + (half * 2 + (p >> 1)) * 32 + (p & 1) * 16);
        const u32x4 qh = load16(blk + 16 + (p & 1) * 16);
        const u32x4 hdr = load16(blk);
        const int gl = p >> 1, g = half * 2 + gl;
        int scl, mnl, sch, mnh;
        q4k_scale_min(hdr[1], hdr[2], hdr[3], 2 * g, scl, mnl);
        q4k_scale_min(hdr[1], hdr[2], hdr[3], 2 * g + 1, sch, mnh);
        if (live) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const u32 nl = (q[i] & 0x0F0F0F0Fu) | (((qh[i] >> (2 * g)) & 0x01010101u) << 4);
                const u32 nh = ((q[i] >> 4) & 0x0F0F0F0Fu) | (((qh[i] >> (2 * g + 1)) & 0x01010101u) << 4);
                u32 hi, lo;
                wt_q5k_planes(nl, scl, hi, lo);
                a1[i] = hi; a0[i] = lo;
                wt_q5k_planes(nh, sch, hi, lo);
                b1[i] = hi; b0[i] = lo;
            }
        }
        c0 = 4 * gl + (p & 1);
        c1 = c0 + 2;
        if (half == 0 && p == 0) {
            uint8_t *e = aux + (sb * n_rb_pad + (row >> 4)) * W_AUX;
            const int r = (int)(row & 15);
            f16x8 m1, m64;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                int sc, mn;
                q4k_scale_min(hdr[1], hdr[2], hdr[3], j, sc, mn);
                if (!live) mn = 0;
                m1[j] = (_Float16)(float)mn;
                m64[j] = (_Float16)(float)(64 * mn);
            }
            *(f16x8 *)(e + r * 32) = m1;
            *(f16x8 *)(e + r * 32 + 16) = m64;
            *(float *)(e + 512 + r * 4) = live ? half_bits_to_float((unsigned short)(hdr[0] & 0xFFFFu)) : 0.0f;
            *(float *)(e + 576 + r * 4) = live ? half_bits_to_float((unsigned short)(hdr[0] >> 16)) : 0.0f;
        }
    } else if constexpr (TYPE == MI355_IQ4_XS) {
        // block ib = 4 half + p of the super-block (block_iq4_xs, ggml/src/ggml-common.h:406-412): byte l of its 16 holds the table
        // index of element l in the low nibble and of element 16 + l in the high one; value = d * (ls - 32) * table[index]
        const int ib = half * 4 + p;
        const u32x4 q = load16(wrow + sb * 128 + ib * 16);
        const uint2 h = *(const uint2 *)(wrow + L.off_b + sb * 8);
        const int ls = (int)(((h.y >> (4 * ib)) & 0xFu) | (((h.x >> (16 + 2 * ib)) & 3u) << 4)) - 32;
        if (live) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                u32 hi, lo;
                wt_iq4xs_planes(iq4nl_lookup4(q[i] & 0x0F0F0F0Fu), ls, hi, lo);
                a1[i] = hi; a0[i] = lo;
                wt_iq4xs_planes(iq4nl_lookup4((q[i] >> 4) & 0x0F0F0F0Fu), ls, hi, lo);
                b1[i] = hi; b0[i] = lo;
            }
        }
        c0 = 2 * p;
        c1 = c0 + 1;
        if (half == 0 && p == 0) {   // the Q4_K entry with no minima
            uint8_t *e = aux + (sb * n_rb_pad + (row >> 4)) * W_AUX;
            const int r = (int)(row & 15);
            const u32x4 z = {0, 0, 0, 0};
            *(u32x4 *)(e + r * 32) = z;
            *(u32x4 *)(e + r * 32 + 16) = z;
            *(float *)(e + 512 + r * 4) = live ? half_bits_to_float((unsigned short)(h.x & 0xFFFFu)) : 0.0f;
            *(float *)(e + 576 + r * 4) = 0.0f;
        }
    } else {
        const int l0 = 16 * (p & 1), qa = p >> 1;
        const u32x4 ql = load16(wrow + sb * 128 + half * 64 + p * 16);
        const u32x4 qh = load16(wrow + L.off_b + sb * 64 + half * 32 + l0);
        const int8_t *sc = (const int8_t *)(wrow + L.off_c + sb * 16 + half * 8 + (l0 >> 4));
        const int scA = sc[2 * qa], scB = sc[2 * qa + 4];
        if (live) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const u32 va = (ql[i] & 0x0F0F0F0Fu) | (((qh[i] >> (2 * qa)) & 0x03030303u) << 4);
                const u32 vb = ((ql[i] >> 4) & 0x0F0F0F0Fu) | (((qh[i] >> (2 * qa + 4)) & 0x03030303u) << 4);
                u32 hi, lo;
                wt_q6k_planes(va, scA, hi, lo);
                a1[i] = hi; a0[i] = lo;
                wt_q6k_planes(vb, scB, hi, lo);
                b1[i] = hi; b0[i] = lo;
            }
        }
        c0 = 2 * qa + (p & 1);
        c1 = c0 + 4;
        if (half == 0 && p == 0) {   // the Q4_K entry with no minima
            uint8_t *e = aux + (sb * n_rb_pad + (row >> 4)) * W_AUX;
            const int r = (int)(row & 15);
            const u32x4 z = {0, 0, 0, 0};
            *(u32x4 *)(e + r * 32) = z;
            *(u32x4 *)(e + r * 32 + 16) = z;
            *(float *)(e + 512 + r * 4) = live ? half_bits_to_float(*(const unsigned short *)(wrow + L.off_d + sb * 2)) : 0.0f;
            *(float *)(e + 576 + r * 4) = 0.0f;
        }
    }
    *(u32x4 *)(hi_img + wt_tile_off(row, k0 + c0 * 16, K)) = a1;
    *(u32x4 *)(lo_img + wt_tile_off(row, k0 + c0 * 16, K)) = a0;
    *(u32x4 *)(hi_img + wt_tile_off(row, k0 + c1 * 16, K)) = b1;
    *(u32x4 *)(lo_img + wt_tile_off(row, k0 + c1 * 16, K)) = b0;
}

// One wave per (row, super-block); 4 super-blocks per group.  Rows that pad the last 16-row block get zeros.
__global__ void __launch_bounds__(256) k_quantize_q8k_tiled(const float *__restrict__ x, uint8_t *__restrict__ act, int64_t K, int64_t B, int64_t x_stride) {
    const int lane = threadIdx.x & 63;
    const int64_t sb = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t row = blockIdx.y;
    if (sb >= (K >> 8)) return;   // whole wave
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (row < B) v = *(const f32x4 *)(x + row * x_stride + sb * QKK + lane * 4);
    q8k_quantize_wave_tiled(v, lane, act, K, B, row, sb);
}

constexpr int WT_BM = 128, WT_BN = 128;

// MUL_MAT_ID on tile images: column tile ct of the sorted slot list (at most 128 slots of one expert) owns rows
// [128 ct, 128 ct + 128) of the activation image; rows past the tile's slots are zeros.
struct wt_route {
    const int32_t *dst_row;
    const int32_t *tiles;
    const int32_t *n_tiles;
    int64_t expert_img_bytes;   // from one expert's weight images to the next
};
__global__ void __launch_bounds__(256) k_quantize_q8k_tiled_routed(const float *__restrict__ x, uint8_t *__restrict__ act, int64_t K, int64_t B_img, int64_t x_stride,
                                                                   const int32_t *__restrict__ act_row, const int32_t *__restrict__ tiles,
                                                                   const int32_t *__restrict__ n_tiles) {
    const int lane = threadIdx.x & 63;
    const int64_t sb = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t row = blockIdx.y;
    if (sb >= (K >> 8)) return;   // whole wave
    const int ct = (int)(row / WT_BN);
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (ct < *n_tiles) {
        const int c = tiles[4 * ct + 1] + (int)(row % WT_BN);
        if (c < tiles[4 * ct + 2]) v = *(const f32x4 *)(x + (int64_t)act_row[c] * x_stride + sb * QKK + lane * 4);
    }
    q8k_quantize_wave_tiled(v, lane, act, K, B_img, row, sb);
}
constexpr int WT_A_AUX_TILE = (WT_BN / 16) * WT_A_AUX;       // 4608 bytes of activation scales per tile and super-block

// s_waitcnt that waits until at most n vector-memory operations of this wave are outstanding (nothing else)
#define WT_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (7 << 4) | (0xF << 8))

// One launch: up to three matrices of one type that share the activation.  Their tiles are numbered one matrix after the other,
// row tile by row tile, so that together they fill rounds of groups that each matrix alone would leave partly empty (gate + up at
// batch 512: 2 x 448 tiles = 3.5 rounds on 256 compute units instead of 2 x 2).  Cutting the last, partly empty round's tiles
// along K so that short groups fill it was measured and dropped: 162 us against 160 us uncut for gate + up - with half of the
// compute units idle the others run faster, so the uncut tail costs less than its group count suggests.
// gridDim.y > 1 cuts every tile into gridDim.y slices (single matrices with few tiles; partial sums in dst, one N x B slab per
// slice, added by k_wt_split_sum).
struct wt_mat {
    const int8_t *w_img;
    float *dst;
    const float *residual;   // may be null; same shape and stride as dst; may be dst itself
    int64_t N, dst_stride;
    int first_tile;          // index of this matrix's first tile in the launch (unused entries: INT_MAX)
    int shift;               // log2 of the radix between the matrix's two planes: 3 Q4_K, 4 Q5_K, 6 Q6_K
    int epi;                 // EPI launches: WT_EPI_*
    int64_t nb1, nb2;        // WT_EPI_*CACHE: dst = base of an f16 cache; byte strides of a cell and of a head inside it
};
// EPI launches (Q, K and V of a prompt batch): what becomes of a finished sum.  The rotation is ROPE in its adjacent-pair mode, the
// pair (2 p, 2 p + 1) of a head being two neighbouring rows of the matrix, i.e. two neighbouring lanes.
enum { WT_EPI_ROPE = 1, WT_EPI_ROPE_CACHE = 2, WT_EPI_CACHE = 3 };   // rotate -> f32 dst | rotate -> f16 cache | f16 cache
struct wt_rope {
    const float2 *cs;        // [B][D / 2] {cos, sin} of the rotation of pair p at token b's position (k_rope_table)
    const int32_t *cells;    // [B] cache cell of token b
    int D, n_dims;           // head size; elements of a head that are rotated
};
struct wt_launch {
    wt_mat m[3];
    int n_col_tiles;
    int n_tiles, n_tiles_padded;   // n_tiles_padded: rounded up to a multiple of 8
    wt_rope rope;
};

// ID: MUL_MAT_ID.  The "matrix" is expert 0's images, the column tiles are those of the sorted slot list (rt), B the rows of the
// activation image (128 per column tile); a tile's rows go to the dst rows of its slots.
// TYPE: MI355_Q4_K = the form with the min term, the radix between the planes taken from the matrix (Q4_K, Q5_K, and Q6_K images,
// whose minima are zeros, in a launch they share with the other two); MI355_Q6_K = launches of Q6_K matrices only: no min term.
template <int TYPE, bool ID = false, bool EPI = false>
__global__ void __launch_bounds__(512, 1) k_mmq_w(wt_launch P, const int8_t *__restrict__ a_img, int64_t K, int64_t B, wt_route rt) {
    static_assert(TYPE == MI355_Q4_K || TYPE == MI355_Q6_K, "two forms");
    static_assert(!(ID && EPI), "one or the other");
    constexpr bool Q4 = TYPE == MI355_Q4_K;   // sub-block mins: the min term and its scale records
    constexpr int NP = 2;                                                      // weight planes
    constexpr int W_AUX = wt_w_aux_bytes(TYPE);
    constexpr int STAGE = (NP * WT_BM + WT_BN) * 64;                           // bytes of one 64-element stage: plane(s), activations
    constexpr int OFF_LO = WT_BM * 64, OFF_A = NP * WT_BM * 64;
    constexpr int DPS = NP + 1;                                                // transfers per wave and stage
    constexpr int N_A_CHUNKS = (WT_A_AUX_TILE + 1023) / 1024;                  // 5, the last one half full
    constexpr int N_W_CHUNKS = (WT_BM / 16) * W_AUX / 1024;                    // 5
    constexpr int N_CHUNKS = N_A_CHUNKS + N_W_CHUNKS;                          // scale transfers per super-block
    constexpr int AUX_W_OFF = N_A_CHUNKS * 1024;                               // weight entries behind the (padded) activation entries
    // Ring of stage buffers: 8 (two super-blocks) where they fit, else 4; a stage's transfers are issued DIST stages ahead.
    // The operand reads from the ring are inline assembly with waits placed by hand: for accesses it can see, the compiler
    // waits for every transfer in flight whose target it cannot tell from the array being read, and it tells nothing apart
    // inside one array and at most eight arrays in all.
    constexpr int NBUF = 4, DIST = NBUF - 1;
    __shared__ __attribute__((aligned(1024))) int8_t ring_buf[NBUF * STAGE];
    __shared__ __attribute__((aligned(1024))) uint8_t aux0[AUX_W_OFF + 5 * 1024], aux1[AUX_W_OFF + 5 * 1024];   // scale entries of a super-block
    // The buffers are written by global-to-LDS transfers only; the empty asm makes them memory that unknown code may have written.
    asm volatile("" ::"v"((void *)ring_buf), "v"((void *)aux0), "v"((void *)aux1) : "memory");
    auto ring = [&](int i) -> int8_t * { return ring_buf + (i & (NBUF - 1)) * STAGE; };

    // groups of one XCD (every eighth group index) take consecutive tiles: the column tiles of a weight row tile meet in one L2
    const int tile = (int)(blockIdx.x & 7) * (P.n_tiles_padded >> 3) + (int)(blockIdx.x >> 3);
    if (tile >= P.n_tiles) return;
    const int mi = (tile >= P.m[1].first_tile ? 1 : 0) + (tile >= P.m[2].first_tile ? 1 : 0);
    const int8_t *__restrict__ w_img = P.m[mi].w_img;
    float *dst = P.m[mi].dst;
    const float *residual = P.m[mi].residual;
    const int64_t N = P.m[mi].N;
    const int64_t dst_stride = P.m[mi].dst_stride;
    const int radix_shift = Q4 ? __builtin_amdgcn_readfirstlane(P.m[mi].shift) : 6;
    const int n_col_tiles = P.n_col_tiles;
    const int ltile = tile - P.m[mi].first_tile;
    const int64_t row0 = (int64_t)(ltile / n_col_tiles) * WT_BM;
    const int64_t col0 = (int64_t)(ltile % n_col_tiles) * WT_BN;
    int slot_first = 0, slot_end = 0;   // ID: the tile's columns of the sorted slot list
    if constexpr (ID) {
        const int ct = ltile % n_col_tiles;
        if (ct >= *rt.n_tiles) return;   // the whole group
        w_img += (int64_t)rt.tiles[4 * ct] * rt.expert_img_bytes;
        slot_first = rt.tiles[4 * ct + 1];
        slot_end = rt.tiles[4 * ct + 2];
    }

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lhi = lane >> 5;
    const int wrow0 = (wave & 3) * 32;    // weight rows of this wave inside the tile
    const int wcol0 = (wave >> 2) * 64;   // activation rows of this wave inside the tile
    const int64_t nsb = K >> 8, nkb = K >> 6;
    // split K: group y of gridDim.y walks super-blocks [sb_lo, sb_hi) and writes its sums to its own slice of `dst`
    const int64_t sb_per = (nsb + gridDim.y - 1) / gridDim.y;
    const int64_t sb_lo = (int64_t)blockIdx.y * sb_per, sb_hi = sb_lo + sb_per < nsb ? sb_lo + sb_per : nsb;
    // where the sums go: element (b, n) of the product at out[(b - col0) * dst_stride + (n - row0)]
    float *out = dst + col0 * dst_stride + row0;
    if (residual) residual += col0 * dst_stride + row0;
    if (gridDim.y > 1) {
        out += (int64_t)blockIdx.y * B * dst_stride;
        residual = nullptr;
    }

    // ---- sources of this wave's transfers per stage: one tile of each weight plane and one activation tile
    const int64_t n16 = (N + 15) & ~(int64_t)15, b16 = (B + 15) & ~(int64_t)15;
    const int64_t n_rb = n16 >> 4, n_cb = b16 >> 4;
    const int64_t n_rb_pad = wt_rb_pad(N), n_cb_pad = wt_cb_pad(B);
    const int64_t rb0 = row0 >> 4, cb0 = col0 >> 4;
    const int64_t rbw = rb0 + wave < n_rb ? rb0 + wave : n_rb - 1;
    const int64_t cba = cb0 + wave < n_cb ? cb0 + wave : n_cb - 1;
    // wave-uniform bases; the lane's 16 bytes are added at the transfer
    const unsigned lane16 = (unsigned)lane * 16u;
    const int8_t *src_w = w_img + rbw * nkb * WT_TILE;
    const int8_t *src_a = a_img + cba * nkb * WT_TILE;
    const uint8_t *w_aux = (const uint8_t *)w_img + wt_w_aux_offset(N, K) + rb0 * W_AUX;
    const uint8_t *a_aux = (const uint8_t *)a_img + b16 * K + cb0 * WT_A_AUX;
    // aux chunks 2*wave and 2*wave + 1 of the super-block's N_CHUNKS (those past the end repeat the last one)
    const int ch0 = 2 * wave < N_CHUNKS ? 2 * wave : N_CHUNKS - 1, ch1 = 2 * wave + 1 < N_CHUNKS ? 2 * wave + 1 : N_CHUNKS - 1;

    auto dma = [&](const void *g, void *l) {   // g: wave-uniform
        // scalar base + 32-bit lane offset; the empty asm keeps the sum from being formed once per lane ahead of the loop, which
        // would cost two registers per source
        unsigned off = lane16;
        asm volatile("" : "+v"(off));
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)((const char *)g + off),
                                         (void __attribute__((address_space(3))) *)l, 16, 0, 0);
    };
    auto dma_stage = [&](int64_t kb, int8_t *buf) {   // kb: absolute 64-element block
        const int64_t o = kb * WT_TILE;
        dma(src_w + o, buf + wave * WT_TILE);
        dma(src_w + n16 * K + o, buf + OFF_LO + wave * WT_TILE);
        dma(src_a + o, buf + OFF_A + wave * WT_TILE);
    };
    // Scale entries of super-block sb into `buf`.  The activation entries of a tile end in the middle of their last chunk: what
    // follows them in memory comes along and is never read.
    auto dma_aux_chunk = [&](int64_t sb, int ch, uint8_t *buf) {
        const uint8_t *src = ch < N_A_CHUNKS ? a_aux + sb * n_cb_pad * WT_A_AUX + ch * 1024 : w_aux + sb * n_rb_pad * W_AUX + (ch - N_A_CHUNKS) * 1024;
        dma(src, buf + ch * 1024);
    };
    auto dma_aux = [&](int64_t sb, uint8_t *buf) {
        dma_aux_chunk(sb, ch0, buf);
        dma_aux_chunk(sb, ch1, buf);
    };

    // ---- per-lane LDS offsets of the operand reads: row l32 of a 32-row tile, logical chunk 2*ks + lhi of the stage
    int foff[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++) foff[ks] = (l32 >> 4) * WT_TILE + (l32 & 15) * 64 + (((2 * ks + lhi) ^ ((l32 >> 2) & 3)) << 4);
    const int a_base = OFF_A + (wcol0 >> 4) * WT_TILE, w_base = (wrow0 >> 4) * WT_TILE;
    // scale entries of this lane's weight row and of the activation row it feeds to the min-term matrix instruction
    const int we_off = AUX_W_OFF + ((wrow0 >> 4) + (l32 >> 4)) * W_AUX;
    const int ae_off = (wcol0 >> 4) * WT_A_AUX;
    // Offset of the activation sub-block sums this lane feeds to the min-term matrix instruction (tile 0; tile 1 is two entries on).
    // The empty asm hides how it is made up: split into a chain of pointer increments by the optimizer, the access loses the
    // compiler's knowledge of which LDS array it reads, and every such read would then wait for all transfers in flight.
    int am_off = ae_off + (l32 >> 4) * WT_A_AUX + 64 + (l32 & 15) * 32 + lhi * 16;
    asm volatile("" : "+v"(am_off));

    f32x16 acc[2];
#pragma unroll
    for (int tb = 0; tb < 2; tb++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[tb][r] = 0.0f;
    i32x16 hiX[2], loX[2], hiY[2], loY[2];   // integer sums of the even / odd super-blocks of the slice

    // One eighth of the scaling of a finished super-block: registers 4*q .. 4*q+3 of tile tb.  M: the min term of the tile.
    // activation scales of registers 4*q .. 4*q+3 of tile tb
    auto load_d8 = [&](const uint8_t *ax, int tb, int q) {
        return *(const f32x4 *)(ax + (ae_off + (2 * tb + (q >> 1)) * WT_A_AUX + (8 * (q & 1) + 4 * lhi) * 4));
    };
    auto scale_piece = [&](const f32x4 &d8, const i32x16 &h, const i32x16 &l, const f32x16 &M, float dw, float dn, int tb, int q) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int r = 4 * q + i;
            const float f = (float)((h[r] << radix_shift) + l[r]);
            if constexpr (Q4) acc[tb][r] = __builtin_fmaf(d8[i], __builtin_fmaf(-dn, M[r], mul_rn(dw, f)), acc[tb][r]);
            else acc[tb][r] = __builtin_fmaf(d8[i], mul_rn(dw, f), acc[tb][r]);
        }
    };
    // operands of the min-term matrix instruction: sub-block sums of tile tb's activation rows / mins of the weight rows
    auto load_am = [&](const uint8_t *ax, int tb) { return *(const f16x8 *)(ax + (am_off + tb * 2 * WT_A_AUX)); };
    auto load_bm = [&](const uint8_t *ax) { return *(const f16x8 *)(ax + (we_off + (l32 & 15) * 32 + lhi * 16)); };
    auto min_term = [&](const f16x8 &am, const f16x8 &bm) {
        f32x16 z;
#pragma unroll
        for (int r = 0; r < 16; r++) z[r] = 0.0f;
        if constexpr (Q4) return __builtin_amdgcn_mfma_f32_32x32x16_f16(am, bm, z, 0, 0, 0);
        else return z;
    };
    // operand registers of one 32-element step: two activation tiles, both planes of the weight tile
    struct frags { i32x4 a[2], w[2]; };
    // LDS byte addresses of this lane's reads in ring position 0 (activation / weight tile, first / second step of a stage); the
    // second pair is 64 KiB on, for the ring positions an instruction's 16-bit offset does not reach from the first
    const unsigned ring_addr = (unsigned)(size_t)(__attribute__((address_space(3))) int8_t *)ring_buf;
    unsigned fa[2][2], fw[2][2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
            fa[h][ks] = ring_addr + (unsigned)(a_base + foff[ks]) + h * 65536u;
            fw[h][ks] = ring_addr + (unsigned)(w_base + foff[ks]) + h * 65536u;
        }
#define WT_DS_READ(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(off))
    // rs: ring position (compile-time constant after unrolling).  The values are valid after frags_wait.
    auto load_frags = [&](frags &F, int rs, int ks) {
        const int o = (rs & (NBUF - 1)) * STAGE, h = o >> 16, ol = o & 65535;
        // every offset below must fit 16 bits: a stage never straddles a 64 KiB boundary (STAGE divides 64 KiB or ol + STAGE <= 64 KiB)
        if (h == 0) {
            WT_DS_READ(F.a[0], fa[0][ks], ol);
            WT_DS_READ(F.a[1], fa[0][ks], ol + 2 * WT_TILE);
            WT_DS_READ(F.w[0], fw[0][ks], ol);
            WT_DS_READ(F.w[1], fw[0][ks], ol + OFF_LO);
        } else {
            WT_DS_READ(F.a[0], fa[1][ks], ol);
            WT_DS_READ(F.a[1], fa[1][ks], ol + 2 * WT_TILE);
            WT_DS_READ(F.w[0], fw[1][ks], ol);
            WT_DS_READ(F.w[1], fw[1][ks], ol + OFF_LO);
        }
    };
    // all LDS reads of this wave have returned; the registers pass through the statement so that their users stay behind it
    auto frags_wait = [&](frags &F) {
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(F.a[0]), "+v"(F.a[1]), "+v"(F.w[0]), "+v"(F.w[1]));
    };

    // ---- prologue: scales of the first super-block, stages 0..2 of the slice
    const int64_t kb_lo = sb_lo * 4, kb_last = sb_hi * 4 - 1;
    auto clamp_kb = [&](int64_t kb) { return kb < kb_last ? kb : kb_last; };
#pragma unroll
    for (int i = 0; i < DIST; i++) dma_stage(clamp_kb(kb_lo + i), ring(i));
    WT_WAIT_VM((DIST - 1) * DPS);
    __builtin_amdgcn_s_barrier();
    frags F0, F1;   // steps with even / odd index
    load_frags(F0, 0, 0);

    // Scale data of the super-block whose sums are being scaled, read from LDS one step ahead of their use.
    f32x4 e_d8 = {0.f, 0.f, 0.f, 0.f};                  // activation scales of the next piece
    f16x8 e_am = {0, 0, 0, 0, 0, 0, 0, 0}, e_bm = e_am;   // min-term operands: next tile's sub-block sums, the weight rows' mins
    float e_dw = 0.0f, e_dn = 0.0f;                     // d and dmin of this lane's weight row
    f32x16 e_M;                                         // min term of the tile whose pieces come next
#pragma unroll
    for (int r = 0; r < 16; r++) e_M[r] = 0.0f;

    // One super-block.  ODD: parity of its position in the slice (picks accumulator set and scale buffers at compile time);
    // PREV: the super-block before it exists and is scaled between this one's matrix instructions.
    // A step first waits for the LDS reads issued during the step before (its operands and scales), then issues the reads of
    // the step after it, then computes: no read is waited for right after its issue.
    auto super_block = [&](auto odd_c, auto prev_c, const int64_t sb) {
        constexpr bool ODD = decltype(odd_c)::value, PREV = decltype(prev_c)::value;
        i32x16(&hi)[2] = ODD ? hiY : hiX;
        i32x16(&lo)[2] = ODD ? loY : loX;
        const i32x16(&phi)[2] = ODD ? hiX : hiY;
        const i32x16(&plo)[2] = ODD ? loX : loY;
        uint8_t *ax_cur = ODD ? aux1 : aux0;           // receives this super-block's scale entries
        const uint8_t *ax_prev = ODD ? aux0 : aux1;    // holds the previous super-block's
        float dw = e_dw, dn = e_dn;
        f16x8 bm = e_bm;
#pragma unroll
        for (int piece = 0; piece < 8; piece++) {
            const int st = piece >> 1, ks = piece & 1;
            const int rs = (ODD ? 4 : 0) + st;              // position of this stage in the ring (the slice starts at 0)
            int8_t *nxt = ring(rs + DIST);                  // buffer of the stage DIST ahead = of the stage before this one
            frags &F = ks == 0 ? F0 : F1;
            frags &Fn = ks == 0 ? F1 : F0;
            const f32x4 d8 = e_d8;
            const f16x8 am = e_am;
            frags_wait(F);   // all LDS reads of this wave have returned
            if (ks == 0) {
                // scale entries first: they are then complete a stage earlier
                if (st == 0) dma_aux(sb, ax_cur);
                dma_stage(clamp_kb(sb * 4 + st + DIST), nxt);
                load_frags(Fn, rs, 1);
            } else {
                // The next stage's transfers must have landed, and every wave must be done reading this stage, whose buffer the
                // next transfers overwrite.  Issued since the next stage's: DIST - 1 stages and the scale entries (2 transfers,
                // ahead of the first stage's) of every super-block that began among them; the first super-block of a slice has
                // no predecessor that issued any.
                // (super-block starts among stages s - DIST + 2 .. s, s = this stage)
                if (st < 2) WT_WAIT_VM((DIST - 1) * DPS + 2);
                else WT_WAIT_VM((DIST - 1) * DPS);   // the scale entries are complete from here on: they are read at the end of the super-block
                __builtin_amdgcn_s_barrier();
                load_frags(Fn, rs + 1, 0);
            }
            // scale data of the next step; the min-term operands one step earlier still, so that the min term of a tile is issued
            // at the end of the step before the tile's first piece and has left the matrix pipe when that piece reads it
            if (piece == 7) e_d8 = load_d8(ax_cur, 0, 0);   // the next super-block scales this one's sums
            else if (PREV) e_d8 = load_d8(ax_prev, (piece + 1) >> 2, (piece + 1) & 3);
            if (piece == 6) {   // this super-block's entries are complete since the barrier of the stage before
                if constexpr (Q4) {
                    e_am = load_am(ax_cur, 0);
                    e_bm = load_bm(ax_cur);
                    e_dw = *(const float *)(ax_cur + (we_off + 512 + (l32 & 15) * 4));
                    e_dn = *(const float *)(ax_cur + (we_off + 576 + (l32 & 15) * 4));
                } else {
                    e_dw = *(const float *)(ax_cur + (we_off + 512 + (l32 & 15) * 4));
                }
            }
            if (Q4 && PREV && piece == 2) e_am = load_am(ax_prev, 1);
            const i32x4 b1 = F.w[0], b0 = F.w[1];
#pragma unroll
            for (int tb = 0; tb < 2; tb++) {
                if (piece == 0) {   // the first block of a super-block starts the integer sums
                    i32x16 z;
#pragma unroll
                    for (int r = 0; r < 16; r++) z[r] = 0;
                    hi[tb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(F.a[tb], b1, z, 0, 0, 0);
                    lo[tb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(F.a[tb], b0, z, 0, 0, 0);
                } else {
                    hi[tb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(F.a[tb], b1, hi[tb], 0, 0, 0);
                    lo[tb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(F.a[tb], b0, lo[tb], 0, 0, 0);
                }
            }
            if (PREV) scale_piece(d8, phi[piece >> 2], plo[piece >> 2], e_M, dw, dn, piece >> 2, piece & 3);
            if (Q4 && ((PREV && piece == 3) || piece == 7)) e_M = min_term(am, piece == 7 ? e_bm : bm);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    super_block(std::false_type{}, std::false_type{}, sb_lo);
    for (int64_t sb = sb_lo + 1; sb < sb_hi; sb += 2) {
        super_block(std::true_type{}, std::true_type{}, sb);
        if (sb + 1 < sb_hi) super_block(std::false_type{}, std::true_type{}, sb + 1);
    }
    // the last super-block's sums; its scale data for the first piece are in the registers
    {
        const bool odd = (sb_hi - 1 - sb_lo) & 1;
        const uint8_t *ax = odd ? aux1 : aux0;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int tb = 0; tb < 2; tb++) {
            const f32x16 M = tb == 0 ? e_M : min_term(load_am(ax, 1), e_bm);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const f32x4 d8 = tb == 0 && q == 0 ? e_d8 : load_d8(ax, tb, q);
                if (odd) scale_piece(d8, hiY[tb], loY[tb], M, e_dw, e_dn, tb, q);
                else scale_piece(d8, hiX[tb], loX[tb], M, e_dw, e_dn, tb, q);
            }
        }
    }

    if constexpr (EPI) {
        // Q, K and V of a prompt batch: the rotation and the cache stores ride in the epilogue.  A lane holds row n of the matrix =
        // element d of head n / D; its partner in the pair is the neighbouring lane.  Same roundings as k_rope_kv_store.
        const int kind = P.m[mi].epi;   // uniform over the group
        const int64_t n = row0 + wrow0 + l32;
        const int D = P.rope.D, d = (int)(n % D);
        const int64_t head = n / D;
        const bool rot = kind != WT_EPI_CACHE && d < P.rope.n_dims;
        const float2 *cs = P.rope.cs + (d >> 1);
        uint8_t *cache = (uint8_t *)dst + head * P.m[mi].nb2 + 2 * d;
        // Every load before the first store: on this hardware a wait for a load also waits for the stores issued before it, so loads
        // between the stores would put a store's trip to memory into the chain once per token.  The rotations of a 32-token tile
        // are requested and applied in place, then those of the other tile, then everything is stored; the wave's 64 cache cells
        // sit one per lane and are read across lanes.
        const bool row_live = n < N;
        const int64_t nb1 = P.m[mi].nb1;
        int cell_of_lane = 0;
        if (kind != WT_EPI_ROPE) {
            const int64_t bl = col0 + wcol0 + lane;
            cell_of_lane = P.rope.cells[bl < B ? bl : B - 1];
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);   // (no load ahead of this point either, where the registers are still in use)
        if (rot) {
#pragma unroll
            for (int tb = 0; tb < 2; tb++) {
                float2 t[16];
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int64_t b = col0 + wcol0 + tb * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
                    t[r] = cs[(b < B ? b : B - 1) * (D >> 1)];
                }
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const float x = acc[tb][r];
                    const float xp = __builtin_bit_cast(float, dpp_get<0xB1>(__builtin_bit_cast(int, x)));   // quad_perm [1, 0, 3, 2]: the other element of the pair
                    acc[tb][r] = (d & 1) ? add_rn(mul_rn(xp, t[r].y), mul_rn(x, t[r].x)) : sub_rn(mul_rn(x, t[r].x), mul_rn(xp, t[r].y));
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int tb = 0; tb < 2; tb++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int tl = tb * 32 + 8 * (r >> 2) + (r & 3);   // the token's place in the wave's 64, for lhi = 0; lhi = 1: 4 further on
                const int64_t b = col0 + wcol0 + tl + 4 * lhi;
                if (kind == WT_EPI_ROPE) {
                    if (row_live && b < B) dst[b * dst_stride + n] = acc[tb][r];
                } else {
                    const int c0 = __builtin_amdgcn_readlane(cell_of_lane, tl), c1 = __builtin_amdgcn_readlane(cell_of_lane, tl + 4);
                    if (row_live && b < B) *(_Float16 *)(cache + (int64_t)(lhi ? c1 : c0) * nb1) = (_Float16)acc[tb][r];
                }
            }
        return;
    }
#pragma unroll
    for (int tb = 0; tb < 2; tb++) {
        const int64_t n = row0 + wrow0 + l32;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int64_t b = col0 + wcol0 + tb * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
            if constexpr (ID) {
                const int c = slot_first + (int)(b - col0);
                if (n < N && c < slot_end) dst[(int64_t)rt.dst_row[c] * dst_stride + n] = acc[tb][r];
                continue;
            }
            if (n < N && b < B) {
                const int64_t o = (b - col0) * dst_stride + (n - row0);
                out[o] = residual ? acc[tb][r] + residual[o] : acc[tb][r];   // residual may be dst itself: one reader and writer per element
            }
        }
    }
}

// slices along K for products with few 128 x 256 tiles (same idea as mmq_k.hip's split: partial sums to a workspace, then k_split_sum)
static int wt_split_slices(int64_t N, int64_t K, int64_t B) {
    const int64_t groups = ((N + WT_BM - 1) / WT_BM) * ((B + WT_BN - 1) / WT_BN), nsb = K / QKK;
    if (groups >= 160) return 1;
    int64_t n = 256 / groups;
    if (n > nsb / 2) n = nsb / 2;
    if (n > 8) n = 8;
    if (n < 2) return 1;
    const int64_t per = (nsb + n - 1) / n;
    return (int)((nsb + per - 1) / per);
}

__global__ void __launch_bounds__(256) k_wt_split_sum(const float *__restrict__ part, float *__restrict__ dst, const float *__restrict__ residual,
                                                      int64_t N, int64_t B, int64_t dst_stride, int n_slices) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;   // N % 4 == 0 here
    if (i >= N * B) return;
    const int64_t b = i / N, n = i % N;
    f32x4 acc = *(const f32x4 *)(part + i);
    for (int sl = 1; sl < n_slices; sl++) {
        const f32x4 v = *(const f32x4 *)(part + (int64_t)sl * N * B + i);
#pragma unroll
        for (int j = 0; j < 4; j++) acc[j] = add_rn(acc[j], v[j]);
    }
    const int64_t o = b * dst_stride + n;
    if (residual) {
#pragma unroll
        for (int j = 0; j < 4; j++) acc[j] = add_rn(acc[j], residual[o + j]);
    }
#pragma unroll
    for (int j = 0; j < 4; j++) dst[o + j] = acc[j];
}

// The same sum for a product whose rows are normalised next: one 256-thread group per activation row adds the row's slices and
// the residual in k_wt_split_sum's order, stores the row, and continues with RMS_NORM -> MUL(w) -> the row of y and its part of
// the tile image from the registers (what k_rms_norm_mul_quant<NV, 2> does after loading the row).
template <int NV>
__global__ void __launch_bounds__(256) k_wt_split_sum_norm(const float *__restrict__ part, float *__restrict__ dst, const float *__restrict__ residual,
                                                           int64_t N, int64_t B, int64_t dst_stride, int n_slices, const float *__restrict__ w, float eps,
                                                           float *__restrict__ y, int64_t y_stride, uint8_t *__restrict__ act_out) {
    __shared__ float sh[4];
    const int64_t b = blockIdx.x;
    f32x4 v[NV];
#pragma unroll
    for (int it = 0; it < NV; it++) {
        const int64_t n = ((int64_t)it * 256 + threadIdx.x) * 4;
        v[it] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (n < N) {
            f32x4 acc = *(const f32x4 *)(part + b * N + n);
            for (int sl = 1; sl < n_slices; sl++) {
                const f32x4 t = *(const f32x4 *)(part + ((int64_t)sl * B + b) * N + n);
#pragma unroll
                for (int j = 0; j < 4; j++) acc[j] = add_rn(acc[j], t[j]);
            }
            const int64_t o = b * dst_stride + n;
            if (residual) {
                const f32x4 t = *(const f32x4 *)(residual + o);
#pragma unroll
                for (int j = 0; j < 4; j++) acc[j] = add_rn(acc[j], t[j]);
            }
            *(f32x4 *)(dst + o) = acc;
            v[it] = acc;
        }
    }
    rms_norm_quant_row<NV, 2, false>(nullptr, w, y ? y + b * y_stride : nullptr, act_out, b, N, B, eps, sh, nullptr, v);
}

void launch_split_sum_norm(hipStream_t s, const float *part, float *dst, const float *residual, int64_t N, int64_t B, int64_t dst_stride, int n_slices,
                           const float *w, float eps, float *y, int64_t y_stride, void *act_out) {
    MI355_LAUNCH((k_wt_split_sum_norm<4>), dim3((unsigned)B), dim3(256), 0, s, part, dst, residual, N, B, dst_stride, n_slices, w, eps, y, y_stride,
                 (uint8_t *)act_out);
}

}  // namespace mi355

using namespace mi355;

extern "C" {

size_t mi355_act_q8k_tiled_bytes(int64_t k, int64_t nrows) {
    if (k <= 0 || nrows <= 0 || k % QKK != 0) return 0;
    return wt_act_bytes(k, nrows);
}

int mi355_quantize_act_q8k_tiled(void *stream, const float *x, void *act, int64_t k, int64_t nrows, int64_t x_stride) {
    MI355_REQUIRE(k > 0 && k % QKK == 0, "quantize_act_q8k_tiled: k=%lld is not a multiple of 256", (long long)k);
    MI355_REQUIRE(nrows > 0 && nrows <= 65520, "quantize_act_q8k_tiled: nrows=%lld out of range", (long long)nrows);
    MI355_REQUIRE(x_stride >= k && x_stride % 4 == 0 && ((uintptr_t)x & 15) == 0, "quantize_act_q8k_tiled: x must be 16-byte aligned with a row stride that is a multiple of 4 floats");
    MI355_REQUIRE(((uintptr_t)act & 15) == 0, "quantize_act_q8k_tiled: workspace must be 16-byte aligned");
    const int64_t b16 = (nrows + 15) & ~(int64_t)15;
    const dim3 grid((unsigned)((k / QKK + 3) / 4), (unsigned)b16);
    MI355_LAUNCH(k_quantize_q8k_tiled, grid, dim3(256), 0, (hipStream_t)stream, x, (uint8_t *)act, k, nrows, x_stride);
    return launch_status("k_quantize_q8k_tiled");
}

size_t mi355_kq_tiles_bytes(int type, int64_t rows, int64_t K) {
    if (rows <= 0 || K <= 0 || K % QKK != 0 || !wt_has_images(type)) return 0;
    return wt_weight_bytes(type, rows, K);
}

int mi355_kq_unpack_tiles(void *stream, int type, const void *W, void *tiles, int64_t rows, int64_t K) {
    MI355_REQUIRE(wt_has_images(type), "kq_unpack_tiles: weight type %d has no tile images", type);
    MI355_REQUIRE(rows > 0 && K > 0 && K % QKK == 0, "kq_unpack_tiles: bad shape rows=%lld K=%lld", (long long)rows, (long long)K);
    const row_layout L = make_row_layout(type, K);
    MI355_REQUIRE(layout_aligned(W, L) && ((uintptr_t)tiles & 15) == 0, "kq_unpack_tiles: rows are not 16-byte aligned (K=%lld)", (long long)K);
    const int64_t pieces = ((rows + 15) & ~(int64_t)15) * (K >> 8) * 8;
    MI355_REQUIRE((pieces + 255) / 256 < 0x7fffffff, "kq_unpack_tiles: too many pieces for one launch");
    const dim3 grid((unsigned)((pieces + 255) / 256)), block(256);
    if (type == MI355_Q4_K) MI355_LAUNCH(k_unpack_tiles<MI355_Q4_K>, grid, block, 0, (hipStream_t)stream, (const uint8_t *)W, (int8_t *)tiles, rows, K, L);
    else if (type == MI355_Q5_K) MI355_LAUNCH(k_unpack_tiles<MI355_Q5_K>, grid, block, 0, (hipStream_t)stream, (const uint8_t *)W, (int8_t *)tiles, rows, K, L);
    else if (type == MI355_IQ4_XS) MI355_LAUNCH(k_unpack_tiles<MI355_IQ4_XS>, grid, block, 0, (hipStream_t)stream, (const uint8_t *)W, (int8_t *)tiles, rows, K, L);
    else MI355_LAUNCH(k_unpack_tiles<MI355_Q6_K>, grid, block, 0, (hipStream_t)stream, (const uint8_t *)W, (int8_t *)tiles, rows, K, L);
    return launch_status("k_unpack_tiles");
}

// The plan of one launch over n_mats matrices (rows Ns[]) sharing B activation rows; a single matrix with few tiles is cut along K.
struct wt_plan {
    int n_col_tiles, n_tiles, first_tile[3];
    int slices;   // > 1: every tile cut (single matrix only)
};
static wt_plan wt_make_plan(int n_mats, const int64_t *Ns, int64_t K, int64_t B, bool have_ws) {
    wt_plan p;
    p.n_col_tiles = (int)((B + WT_BN - 1) / WT_BN);
    p.n_tiles = 0;
    for (int i = 0; i < 3; i++) {
        p.first_tile[i] = i < n_mats ? p.n_tiles : 0x7fffffff;
        if (i < n_mats) p.n_tiles += (int)((Ns[i] + WT_BM - 1) / WT_BM) * p.n_col_tiles;
    }
    p.slices = have_ws && n_mats == 1 && Ns[0] % 4 == 0 ? wt_split_slices(Ns[0], K, B) : 1;
    return p;
}
static size_t wt_plan_ws_bytes(const wt_plan &p, const int64_t *Ns, int64_t B) {
    return p.slices > 1 ? (size_t)p.slices * (size_t)Ns[0] * (size_t)B * sizeof(float) : 0;
}

size_t mi355_mul_mat_q8k_tiled_ws_bytes(int64_t N, int64_t K, int64_t B) {
    if (N <= 0 || K <= 0 || B <= 0 || K % QKK != 0) return 0;
    return wt_plan_ws_bytes(wt_make_plan(1, &N, K, B, true), &N, B);
}

size_t mi355_mul_mat_q8k_tiled_multi_ws_bytes(int n_mats, const int64_t *Ns, int64_t K, int64_t B) {
    if (n_mats < 1 || n_mats > 3 || Ns == nullptr || K <= 0 || B <= 0 || K % QKK != 0) return 0;
    for (int i = 0; i < n_mats; i++)
        if (Ns[i] <= 0) return 0;
    return wt_plan_ws_bytes(wt_make_plan(n_mats, Ns, K, B, true), Ns, B);
}

// norm: the single matrix's rows are normalised next (mi355_mul_mat_q8k_tiled_norm); taken when the product is cut along K, whose
// sum launch then carries the norm.  *norm_done says whether it did.
struct wt_norm {
    const float *w;
    float eps;
    float *y;
    int64_t y_stride;
    void *act_out;
};
static int wt_radix_shift(int type) { return type == MI355_Q4_K ? 3 : type == MI355_Q5_K ? 4 : 6; }

// qkv: the three matrices are Q, K and V of a prompt batch; their rows are rotated and stored as wt_mat::epi says
struct wt_qkv {
    wt_rope rope;
    int64_t k_nb1, k_nb2, v_nb1, v_nb2;
};
static int mul_mat_q8k_tiled_launch(void *stream, const int *types, int n_mats, const mi355_tiled_mat *mats, const void *act, int64_t K, int64_t B, void *ws,
                                    size_t ws_bytes, const wt_norm *norm, bool *norm_done, const wt_qkv *qkv = nullptr);

int mi355_mul_mat_q8k_tiled_multi(void *stream, int type, int n_mats, const mi355_tiled_mat *mats, const void *act, int64_t K, int64_t B,
                                  void *ws, size_t ws_bytes) {
    const int types[3] = {type, type, type};
    return mul_mat_q8k_tiled_launch(stream, types, n_mats, mats, act, K, B, ws, ws_bytes, nullptr, nullptr);
}

int mi355_mul_mat_q8k_tiled_mixed(void *stream, int n_mats, const int *types, const mi355_tiled_mat *mats, const void *act, int64_t K, int64_t B) {
    MI355_REQUIRE(types != nullptr, "mul_mat_q8k_tiled_mixed: no types");
    return mul_mat_q8k_tiled_launch(stream, types, n_mats, mats, act, K, B, nullptr, 0, nullptr, nullptr);
}

int mi355_mul_mat_q8k_tiled_qkv_rope(void *stream, const int *types, const mi355_tiled_mat *mats, const void *act, int64_t K, int64_t B, const float *rope_table,
                                     const int32_t *cells, int64_t D, int n_dims, size_t k_nb1, size_t k_nb2, size_t v_nb1, size_t v_nb2) {
    MI355_REQUIRE(types != nullptr && mats != nullptr && rope_table != nullptr && cells != nullptr, "mul_mat_q8k_tiled_qkv_rope: null operand");
    MI355_REQUIRE(D > 0 && D % 2 == 0 && n_dims > 0 && n_dims % 2 == 0 && n_dims <= D, "mul_mat_q8k_tiled_qkv_rope: bad head size or n_dims");
    for (int i = 0; i < 3; i++)
        MI355_REQUIRE(mats[i].N > 0 && mats[i].N % D == 0 && mats[i].residual == nullptr, "mul_mat_q8k_tiled_qkv_rope: matrix %d: whole heads, no residual", i);
    MI355_REQUIRE(mats[1].N == mats[2].N && (((uintptr_t)mats[1].dst | (uintptr_t)mats[2].dst | k_nb1 | k_nb2 | v_nb1 | v_nb2) & 1) == 0 &&
                  ((uintptr_t)rope_table & 7) == 0, "mul_mat_q8k_tiled_qkv_rope: K and V have the same heads; caches and strides are 2-byte aligned");
    wt_qkv q;
    q.rope.cs = (const float2 *)rope_table;
    q.rope.cells = cells;
    q.rope.D = (int)D;
    q.rope.n_dims = n_dims;
    q.k_nb1 = (int64_t)k_nb1; q.k_nb2 = (int64_t)k_nb2; q.v_nb1 = (int64_t)v_nb1; q.v_nb2 = (int64_t)v_nb2;
    return mul_mat_q8k_tiled_launch(stream, types, 3, mats, act, K, B, nullptr, 0, nullptr, nullptr, &q);
}

static int mul_mat_q8k_tiled_launch(void *stream, const int *types, int n_mats, const mi355_tiled_mat *mats, const void *act, int64_t K, int64_t B, void *ws,
                                    size_t ws_bytes, const wt_norm *norm, bool *norm_done, const wt_qkv *qkv) {
    MI355_REQUIRE(n_mats >= 1 && n_mats <= 3 && mats != nullptr, "mul_mat_q8k_tiled: 1 to 3 matrices per launch, got %d", n_mats);
    bool all_q6 = true;
    for (int i = 0; i < n_mats; i++) {
        MI355_REQUIRE(wt_has_images(types[i]), "mul_mat_q8k_tiled: weight type %d has no tile images", types[i]);
        all_q6 = all_q6 && wt_radix_shift(types[i]) == 6;   // Q6_K, IQ4_XS: radix 64 and no minima
    }
    MI355_REQUIRE(K > 0 && B > 0 && K % QKK == 0, "mul_mat_q8k_tiled: bad shape K=%lld B=%lld (K must be a multiple of 256)", (long long)K, (long long)B);
    MI355_REQUIRE(act != nullptr && ((uintptr_t)act & 15) == 0, "mul_mat_q8k_tiled: the activation image is not 16-byte aligned");
    int64_t Ns[3] = {0, 0, 0};
    for (int i = 0; i < n_mats; i++) {
        MI355_REQUIRE(mats[i].N > 0 && mats[i].dst_stride >= mats[i].N, "mul_mat_q8k_tiled: matrix %d has N=%lld, dst_stride=%lld", i, (long long)mats[i].N,
                      (long long)mats[i].dst_stride);
        MI355_REQUIRE(mats[i].tiles != nullptr && ((uintptr_t)mats[i].tiles & 15) == 0 && mats[i].dst != nullptr, "mul_mat_q8k_tiled: matrix %d: bad pointers", i);
        Ns[i] = mats[i].N;
    }
    wt_plan p = wt_make_plan(n_mats, Ns, K, B, ws != nullptr && ((uintptr_t)ws & 15) == 0);
    if (ws_bytes < wt_plan_ws_bytes(p, Ns, B)) p = wt_make_plan(n_mats, Ns, K, B, false);
    MI355_REQUIRE((int64_t)p.n_tiles + 8 < (1 << 30), "mul_mat_q8k_tiled: too many tiles");
    hipStream_t s = (hipStream_t)stream;
    wt_launch L;
    for (int i = 0; i < 3; i++) {
        const int k = i < n_mats ? i : 0;
        L.m[i].w_img = (const int8_t *)mats[k].tiles;
        L.m[i].dst = mats[k].dst;
        L.m[i].residual = mats[k].residual;
        L.m[i].N = mats[k].N;
        L.m[i].dst_stride = mats[k].dst_stride;
        L.m[i].first_tile = p.first_tile[i];
        L.m[i].shift = wt_radix_shift(types[k]);
        L.m[i].epi = 0;
        L.m[i].nb1 = L.m[i].nb2 = 0;
    }
    L.rope = wt_rope{nullptr, nullptr, 0, 0};
    if (qkv) {
        L.rope = qkv->rope;
        L.m[0].epi = WT_EPI_ROPE;
        L.m[1].epi = WT_EPI_ROPE_CACHE; L.m[1].nb1 = qkv->k_nb1; L.m[1].nb2 = qkv->k_nb2;
        L.m[2].epi = WT_EPI_CACHE;      L.m[2].nb1 = qkv->v_nb1; L.m[2].nb2 = qkv->v_nb2;
    }
    L.n_col_tiles = p.n_col_tiles;
    L.n_tiles = p.n_tiles;
    L.n_tiles_padded = (p.n_tiles + 7) & ~7;
    if (p.slices > 1) {   // partial sums: one N x B slab per slice in the workspace
        L.m[0].dst = (float *)ws;
        L.m[0].residual = nullptr;
        L.m[0].dst_stride = Ns[0];
    }
    const dim3 grid((unsigned)L.n_tiles_padded, (unsigned)p.slices);
    if (qkv) {
        if (all_q6) MI355_LAUNCH((k_mmq_w<MI355_Q6_K, false, true>), grid, dim3(512), 0, s, L, (const int8_t *)act, K, B, wt_route{});
        else MI355_LAUNCH((k_mmq_w<MI355_Q4_K, false, true>), grid, dim3(512), 0, s, L, (const int8_t *)act, K, B, wt_route{});
        return launch_status("k_mmq_w (Q/K/V)");
    }
    if (all_q6) MI355_LAUNCH(k_mmq_w<MI355_Q6_K>, grid, dim3(512), 0, s, L, (const int8_t *)act, K, B, wt_route{});
    else MI355_LAUNCH(k_mmq_w<MI355_Q4_K>, grid, dim3(512), 0, s, L, (const int8_t *)act, K, B, wt_route{});
    if (p.slices > 1 && norm && Ns[0] <= 4096 && mats[0].dst_stride % 4 == 0 && ((uintptr_t)mats[0].dst & 15) == 0 &&
        (mats[0].residual == nullptr || ((uintptr_t)mats[0].residual & 15) == 0)) {
        launch_split_sum_norm(s, (const float *)ws, mats[0].dst, mats[0].residual, Ns[0], B, mats[0].dst_stride, p.slices, norm->w, norm->eps, norm->y,
                              norm->y_stride, norm->act_out);
        *norm_done = true;
    } else if (p.slices > 1) {
        MI355_LAUNCH(k_wt_split_sum, dim3((unsigned)((Ns[0] * B / 4 + 255) / 256)), dim3(256), 0, s, (const float *)ws, mats[0].dst, mats[0].residual, Ns[0], B,
                     mats[0].dst_stride, p.slices);
    }
    return launch_status("k_mmq_w");
}

int mi355_mul_mat_q8k_tiled_norm(void *stream, int type, const void *tiles, const void *act, float *dst, const float *residual, int64_t N, int64_t K,
                                 int64_t B, int64_t dst_stride, void *ws, size_t ws_bytes, const float *norm_w, float eps, float *y, int64_t y_stride,
                                 void *act_out) {
    MI355_REQUIRE(N > 0 && K > 0 && B > 0 && N % QKK == 0, "mul_mat_q8k_tiled_norm: bad shape N=%lld K=%lld B=%lld (N must be a multiple of 256)", (long long)N,
                  (long long)K, (long long)B);
    MI355_REQUIRE(norm_w != nullptr && act_out != nullptr && ((uintptr_t)norm_w & 15) == 0 && ((uintptr_t)act_out & 15) == 0 && ((uintptr_t)y & 15) == 0 &&
                  y_stride % 4 == 0, "mul_mat_q8k_tiled_norm: the norm's operands must be 16-byte aligned");
    mi355_tiled_mat m;
    m.tiles = tiles;
    m.dst = dst;
    m.residual = residual;
    m.N = N;
    m.dst_stride = dst_stride;
    const wt_norm nm = {norm_w, eps, y, y_stride, act_out};
    bool done = false;
    const int rc = mul_mat_q8k_tiled_launch(stream, &type, 1, &m, act, K, B, ws, ws_bytes, &nm, &done);
    if (rc != MI355_OK || done) return rc;
    return mi355_rms_norm_mul_quant_q8k_tiled(stream, dst, dst_stride, norm_w, y, y_stride, act_out, N, B, eps);   // an uncut product: the norm is its own launch
}

int mi355_mul_mat_q8k_tiled(void *stream, int type, const void *tiles, const void *act, float *dst, const float *residual, int64_t N,
                            int64_t K, int64_t B, int64_t dst_stride, void *ws, size_t ws_bytes) {
    MI355_REQUIRE(N > 0 && K > 0 && B > 0, "mul_mat_q8k_tiled: bad shape N=%lld K=%lld B=%lld", (long long)N, (long long)K, (long long)B);
    mi355_tiled_mat m;
    m.tiles = tiles;
    m.dst = dst;
    m.residual = residual;
    m.N = N;
    m.dst_stride = dst_stride;
    return mi355_mul_mat_q8k_tiled_multi(stream, type, 1, &m, act, K, B, ws, ws_bytes);
}

// ---- MUL_MAT_ID on tile images ------------------------------------------------------------------------------------------------
static int64_t wt_id_max_tiles(int64_t n_expert, int64_t S) { return (S + WT_BN - 1) / WT_BN + n_expert; }

size_t mi355_mul_mat_id_q8k_tiled_ws_bytes(int64_t K, int64_t n_expert, int64_t n_used, int64_t T) {
    if (K <= 0 || n_expert <= 0 || n_used <= 0 || T <= 0 || K % QKK != 0) return 0;
    const int64_t S = T * n_used, max_tiles = wt_id_max_tiles(n_expert, S);
    const size_t img = (wt_act_bytes(K, max_tiles * WT_BN) + 255) & ~(size_t)255;
    return img + ((2 * (size_t)S + 4 * (size_t)max_tiles + 4) * sizeof(int32_t) + 255 & ~(size_t)255);
}

int mi355_mul_mat_id_q8k_tiled(void *stream, int type, const void *expert_tiles, size_t expert_tiles_bytes, const float *b, const int32_t *ids,
                               int64_t ids_stride, float *dst, int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T,
                               void *ws, size_t ws_bytes) {
    MI355_REQUIRE(wt_has_images(type), "mul_mat_id_q8k_tiled: weight type %d has no tile images", type);
    MI355_REQUIRE(N > 0 && K > 0 && n_expert > 0 && n_expert <= 256 && n_used > 0 && nb1 > 0 && T > 0 && K % QKK == 0, "mul_mat_id_q8k_tiled: bad shape");
    MI355_REQUIRE(ids_stride >= n_used && T * n_used < (1 << 24) && nb1 * T < (1 << 24), "mul_mat_id_q8k_tiled: bad ids stride or too many slots");
    MI355_REQUIRE(expert_tiles != nullptr && ((uintptr_t)expert_tiles & 15) == 0 && expert_tiles_bytes % 16 == 0 && expert_tiles_bytes >= wt_weight_bytes(type, N, K),
                  "mul_mat_id_q8k_tiled: expert images must be 16-byte aligned and %zu bytes or more apart", wt_weight_bytes(type, N, K));
    MI355_REQUIRE(((uintptr_t)b & 15) == 0, "mul_mat_id_q8k_tiled: b must be 16-byte aligned");
    if (ws == nullptr || ((uintptr_t)ws & 15) != 0 || ws_bytes < mi355_mul_mat_id_q8k_tiled_ws_bytes(K, n_expert, n_used, T)) {
        set_error("mul_mat_id_q8k_tiled: workspace of %zu bytes, need %zu (16-byte aligned)", ws_bytes, mi355_mul_mat_id_q8k_tiled_ws_bytes(K, n_expert, n_used, T));
        return MI355_ERR_WORKSPACE;
    }
    const int64_t S = T * n_used, max_tiles = wt_id_max_tiles(n_expert, S), B_img = max_tiles * WT_BN;
    MI355_REQUIRE(B_img <= 65535, "mul_mat_id_q8k_tiled: too many slots for one launch");
    uint8_t *img = (uint8_t *)ws;
    int32_t *act_row = (int32_t *)(img + ((wt_act_bytes(K, B_img) + 255) & ~(size_t)255)), *dst_row = act_row + S, *tiles = dst_row + S, *n_tiles = tiles + 4 * max_tiles;
    hipStream_t s = (hipStream_t)stream;
    launch_route_slots(s, ids, ids_stride, n_expert, n_used, nb1, T, WT_BN, act_row, dst_row, tiles, n_tiles);
    const dim3 qgrid((unsigned)((K / QKK + 3) / 4), (unsigned)B_img);
    MI355_LAUNCH(k_quantize_q8k_tiled_routed, qgrid, dim3(256), 0, s, b, img, K, B_img, K, act_row, tiles, n_tiles);
    wt_launch L;
    L.rope = wt_rope{nullptr, nullptr, 0, 0};
    for (int i = 0; i < 3; i++) {
        L.m[i].w_img = (const int8_t *)expert_tiles;
        L.m[i].dst = dst;
        L.m[i].residual = nullptr;
        L.m[i].N = N;
        L.m[i].dst_stride = N;
        L.m[i].first_tile = i == 0 ? 0 : 0x7fffffff;
        L.m[i].shift = wt_radix_shift(type);
        L.m[i].epi = 0;
        L.m[i].nb1 = L.m[i].nb2 = 0;
    }
    const int64_t n_row_tiles = (N + WT_BM - 1) / WT_BM;
    MI355_REQUIRE(n_row_tiles * max_tiles + 8 < (1 << 30), "mul_mat_id_q8k_tiled: too many tiles");
    L.n_col_tiles = (int)max_tiles;
    L.n_tiles = (int)(n_row_tiles * max_tiles);
    L.n_tiles_padded = (L.n_tiles + 7) & ~7;
    const wt_route rt = {dst_row, tiles, n_tiles, (int64_t)expert_tiles_bytes};
    const dim3 grid((unsigned)L.n_tiles_padded);
    if (wt_radix_shift(type) == 6) MI355_LAUNCH((k_mmq_w<MI355_Q6_K, true>), grid, dim3(512), 0, s, L, (const int8_t *)img, K, B_img, rt);
    else MI355_LAUNCH((k_mmq_w<MI355_Q4_K, true>), grid, dim3(512), 0, s, L, (const int8_t *)img, K, B_img, rt);
    return launch_status("k_mmq_w (routed)");
}

}  // extern "C"
