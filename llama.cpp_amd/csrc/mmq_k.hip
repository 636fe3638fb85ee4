// Batched GEMM for the K-quants (Q4_K, Q6_K) on the int8 matrix cores with integer
// accumulation over whole 256-element super-blocks (B > 8):
//   dst[b][n] = sum_k W[n][k] * x[b][k]
//
// Activations are quantized per super-block exactly as ggml-cpu does for these weight types
// (quantize_row_q8_K_ref, ggml/src/ggml-quants.c:2479-2516: one f32 scale d8 per 256 elements,
// int8 levels, integer sums per sub-block), so a super-block contributes
//   Q4_K:  d*d8 * sum_j sc_j * (n . q)_j  -  dmin*d8 * sum_j m_j * bsum_j      (ggml-cpu-quants.c:6817-6848)
//   Q6_K:  d*d8 * sum_g sc_g * ((l-32) . q)_g                                  (ggml-cpu-quants.c:8262-8283)
// with every sum an exact integer.  The 6-bit / 8-bit sub-scales are folded into the weight
// operand when a tile is unpacked to LDS: the integer sc*n (10 bits) or sc*(l-32) (14 bits) is
// split into two int8 planes, value = R*hi + lo (R = 8 for Q4_K with sc = 8a+b, hi = a*n,
// lo = b*n; R = 64 for Q6_K with hi = v >> 6, lo = v & 63).  Each plane is contracted with
// v_mfma_i32_32x32x32_i8 into an int32 accumulator that runs over all 8 blocks of a
// super-block, so the vector ALU touches a result tile once per 256 elements instead of once
// per 32.  The Q4_K min term is one v_mfma_f32_32x32x16_f16 per super-block on exact small
// integers: k slots 0..7 carry (bsum & 63) x m_j, slots 8..15 carry (bsum >> 6) x 64*m_j.
//
// A 256-thread group (4 waves, 2 x 2) owns a 64 (weight rows) x 128 (activation rows) tile of
// dst; each wave a 32 x 64 sub-tile (1 x 2 MFMA tiles).  K is walked in stages of 128 elements.  k_mmq_kp is the kernel
// of the full-width tile: double-buffered LDS, one barrier per stage, activations by direct global-to-LDS transfers, the
// weight unpack interleaved with the matrix instructions.  (Keeping the unpacked weights in the registers of the lane that
// feeds them to the matrix cores, with no LDS round trip, measured the same: the unpack is then repeated by the two waves
// that share rows, and the vector ALU is the limit either way at ~11 instructions per matrix instruction.)  k_mmq_k is
// the single-buffered kernel (register prefetch, two barriers per stage) kept for the 64 x 64 tile that sparse expert
// routing uses.
//
// MFMA operand mapping (A = activations, B = weights, D[i][j]): lane l supplies row l % 32
// and k bytes [16*(l/32), +16) (f16: k slots [8*(l/32), +8)); D register r of lane l is
// i = 8*(r/4) + 4*(l/32) + r%4, j = l % 32.
#include "common.hpp"
#include "q8k.hpp"
#include "qdot.hpp"

namespace mi355 {

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef short i16x2 __attribute__((ext_vector_type(2)));

constexpr int KQ_BK = 128;            // K elements per stage (half a super-block)
constexpr int KQ_LDK = KQ_BK + 16;    // LDS row pitch in bytes

// One wave per (row, super-block); 4 super-blocks per group.
__global__ void __launch_bounds__(256) k_quantize_q8k(const float *__restrict__ x, int8_t *__restrict__ q, float *__restrict__ d8,
                                                      _Float16 *__restrict__ bs, int64_t K, int64_t x_stride) {
    const int lane = threadIdx.x & 63;
    const int64_t sb = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t row = blockIdx.y;
    const int64_t nsb = K / QKK;
    if (sb >= nsb) return;   // whole wave
    const f32x4 v = *(const f32x4 *)(x + row * x_stride + sb * QKK + lane * 4);
    q8k_quantize_wave(v, lane, q + row * K + sb * QKK, d8 + row * nsb + sb, bs + (row * nsb + sb) * 16);
}

// ---- per-thread prefetch registers of one stage -------------------------------------------
// WI / AI: 16-byte weight pieces (of BM rows x 4) and activation pieces (of BN rows x 8) per thread
template <int TYPE, int WI, int AI> struct kq_regs;
template <int WI, int AI> struct kq_regs<MI355_Q4_K, WI, AI> {
    u32x4 q[WI], hdr[WI];
    u32x4 a[AI];
};
template <int WI, int AI> struct kq_regs<MI355_Q6_K, WI, AI> {
    u32x4 ql[WI], qh[WI];
    int scA[WI], scB[WI];   // int8 scales of the two 16-element groups of each chunk
    float d[WI];
    u32x4 a[AI];
};

struct kq_smem {
    int8_t *sW1, *sW0, *sA;     // [128][KQ_LDK] planes
    float *sWd, *sWn;           // [128] d and dmin of the current super-block
    _Float16 *sWm;              // [128][16] m_j and 64*m_j (Q4_K)
    float *sAd;                 // [128] d8
    _Float16 *sAb;              // [128][16]
};

template <int TYPE, int WI, int AI>
__device__ __forceinline__ void kq_fetch(kq_regs<TYPE, WI, AI> &R, const uint8_t *__restrict__ W, const row_layout &L, int64_t row0, int64_t N,
                                         const int8_t *__restrict__ aq, const int (&arow)[AI], int64_t K, int64_t k0) {
    const int tid = threadIdx.x;
    const int64_t sb = k0 >> 8;
    const int half = (int)((k0 >> 7) & 1);
#pragma unroll
    for (int it = 0; it < WI; it++) {
        const int idx = tid + it * 256;
        const int r = idx >> 2, p = idx & 3;
        const int64_t row = row0 + r < N ? row0 + r : N - 1;
        const uint8_t *wrow = W + row * L.row_bytes;
        if constexpr (TYPE == MI355_Q4_K) {
            const uint8_t *blk = wrow + sb * Q4_K_BYTES;
            R.q[it] = load16(blk + 16 + (half * 2 + (p >> 1)) * 32 + (p & 1) * 16);
            R.hdr[it] = load16(blk);
        } else {
            const int l0 = 16 * (p & 1), qa = p >> 1;
            R.ql[it] = load16(wrow + sb * 128 + half * 64 + p * 16);
            R.qh[it] = load16(wrow + L.off_b + sb * 64 + half * 32 + l0);
            const int8_t *sc = (const int8_t *)(wrow + L.off_c + sb * 16 + half * 8 + (l0 >> 4));
            R.scA[it] = sc[2 * qa];
            R.scB[it] = sc[2 * qa + 4];
            R.d[it] = half_bits_to_float(*(const unsigned short *)(wrow + L.off_d + sb * 2));
        }
    }
#pragma unroll
    for (int it = 0; it < AI; it++) {
        const int idx = tid + it * 256;
        const int c = idx & 7;
        R.a[it] = load16(aq + (int64_t)arow[it] * K + k0 + c * 16);
    }
}

// Routing of a MUL_MAT_ID launch (semantics ggml/src/ggml.c:2723-2759): the (token, expert slot) pairs sorted by expert.
// Column c of the sorted list reads activation row act_row[c] and writes dst row dst_row[c]; every column tile
// belongs to one expert: tiles[4*i] = {expert, first column, end column, 0}.
struct mmq_route {
    const int32_t *act_row;
    const int32_t *dst_row;
    const int32_t *tiles;
    const int32_t *n_tiles;        // number of column tiles in use (device value)
    int64_t expert_bytes;          // bytes from one expert's matrix to the next
};

// 4 packed bytes (each <= 15) times a small factor (<= 7): no byte overflows, so two 16-bit multiplies do it
__device__ __forceinline__ u32 mul_bytes(u32 x, u32 f) {
    const u16x2 v = __builtin_bit_cast(u16x2, x);
    const u16x2 m = {(unsigned short)f, (unsigned short)f};
    const u16x2 p = v * m;
    return __builtin_bit_cast(u32, p);
}

// Q5_K: four levels 0..31 (bytes of a) times the sub-block scale 0..63 -> value = 16*hi + lo, hi <= 122, lo <= 15
__device__ __forceinline__ void q5k_planes(u32 a, int sc, u32 &hi, u32 &lo) {
    const u16x2 s = {(unsigned short)sc, (unsigned short)sc};
    const u16x2 e = __builtin_bit_cast(u16x2, a & 0x00FF00FFu);
    const u16x2 o = __builtin_bit_cast(u16x2, (a >> 8) & 0x00FF00FFu);
    const u16x2 pe = e * s, po = o * s;
    const u16x2 four = {4, 4};
    const u32 he = __builtin_bit_cast(u32, pe >> four), ho = __builtin_bit_cast(u32, po >> four);
    const u32 le = __builtin_bit_cast(u32, pe) & 0x000F000Fu, lo_ = __builtin_bit_cast(u32, po) & 0x000F000Fu;
    hi = (he & 0x00FF00FFu) | ((ho & 0x00FF00FFu) << 8);
    lo = le | (lo_ << 8);
}
// IQ4_XS: four table values (int8 bytes of a) times the block scale -32..31 -> value = 64*hi + lo, hi -64..63, lo 0..63 (the Q6_K form)
__device__ __forceinline__ void iq4xs_planes(u32 a, int sc, u32 &hi, u32 &lo) {
    const i16x2 s = {(short)sc, (short)sc};
    const i16x2 eight = {8, 8}, six = {6, 6};
    const i16x2 e = __builtin_bit_cast(i16x2, a << 8) >> eight;   // sign-extended even bytes
    const i16x2 o = __builtin_bit_cast(i16x2, a) >> eight;        // ... odd bytes
    const i16x2 pe = e * s, po = o * s;
    const u32 he = __builtin_bit_cast(u32, pe >> six), ho = __builtin_bit_cast(u32, po >> six);
    const u32 le = __builtin_bit_cast(u32, pe) & 0x003F003Fu, lo_ = __builtin_bit_cast(u32, po) & 0x003F003Fu;
    hi = (he & 0x00FF00FFu) | ((ho & 0x00FF00FFu) << 8);
    lo = le | (lo_ << 8);
}

// Q6_K: four unsigned 6-bit levels (bytes of a) -> int8 planes of sc*(level-32): value = 64*hi + lo
__device__ __forceinline__ void q6k_planes(u32 a, int sc, u32 &hi, u32 &lo) {
    const i16x2 s = {(short)sc, (short)sc};
    const i16x2 off = {(short)(-32 * sc), (short)(-32 * sc)};
    const i16x2 e = __builtin_bit_cast(i16x2, a & 0x00FF00FFu);
    const i16x2 o = __builtin_bit_cast(i16x2, (a >> 8) & 0x00FF00FFu);
    const i16x2 pe = e * s + off, po = o * s + off;
    const i16x2 six = {6, 6};
    const u32 he = __builtin_bit_cast(u32, pe >> six), ho = __builtin_bit_cast(u32, po >> six);
    const u32 le = __builtin_bit_cast(u32, pe) & 0x003F003Fu, lo_ = __builtin_bit_cast(u32, po) & 0x003F003Fu;
    hi = (he & 0x00FF00FFu) | ((ho & 0x00FF00FFu) << 8);
    lo = le | (lo_ << 8);
}

template <int TYPE, int WI, int AI>
__device__ __forceinline__ void kq_commit(const kq_regs<TYPE, WI, AI> &R, const kq_smem &S, int half) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int it = 0; it < WI; it++) {
        const int idx = tid + it * 256;
        const int r = idx >> 2, p = idx & 3;
        if constexpr (TYPE == MI355_Q4_K) {
            const int gl = p >> 1, h = p & 1;
            const u32x4 hdr = R.hdr[it];
            int scl, mnl, sch, mnh;
            q4k_scale_min(hdr[1], hdr[2], hdr[3], half * 4 + 2 * gl, scl, mnl);
            q4k_scale_min(hdr[1], hdr[2], hdr[3], half * 4 + 2 * gl + 1, sch, mnh);
            u32x4 l1, l0, h1, h0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const u32 nl = R.q[it][i] & 0x0F0F0F0Fu, nh = (R.q[it][i] >> 4) & 0x0F0F0F0Fu;
                l1[i] = mul_bytes(nl, (u32)scl >> 3);
                l0[i] = mul_bytes(nl, (u32)scl & 7u);
                h1[i] = mul_bytes(nh, (u32)sch >> 3);
                h0[i] = mul_bytes(nh, (u32)sch & 7u);
            }
            const int o = r * KQ_LDK + (2 * gl) * 32 + h * 16;
            *(u32x4 *)(S.sW1 + o) = l1;
            *(u32x4 *)(S.sW0 + o) = l0;
            *(u32x4 *)(S.sW1 + o + 32) = h1;
            *(u32x4 *)(S.sW0 + o + 32) = h0;
            if (half == 0 && p == 0) {   // per super-block: d, dmin and the eight mins
                S.sWd[r] = half_bits_to_float((unsigned short)(hdr[0] & 0xFFFFu));
                S.sWn[r] = half_bits_to_float((unsigned short)(hdr[0] >> 16));
                f16x8 m1, m64;
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    int sc, mn;
                    q4k_scale_min(hdr[1], hdr[2], hdr[3], j, sc, mn);
                    m1[j] = (_Float16)(float)mn;
                    m64[j] = (_Float16)(float)(64 * mn);
                }
                *(f16x8 *)(S.sWm + r * 16) = m1;
                *(f16x8 *)(S.sWm + r * 16 + 8) = m64;
            }
        } else {
            const int l0 = 16 * (p & 1), qa = p >> 1;
            u32x4 a1, a0, b1, b0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const u32 va = (R.ql[it][i] & 0x0F0F0F0Fu) | (((R.qh[it][i] >> (2 * qa)) & 0x03030303u) << 4);
                const u32 vb = ((R.ql[it][i] >> 4) & 0x0F0F0F0Fu) | (((R.qh[it][i] >> (2 * qa + 4)) & 0x03030303u) << 4);
                u32 hi, lo;
                q6k_planes(va, R.scA[it], hi, lo);
                a1[i] = hi; a0[i] = lo;
                q6k_planes(vb, R.scB[it], hi, lo);
                b1[i] = hi; b0[i] = lo;
            }
            const int o = r * KQ_LDK + qa * 32 + l0;
            *(u32x4 *)(S.sW1 + o) = a1;
            *(u32x4 *)(S.sW0 + o) = a0;
            *(u32x4 *)(S.sW1 + o + 64) = b1;
            *(u32x4 *)(S.sW0 + o + 64) = b0;
            if (half == 0 && p == 0) S.sWd[r] = R.d[it];
        }
    }
#pragma unroll
    for (int it = 0; it < AI; it++) {
        const int idx = tid + it * 256;
        const int r = idx >> 3, c = idx & 7;
        *(u32x4 *)(S.sA + r * KQ_LDK + c * 16) = R.a[it];
    }
}

// TW x TB: 32 x 32 MFMA tiles per wave along the weight / activation rows; waves are 2 x 2
template <int TYPE, int TW, int TB, int OCC, bool ID>
__global__ void __launch_bounds__(256, OCC) k_mmq_k(const uint8_t *__restrict__ W, const int8_t *__restrict__ aq, const float *__restrict__ ad8,
                                                    const _Float16 *__restrict__ abs_, float *dst, const float *residual,
                                                    int64_t N, int64_t K, int64_t B, int64_t dst_stride, row_layout L, int n_col_tiles,
                                                    int n_groups, int n_groups_padded, mmq_route route) {
    constexpr bool Q4 = TYPE == MI355_Q4_K;
    constexpr int RADIX_SHIFT = Q4 ? 3 : 6;
    constexpr int BM = 64 * TW, BN = 64 * TB;
    constexpr int WI = BM / 64, AI = BN / 32;
    __shared__ __attribute__((aligned(16))) int8_t sW1[BM * KQ_LDK];
    __shared__ __attribute__((aligned(16))) int8_t sW0[BM * KQ_LDK];
    __shared__ __attribute__((aligned(16))) int8_t sA[BN * KQ_LDK];
    __shared__ __attribute__((aligned(16))) float sWd[BM];
    __shared__ __attribute__((aligned(16))) float sWn[Q4 ? BM : 4];
    __shared__ __attribute__((aligned(16))) _Float16 sWm[Q4 ? BM * 16 : 8];
    __shared__ __attribute__((aligned(16))) float sAd[BN];
    __shared__ __attribute__((aligned(16))) _Float16 sAb[Q4 ? BN * 16 : 8];
    const kq_smem S = {sW1, sW0, sA, sWd, sWn, sWm, sAd, sAb};

    // hardware deals group ids round-robin over 8 XCDs; make logical neighbours (same weight panel) share one
    const int per_xcd = n_groups_padded >> 3;
    const int lid = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (lid >= n_groups) return;
    const int64_t row0 = (int64_t)(lid / n_col_tiles) * BM;
    int64_t col0 = (int64_t)(lid % n_col_tiles) * BN;
    if constexpr (ID) {   // the grid covers the worst case; B becomes the end of this expert's columns
        const int ct = lid % n_col_tiles;
        if (ct >= *route.n_tiles) return;
        W += (int64_t)route.tiles[4 * ct] * route.expert_bytes;
        col0 = route.tiles[4 * ct + 1];
        B = route.tiles[4 * ct + 2];
    }

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    const int wrow0 = (wave & 1) * (32 * TW);    // weight rows of this wave inside the tile
    const int wcol0 = (wave >> 1) * (32 * TB);   // activation rows of this wave inside the tile
    const int64_t nsb = K >> 8;

    f32x16 acc[TB][TW];
#pragma unroll
    for (int tb = 0; tb < TB; tb++)
#pragma unroll
        for (int tw = 0; tw < TW; tw++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[tb][tw][r] = 0.0f;

    // activation rows of this thread's staging pieces, and of the column whose scales it copies
    int arow[AI];
#pragma unroll
    for (int it = 0; it < AI; it++) {
        const int r = (tid + it * 256) >> 3;
        const int64_t col = col0 + r < B ? col0 + r : B - 1;
        arow[it] = ID ? route.act_row[col] : (int)col;
    }
    int srow = 0;
    if (tid < BN) {
        const int64_t col = col0 + tid < B ? col0 + tid : B - 1;
        srow = ID ? route.act_row[col] : (int)col;
    }

    kq_regs<TYPE, WI, AI> R;
    kq_fetch<TYPE, WI, AI>(R, W, L, row0, N, aq, arow, K, 0);

    for (int64_t sb = 0; sb < nsb; sb++) {
        i32x16 hi[TB][TW], lo[TB][TW];
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const int64_t k0 = sb * QKK + half * KQ_BK;
            __syncthreads();   // everyone is done reading the previous stage
            kq_commit<TYPE, WI, AI>(R, S, half);
            if (half == 0 && tid < BN) {   // per super-block activation scale and sub-block sums
                sAd[tid] = ad8[(int64_t)srow * nsb + sb];
                if constexpr (Q4) {
                    const u32x4 *src = (const u32x4 *)(abs_ + ((int64_t)srow * nsb + sb) * 16);
                    *(u32x4 *)(sAb + tid * 16) = src[0];
                    *(u32x4 *)(sAb + tid * 16 + 8) = src[1];
                }
            }
            __syncthreads();
            if (k0 + KQ_BK < K) kq_fetch<TYPE, WI, AI>(R, W, L, row0, N, aq, arow, K, k0 + KQ_BK);

#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                i32x4 af[TB], b1[TW], b0[TW];
#pragma unroll
                for (int tb = 0; tb < TB; tb++) af[tb] = *(const i32x4 *)(sA + (wcol0 + tb * 32 + l32) * KQ_LDK + ks * 32 + 16 * lhi);
#pragma unroll
                for (int tw = 0; tw < TW; tw++) {
                    b1[tw] = *(const i32x4 *)(sW1 + (wrow0 + tw * 32 + l32) * KQ_LDK + ks * 32 + 16 * lhi);
                    b0[tw] = *(const i32x4 *)(sW0 + (wrow0 + tw * 32 + l32) * KQ_LDK + ks * 32 + 16 * lhi);
                }
#pragma unroll
                for (int tb = 0; tb < TB; tb++)
#pragma unroll
                    for (int tw = 0; tw < TW; tw++) {
                        if (half == 0 && ks == 0) {   // first block of the super-block starts the integer sums
                            i32x16 z;
#pragma unroll
                            for (int r = 0; r < 16; r++) z[r] = 0;
                            hi[tb][tw] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[tb], b1[tw], z, 0, 0, 0);
                            lo[tb][tw] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[tb], b0[tw], z, 0, 0, 0);
                        } else {
                            hi[tb][tw] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[tb], b1[tw], hi[tb][tw], 0, 0, 0);
                            lo[tb][tw] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[tb], b0[tw], lo[tb][tw], 0, 0, 0);
                        }
                    }
            }
        }

        // end of the super-block: scale the integer sums into the f32 accumulators
#pragma unroll
        for (int tb = 0; tb < TB; tb++) {
            f32x4 d8[4];
#pragma unroll
            for (int q = 0; q < 4; q++) d8[q] = *(const f32x4 *)(sAd + wcol0 + tb * 32 + 8 * q + 4 * lhi);
#pragma unroll
            for (int tw = 0; tw < TW; tw++) {
                const int wr = wrow0 + tw * 32 + l32;
                const float dw = sWd[wr];
                if constexpr (Q4) {
                    const float dn = sWn[wr];
                    const f16x8 am = *(const f16x8 *)(sAb + (wcol0 + tb * 32 + l32) * 16 + 8 * lhi);
                    const f16x8 bm = *(const f16x8 *)(sWm + wr * 16 + 8 * lhi);
                    f32x16 z;
#pragma unroll
                    for (int r = 0; r < 16; r++) z[r] = 0.0f;
                    const f32x16 M = __builtin_amdgcn_mfma_f32_32x32x16_f16(am, bm, z, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int t = (hi[tb][tw][r] << RADIX_SHIFT) + lo[tb][tw][r];
                        acc[tb][tw][r] += d8[r >> 2][r & 3] * (dw * (float)t - dn * M[r]);
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int t = (hi[tb][tw][r] << RADIX_SHIFT) + lo[tb][tw][r];
                        acc[tb][tw][r] += d8[r >> 2][r & 3] * (dw * (float)t);
                    }
                }
            }
        }
    }

#pragma unroll
    for (int tb = 0; tb < TB; tb++)
#pragma unroll
        for (int tw = 0; tw < TW; tw++) {
            const int64_t n = row0 + wrow0 + tw * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t b = col0 + wcol0 + tb * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
                if (n < N && b < B) {
                    const int64_t o = (ID ? (int64_t)route.dst_row[b] : b) * dst_stride + n;
                    dst[o] = residual ? acc[tb][tw][r] + residual[o] : acc[tb][tw][r];
                }
            }
        }
}

// ---- pipelined variant of the 64 x 128 tile ---------------------------------------------------------------------------
// Two LDS buffers per operand, one barrier per 128-element stage.  While the matrix cores work on stage s from
// buffer s % 2, the same waves unpack the weights of stage s + 1 (fetched to registers during stage s - 1) into the other
// buffer, and the activations of stage s + 1 go from global memory straight to LDS (global_load_lds, no registers, no
// vector-ALU work).  LDS rows are 128 bytes without padding; the 16-byte chunk c of row r lives at chunk c ^ ((r >> 1) & 7),
// which keeps every 16-lane group of a ds_read_b128 on distinct banks.  A super-block is two stages, so the buffer of a
// stage is its half: every LDS access names its array statically and the compiler can tell the buffer being filled from
// the one being read.
constexpr int KP_ROW = 128;
__device__ __forceinline__ int kp_off(int row, int chunk) { return row * KP_ROW + ((chunk ^ ((row >> 1) & 7)) << 4); }

template <int TYPE> struct kp_w;   // the 16-byte weight piece of one stage that this thread unpacks (row tid / 4, piece tid % 4)
template <> struct kp_w<MI355_Q4_K> { u32x4 q; };
template <> struct kp_w<MI355_Q6_K> { u32x4 ql, qh; int scA, scB; };
template <> struct kp_w<MI355_Q5_K> { u32x4 q, qh; };
template <> struct kp_w<MI355_IQ4_XS> { u32x4 q; int ls; };   // ls: the block's scale, -32..31
// the two forms of the kernel: with a min term and an unsigned product (Q4_K, Q5_K) / signed products and no min term (Q6_K, IQ4_XS)
template <int TYPE> struct kp_form {
    static constexpr bool MIN = TYPE == MI355_Q4_K || TYPE == MI355_Q5_K;
    static constexpr int RADIX_SHIFT = TYPE == MI355_Q4_K ? 3 : TYPE == MI355_Q5_K ? 4 : 6;
};
// per super-block data of this thread's weight row: the Q4_K block header (d, dmin, 12 scale bytes) / the Q6_K d
template <int TYPE> struct kp_h;
template <> struct kp_h<MI355_Q4_K> { u32x4 hdr; };
template <> struct kp_h<MI355_Q6_K> { unsigned short d; };   // raw fp16 bits: converting at the load would wait for it
template <> struct kp_h<MI355_Q5_K> { u32x4 hdr; };
template <> struct kp_h<MI355_IQ4_XS> { unsigned short d; };

template <int TYPE>
__device__ __forceinline__ void kp_fetch_h(kp_h<TYPE> &H, const uint8_t *__restrict__ wrow, const row_layout &L, int64_t sb) {
    if constexpr (TYPE == MI355_Q4_K) H.hdr = load16(wrow + sb * Q4_K_BYTES);
    else if constexpr (TYPE == MI355_Q5_K) H.hdr = load16(wrow + sb * Q5_K_BYTES);
    else if constexpr (TYPE == MI355_IQ4_XS) H.d = *(const unsigned short *)(wrow + L.off_b + sb * 8);
    else H.d = *(const unsigned short *)(wrow + L.off_d + sb * 2);
}

template <int TYPE>
__device__ __forceinline__ void kp_fetch_w(kp_w<TYPE> &R, const uint8_t *__restrict__ wrow, const row_layout &L, int64_t sb, int half) {
    const int p = threadIdx.x & 3;
    if constexpr (TYPE == MI355_Q4_K) {
        const uint8_t *blk = wrow + sb * Q4_K_BYTES;
        R.q = load16(blk + 16 + (half * 2 + (p >> 1)) * 32 + (p & 1) * 16);
    } else if constexpr (TYPE == MI355_Q5_K) {   // the Q4_K geometry behind 32 bytes of fifth bits (bit j of qh[l]: sub-block j, level l)
        const uint8_t *blk = wrow + sb * Q5_K_BYTES;
        R.q = load16(blk + 48 + (half * 2 + (p >> 1)) * 32 + (p & 1) * 16);
        R.qh = load16(blk + 16 + (p & 1) * 16);
    } else if constexpr (TYPE == MI355_IQ4_XS) {   // block 4 half + p: 16 bytes of table indices, its six-bit scale from the header
        const int ib = half * 4 + p;
        R.q = load16(wrow + sb * 128 + ib * 16);
        const uint2 h = *(const uint2 *)(wrow + L.off_b + sb * 8);
        R.ls = (int)(((h.y >> (4 * ib)) & 0xFu) | (((h.x >> (16 + 2 * ib)) & 3u) << 4)) - 32;
    } else {
        const int l0 = 16 * (p & 1), qa = p >> 1;
        R.ql = load16(wrow + sb * 128 + half * 64 + p * 16);
        R.qh = load16(wrow + L.off_b + sb * 64 + half * 32 + l0);
        const int8_t *sc = (const int8_t *)(wrow + L.off_c + sb * 16 + half * 8 + (l0 >> 4));
        R.scA = sc[2 * qa];
        R.scB = sc[2 * qa + 4];
    }
}

// unpacked planes of the piece: two 16-byte chunks per plane
struct kp_planes { u32x4 a1, a0, b1, b0; };

// dword i of the piece -> dword i of the four plane chunks
template <int TYPE>
__device__ __forceinline__ void kp_unpack(const kp_w<TYPE> &R, const kp_h<TYPE> &H, int half, int i, kp_planes &P) {
    const int p = threadIdx.x & 3;
    if constexpr (TYPE == MI355_Q4_K) {
        const int gl = p >> 1;
        int scl, mnl, sch, mnh;
        q4k_scale_min(H.hdr[1], H.hdr[2], H.hdr[3], half * 4 + 2 * gl, scl, mnl);
        q4k_scale_min(H.hdr[1], H.hdr[2], H.hdr[3], half * 4 + 2 * gl + 1, sch, mnh);
        const u32 nl = R.q[i] & 0x0F0F0F0Fu, nh = (R.q[i] >> 4) & 0x0F0F0F0Fu;
        P.a1[i] = mul_bytes(nl, (u32)scl >> 3);
        P.a0[i] = mul_bytes(nl, (u32)scl & 7u);
        P.b1[i] = mul_bytes(nh, (u32)sch >> 3);
        P.b0[i] = mul_bytes(nh, (u32)sch & 7u);
    } else if constexpr (TYPE == MI355_Q5_K) {
        const int g = half * 2 + (p >> 1);
        int scl, mnl, sch, mnh;
        q4k_scale_min(H.hdr[1], H.hdr[2], H.hdr[3], 2 * g, scl, mnl);
        q4k_scale_min(H.hdr[1], H.hdr[2], H.hdr[3], 2 * g + 1, sch, mnh);
        const u32 nl = (R.q[i] & 0x0F0F0F0Fu) | (((R.qh[i] >> (2 * g)) & 0x01010101u) << 4);
        const u32 nh = ((R.q[i] >> 4) & 0x0F0F0F0Fu) | (((R.qh[i] >> (2 * g + 1)) & 0x01010101u) << 4);
        u32 hi, lo;
        q5k_planes(nl, scl, hi, lo);
        P.a1[i] = hi; P.a0[i] = lo;
        q5k_planes(nh, sch, hi, lo);
        P.b1[i] = hi; P.b0[i] = lo;
    } else if constexpr (TYPE == MI355_IQ4_XS) {
        u32 hi, lo;
        iq4xs_planes(iq4nl_lookup4(R.q[i] & 0x0F0F0F0Fu), R.ls, hi, lo);
        P.a1[i] = hi; P.a0[i] = lo;
        iq4xs_planes(iq4nl_lookup4((R.q[i] >> 4) & 0x0F0F0F0Fu), R.ls, hi, lo);
        P.b1[i] = hi; P.b0[i] = lo;
    } else {
        const int qa = p >> 1;
        const u32 va = (R.ql[i] & 0x0F0F0F0Fu) | (((R.qh[i] >> (2 * qa)) & 0x03030303u) << 4);
        const u32 vb = ((R.ql[i] >> 4) & 0x0F0F0F0Fu) | (((R.qh[i] >> (2 * qa + 4)) & 0x03030303u) << 4);
        u32 hi, lo;
        q6k_planes(va, R.scA, hi, lo);
        P.a1[i] = hi; P.a0[i] = lo;
        q6k_planes(vb, R.scB, hi, lo);
        P.b1[i] = hi; P.b0[i] = lo;
    }
}

template <int TYPE>
__device__ __forceinline__ void kp_store(const kp_planes &P, int8_t *__restrict__ sW1, int8_t *__restrict__ sW0) {
    const int r = threadIdx.x >> 2, p = threadIdx.x & 3;
    // Q4_K: low nibbles are sub-block 2*gl, high nibbles sub-block 2*gl + 1 (32 bytes later); Q6_K: the second group is 64 bytes later
    // (Q5_K as Q4_K; IQ4_XS: the two halves of block p follow each other)
    const int c0 = kp_form<TYPE>::MIN ? 4 * (p >> 1) + (p & 1) : TYPE == MI355_IQ4_XS ? 2 * p : 2 * (p >> 1) + (p & 1);
    const int c1 = c0 + (kp_form<TYPE>::MIN ? 2 : TYPE == MI355_IQ4_XS ? 1 : 4);
    *(u32x4 *)(sW1 + kp_off(r, c0)) = P.a1;
    *(u32x4 *)(sW0 + kp_off(r, c0)) = P.a0;
    *(u32x4 *)(sW1 + kp_off(r, c1)) = P.b1;
    *(u32x4 *)(sW0 + kp_off(r, c1)) = P.b0;
}

// activations of one stage: 32 * AI rows x 128 bytes, AI wave-wide 16-byte transfers per wave.  aofs: per-lane byte offsets of
// the 16 bytes this lane moves (row * K + swizzled chunk, fixed for the whole kernel); base: uniform pointer to the stage.
template <int AI>
__device__ __forceinline__ void kp_dma_a(const int8_t *__restrict__ base, const unsigned (&aofs)[AI], int8_t *__restrict__ sA) {
    const int wave = threadIdx.x >> 6;
#pragma unroll
    for (int it = 0; it < AI; it++)
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)(base + aofs[it]),
                                         (void __attribute__((address_space(3))) *)(sA + (wave * AI + it) * 1024), 16, 0, 0);
}
// row of transfer `it` of this lane and the logical chunk that belongs at the lane's LDS position
template <int AI>
__device__ __forceinline__ void kp_dma_slot(int it, int &row, int &chunk) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    row = (wave * AI + it) * 8 + (lane >> 3);
    chunk = (lane & 7) ^ ((row >> 1) & 7);
}

template <int TYPE, bool ID>
__global__ void __launch_bounds__(256, 2) k_mmq_kp(const uint8_t *__restrict__ W, const int8_t *__restrict__ aq, const float *__restrict__ ad8,
                                                   const _Float16 *__restrict__ abs_, float *dst, const float *residual,
                                                   int64_t N, int64_t K, int64_t B, int64_t dst_stride, row_layout L, int n_col_tiles,
                                                   int n_groups, int n_groups_padded, mmq_route route) {
    constexpr bool Q4 = kp_form<TYPE>::MIN;   // the form with a min term (Q4_K, Q5_K)
    constexpr int RADIX_SHIFT = kp_form<TYPE>::RADIX_SHIFT;
    constexpr int BM = 64, BN = 128;
    __shared__ __attribute__((aligned(16))) int8_t sW1a[BM * KP_ROW], sW1b[BM * KP_ROW];
    __shared__ __attribute__((aligned(16))) int8_t sW0a[BM * KP_ROW], sW0b[BM * KP_ROW];
    __shared__ __attribute__((aligned(16))) int8_t sAa[BN * KP_ROW], sAb_[BN * KP_ROW];
    __shared__ __attribute__((aligned(16))) float sWd[2][BM];
    __shared__ __attribute__((aligned(16))) float sWn[2][Q4 ? BM : 4];
    __shared__ __attribute__((aligned(16))) _Float16 sWm[2][Q4 ? BM * 16 : 8];
    __shared__ __attribute__((aligned(16))) float sAd[2][BN];
    __shared__ __attribute__((aligned(16))) _Float16 sAs[2][Q4 ? BN * 16 : 8];
    // sAa / sAb_ are written by global-to-LDS transfers only; a transfer names the wave's first 16 bytes, so to the compiler most
    // of these arrays is never stored to.  The empty asm makes them memory that unknown code may have written.
    asm volatile("" ::"v"((void *)sAa), "v"((void *)sAb_) : "memory");

    const int per_xcd = n_groups_padded >> 3;
    const int lid = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (lid >= n_groups) return;
    const int64_t row0 = (int64_t)(lid / n_col_tiles) * BM;
    int64_t col0 = (int64_t)(lid % n_col_tiles) * BN;
    if constexpr (ID) {
        const int ct = lid % n_col_tiles;
        if (ct >= *route.n_tiles) return;
        W += (int64_t)route.tiles[4 * ct] * route.expert_bytes;
        col0 = route.tiles[4 * ct + 1];
        B = route.tiles[4 * ct + 2];
    }

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    const int wrow0 = (wave & 1) * 32;    // weight rows of this wave inside the tile
    const int wcol0 = (wave >> 1) * 64;   // activation rows of this wave inside the tile
    const int64_t nsb = K >> 8;
    // split K: group y of gridDim.y walks super-blocks [sb_lo, sb_hi) and writes its sums to its own slice of `dst` (see launch)
    const int64_t sb_per = (nsb + gridDim.y - 1) / gridDim.y;
    const int64_t sb_lo = (int64_t)blockIdx.y * sb_per, sb_hi = sb_lo + sb_per < nsb ? sb_lo + sb_per : nsb;
    if (gridDim.y > 1) {
        dst += (int64_t)blockIdx.y * B * dst_stride;
        residual = nullptr;
    }

    // this thread's weight row, the activation rows of its four transfers, and the column whose scales it copies
    const int64_t wr = row0 + (tid >> 2) < N ? row0 + (tid >> 2) : N - 1;
    const uint8_t *wrow = W + wr * L.row_bytes;
    unsigned aofs[4];
#pragma unroll
    for (int it = 0; it < 4; it++) {
        int r, c;
        kp_dma_slot<4>(it, r, c);
        const int64_t col = col0 + r;
        const int64_t cc = col < B ? col : B - 1;
        aofs[it] = (unsigned)((int64_t)(ID ? route.act_row[cc] : (int)cc) * K + c * 16);
    }
    int srow;
    {
        const int64_t col = col0 + (tid >> 1);
        const int64_t cc = col < B ? col : B - 1;
        srow = ID ? route.act_row[cc] : (int)cc;
    }

    f32x16 acc[2];
#pragma unroll
    for (int tb = 0; tb < 2; tb++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[tb][r] = 0.0f;

    // per super-block scales of the weights come with the piece (Q4_K header / Q6_K d); those of the activations are fetched
    // by two threads per column: 16 bytes of the sub-block sums each, the even thread also the scale
    auto fetch_scales = [&](int64_t sb, float &d8, u32x4 &bs) {
        d8 = ad8[(int64_t)srow * nsb + sb];
        if constexpr (Q4) bs = *(const u32x4 *)(abs_ + ((int64_t)srow * nsb + sb) * 16 + 8 * (tid & 1));
    };
    auto store_scales = [&](int sbuf, float d8, const u32x4 &bs, const kp_h<TYPE> &H) {
        sAd[sbuf][tid >> 1] = d8;   // both threads of the column write the same value: an unconditional use keeps the load where it was issued
        if constexpr (Q4) {
            *(u32x4 *)(sAs[sbuf] + (tid >> 1) * 16 + 8 * (tid & 1)) = bs;
            // the four threads of a row share the work (and all use the header, so its load stays where it was issued):
            // each writes d, dmin (same values) and the mins of sub-blocks 2p, 2p + 1
            const int r = tid >> 2, p2 = 2 * (tid & 3);
            sWd[sbuf][r] = half_bits_to_float((unsigned short)(H.hdr[0] & 0xFFFFu));
            sWn[sbuf][r] = half_bits_to_float((unsigned short)(H.hdr[0] >> 16));
            int sc, mn0, mn1;
            q4k_scale_min(H.hdr[1], H.hdr[2], H.hdr[3], p2, sc, mn0);
            q4k_scale_min(H.hdr[1], H.hdr[2], H.hdr[3], p2 + 1, sc, mn1);
            typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
            const f16x2 m1 = {(_Float16)(float)mn0, (_Float16)(float)mn1};
            const f16x2 m64 = {(_Float16)(float)(64 * mn0), (_Float16)(float)(64 * mn1)};
            *(f16x2 *)(sWm[sbuf] + r * 16 + p2) = m1;
            *(f16x2 *)(sWm[sbuf] + r * 16 + 8 + p2) = m64;
        } else {
            sWd[sbuf][tid >> 2] = half_bits_to_float(H.d);   // the four threads of a row write the same value
        }
    };

    kp_w<TYPE> R0, R1;   // pieces of the even / odd stages
    kp_h<TYPE> Hc, Hn;   // super-block data in use / of the next super-block
    float d8n = 0.0f;
    u32x4 bsn = {0, 0, 0, 0};
    // prologue: stage 0 into the "a" buffers, pieces of stage 1 in flight
    kp_fetch_w<TYPE>(R0, wrow, L, sb_lo, 0);
    kp_fetch_w<TYPE>(R1, wrow, L, sb_lo, 1);
    kp_fetch_h<TYPE>(Hc, wrow, L, sb_lo);
    kp_dma_a<4>(aq + sb_lo * QKK, aofs, sAa);
    fetch_scales(sb_lo, d8n, bsn);
    {
        kp_planes P;
#pragma unroll
        for (int i = 0; i < 4; i++) kp_unpack<TYPE>(R0, Hc, 0, i, P);
        kp_store<TYPE>(P, sW1a, sW0a);
        store_scales(0, d8n, bsn, Hc);
    }
    Hn = Hc;
    __syncthreads();

    for (int64_t sb = sb_lo; sb < sb_hi; sb++) {
        i32x16 hi[2], lo[2];
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const int8_t *cA = half == 0 ? sAa : sAb_;
            const int8_t *cW1 = half == 0 ? sW1a : sW1b;
            const int8_t *cW0 = half == 0 ? sW0a : sW0b;
            int8_t *nA = half == 0 ? sAb_ : sAa;
            int8_t *nW1 = half == 0 ? sW1b : sW1a;
            int8_t *nW0 = half == 0 ? sW0b : sW0a;
            kp_w<TYPE> &Rn = half == 0 ? R1 : R0;    // piece of the next stage: unpacked during this one
            kp_w<TYPE> &Rf = half == 0 ? R0 : R1;    // held this stage's piece (unpacked one stage ago): refilled for the stage after next
            // Past the end of K the same work is done on the last super-block again and never read: no branches in the stage,
            // so the compiler schedules it as one block.
            const int64_t sb1 = sb + 1 < sb_hi ? sb + 1 : sb;
            kp_dma_a<4>(aq + (half == 0 ? sb * QKK + 128 : sb1 * QKK), aofs, nA);
            if (half == 1) fetch_scales(sb1, d8n, bsn);
            kp_fetch_w<TYPE>(Rf, wrow, L, sb1, half);
            if (half == 0) kp_fetch_h<TYPE>(Hn, wrow, L, sb1);   // used from the next stage on
            __builtin_amdgcn_sched_barrier(0);   // the loads stay here, a whole stage ahead of their first use

            kp_planes P;
            i32x4 af[2][2], b1[2], b0[2];
            auto load_frags = [&](int ks, int slot) {
#pragma unroll
                for (int tb = 0; tb < 2; tb++) af[slot][tb] = *(const i32x4 *)(cA + kp_off(wcol0 + tb * 32 + l32, ks * 2 + lhi));
                b1[slot] = *(const i32x4 *)(cW1 + kp_off(wrow0 + l32, ks * 2 + lhi));
                b0[slot] = *(const i32x4 *)(cW0 + kp_off(wrow0 + l32, ks * 2 + lhi));
            };
            load_frags(0, 0);
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                if (ks < 3) load_frags(ks + 1, (ks + 1) & 1);   // operands of the next step are in flight during this step's matrix instructions
                const int sl = ks & 1;
#pragma unroll
                for (int tb = 0; tb < 2; tb++) {
                    if (half == 0 && ks == 0) {
                        i32x16 z;
#pragma unroll
                        for (int r = 0; r < 16; r++) z[r] = 0;
                        hi[tb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[sl][tb], b1[sl], z, 0, 0, 0);
                        lo[tb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[sl][tb], b0[sl], z, 0, 0, 0);
                    } else {
                        hi[tb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[sl][tb], b1[sl], hi[tb], 0, 0, 0);
                        lo[tb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[sl][tb], b0[sl], lo[tb], 0, 0, 0);
                    }
                }
                kp_unpack<TYPE>(Rn, half == 0 ? Hc : Hn, half ^ 1, ks, P);   // a quarter of the next stage's piece between the matrix instructions
            }
            kp_store<TYPE>(P, nW1, nW0);

            if (half == 1) {   // end of the super-block: scale the integer sums into the f32 accumulators
                const int sbuf = (int)((sb - sb_lo) & 1);
#pragma unroll
                for (int tb = 0; tb < 2; tb++) {
                    f32x4 d8[4];
#pragma unroll
                    for (int q = 0; q < 4; q++) d8[q] = *(const f32x4 *)(sAd[sbuf] + wcol0 + tb * 32 + 8 * q + 4 * lhi);
                    const int wr_ = wrow0 + l32;
                    const float dw = sWd[sbuf][wr_];
                    if constexpr (Q4) {
                        const float dn = sWn[sbuf][wr_];
                        const f16x8 am = *(const f16x8 *)(sAs[sbuf] + (wcol0 + tb * 32 + l32) * 16 + 8 * lhi);
                        const f16x8 bm = *(const f16x8 *)(sWm[sbuf] + wr_ * 16 + 8 * lhi);
                        f32x16 z;
#pragma unroll
                        for (int r = 0; r < 16; r++) z[r] = 0.0f;
                        const f32x16 M = __builtin_amdgcn_mfma_f32_32x32x16_f16(am, bm, z, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const int t = (hi[tb][r] << RADIX_SHIFT) + lo[tb][r];
                            acc[tb][r] += d8[r >> 2][r & 3] * (dw * (float)t - dn * M[r]);
                        }
                    } else {
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const int t = (hi[tb][r] << RADIX_SHIFT) + lo[tb][r];
                            acc[tb][r] += d8[r >> 2][r & 3] * (dw * (float)t);
                        }
                    }
                }
            }
            if (half == 1) {   // last, so that the loads had the whole stage (the barrier keeps the scheduler from hoisting the wait)
                __builtin_amdgcn_sched_barrier(0);
                store_scales((int)((sb - sb_lo + 1) & 1), d8n, bsn, Hn);
                Hc = Hn;
            }
            __syncthreads();   // also waits for this stage's transfers and loads (issued a whole stage ago)
        }
    }

#pragma unroll
    for (int tb = 0; tb < 2; tb++) {
        const int64_t n = row0 + wrow0 + l32;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int64_t b = col0 + wcol0 + tb * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
            if (n < N && b < B) {
                const int64_t o = (ID ? (int64_t)route.dst_row[b] : b) * dst_stride + n;
                dst[o] = residual ? acc[tb][r] + residual[o] : acc[tb][r];   // residual may be dst itself: one reader and writer per element
            }
        }
    }
}

// ---- planes kept in HBM ----------------------------------------------------------------------------------------------------
// The vector ALU is what limits k_mmq_kp (about 11 instructions per matrix instruction, 4 of them the unpack).  With 288 GB of
// HBM a second, unpacked copy of the K-quant weights is affordable (2 bytes per weight: the two int8 planes, written once by
// k_unpack_planes when the weights are uploaded): k_mmq_pl brings both planes of a stage from global memory straight into
// LDS, like the activations, and spends no vector instruction on the weights.  The packed copy stays the one the GEMV
// streams.  planes: int8 hi[N][K], int8 lo[N][K], then 48 bytes per (row, super-block): the eight mins as f16, the eight mins
// times 64 as f16 (the two operand rows of the min-term matrix instruction), and {d, dmin} as f32.
template <int TYPE>
__global__ void __launch_bounds__(256) k_unpack_planes(const uint8_t *__restrict__ W, int8_t *__restrict__ planes, int64_t N, int64_t K,
                                                       row_layout L) {
    // one thread per 16-byte piece: row, super-block, half, piece = the unpack of k_mmq_kp
    const int64_t per_row = (K >> 8) * 8;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= N * per_row) return;
    const int64_t row = idx / per_row, rem = idx % per_row, sb = rem >> 3;
    const int half = (int)((rem >> 2) & 1), p = (int)(rem & 3);
    const uint8_t *wrow = W + row * L.row_bytes;
    u32x4 a1, a0, b1, b0;
    int c0, c1;
    if constexpr (TYPE == MI355_Q4_K) {
        const uint8_t *blk = wrow + sb * Q4_K_BYTES;
        const u32x4 q = load16(blk + 16 + (half * 2 + (p >> 1)) * 32 + (p & 1) * 16);
        const u32x4 hdr = load16(blk);
        const int gl = p >> 1;
        int scl, mnl, sch, mnh;
        q4k_scale_min(hdr[1], hdr[2], hdr[3], half * 4 + 2 * gl, scl, mnl);
        q4k_scale_min(hdr[1], hdr[2], hdr[3], half * 4 + 2 * gl + 1, sch, mnh);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const u32 nl = q[i] & 0x0F0F0F0Fu, nh = (q[i] >> 4) & 0x0F0F0F0Fu;
            a1[i] = mul_bytes(nl, (u32)scl >> 3);
            a0[i] = mul_bytes(nl, (u32)scl & 7u);
            b1[i] = mul_bytes(nh, (u32)sch >> 3);
            b0[i] = mul_bytes(nh, (u32)sch & 7u);
        }
        c0 = 4 * gl + (p & 1);
        c1 = c0 + 2;
    } else {
        const int l0 = 16 * (p & 1), qa = p >> 1;
        const u32x4 ql = load16(wrow + sb * 128 + half * 64 + p * 16);
        const u32x4 qh = load16(wrow + L.off_b + sb * 64 + half * 32 + l0);
        const int8_t *sc = (const int8_t *)(wrow + L.off_c + sb * 16 + half * 8 + (l0 >> 4));
        const int scA = sc[2 * qa], scB = sc[2 * qa + 4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const u32 va = (ql[i] & 0x0F0F0F0Fu) | (((qh[i] >> (2 * qa)) & 0x03030303u) << 4);
            const u32 vb = ((ql[i] >> 4) & 0x0F0F0F0Fu) | (((qh[i] >> (2 * qa + 4)) & 0x03030303u) << 4);
            u32 hi, lo;
            q6k_planes(va, scA, hi, lo);
            a1[i] = hi; a0[i] = lo;
            q6k_planes(vb, scB, hi, lo);
            b1[i] = hi; b0[i] = lo;
        }
        c0 = 2 * qa + (p & 1);
        c1 = c0 + 4;
    }
    if (half == 0 && p == 0) {   // the row's per-super-block data behind the planes: three 16-byte chunks
        u32x4 *aux = (u32x4 *)(planes + 2 * N * K) + (row * (K >> 8) + sb) * 3;
        if constexpr (TYPE == MI355_Q4_K) {
            const u32x4 hdr = load16(wrow + sb * Q4_K_BYTES);
            f16x8 m1, m64;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                int sc, mn;
                q4k_scale_min(hdr[1], hdr[2], hdr[3], j, sc, mn);
                m1[j] = (_Float16)(float)mn;
                m64[j] = (_Float16)(float)(64 * mn);
            }
            aux[0] = __builtin_bit_cast(u32x4, m1);
            aux[1] = __builtin_bit_cast(u32x4, m64);
            const float d = half_bits_to_float((unsigned short)(hdr[0] & 0xFFFFu)), dmin = half_bits_to_float((unsigned short)(hdr[0] >> 16));
            aux[2] = u32x4{__builtin_bit_cast(u32, d), __builtin_bit_cast(u32, dmin), 0u, 0u};
        } else {
            const float d = half_bits_to_float(*(const unsigned short *)(wrow + L.off_d + sb * 2));
            aux[0] = u32x4{0u, 0u, 0u, 0u};
            aux[1] = u32x4{0u, 0u, 0u, 0u};
            aux[2] = u32x4{__builtin_bit_cast(u32, d), 0u, 0u, 0u};
        }
    }
    int8_t *hi = planes + row * K + sb * QKK + half * 128, *lo = hi + N * K;
    *(u32x4 *)(hi + c0 * 16) = a1;
    *(u32x4 *)(lo + c0 * 16) = a0;
    *(u32x4 *)(hi + c1 * 16) = b1;
    *(u32x4 *)(lo + c1 * 16) = b0;
}

// what a thread of k_mmq_pl moves per super-block from the 48-byte entry k_unpack_planes wrote behind the planes to LDS: thread
// p of the four that share a row takes the mins of sub-blocks 2p, 2p + 1 (plain and times 64, ready as f16) and {d, dmin}.
// Only bytes that are used are loaded: a loaded register that is dead gets reused at once, and that write waits for the load.
template <int TYPE> struct pl_h { u32 v[TYPE == MI355_Q4_K ? 4 : 1]; };
template <int TYPE>
__device__ __forceinline__ void pl_fetch_h(pl_h<TYPE> &H, const u32 *__restrict__ aux_row, int64_t sb) {
    const u32 *a = aux_row + sb * 12;
    if constexpr (TYPE == MI355_Q4_K) {
        const int p = threadIdx.x & 3;
        H.v[0] = a[p];
        H.v[1] = a[4 + p];
        H.v[2] = a[8];
        H.v[3] = a[9];
    } else {
        H.v[0] = a[8];
    }
}

template <int TYPE, bool ID>
__global__ void __launch_bounds__(256, 2) k_mmq_pl(const int8_t *__restrict__ planes, const int8_t *__restrict__ aq, const float *__restrict__ ad8,
                                                   const _Float16 *__restrict__ abs_, float *dst, const float *residual,
                                                   int64_t N, int64_t K, int64_t B, int64_t dst_stride, row_layout L, int n_col_tiles,
                                                   int n_groups, int n_groups_padded, mmq_route route, int64_t plane_stride) {
    constexpr bool Q4 = TYPE == MI355_Q4_K;
    constexpr int RADIX_SHIFT = Q4 ? 3 : 6;
    constexpr int BM = 64, BN = 128;
    __shared__ __attribute__((aligned(16))) int8_t sW1a[BM * KP_ROW], sW1b[BM * KP_ROW];
    __shared__ __attribute__((aligned(16))) int8_t sW0a[BM * KP_ROW], sW0b[BM * KP_ROW];
    __shared__ __attribute__((aligned(16))) int8_t sAa[BN * KP_ROW], sAb_[BN * KP_ROW];
    __shared__ __attribute__((aligned(16))) float sWd[2][BM];
    __shared__ __attribute__((aligned(16))) float sWn[2][Q4 ? BM : 4];
    __shared__ __attribute__((aligned(16))) _Float16 sWm[2][Q4 ? BM * 16 : 8];
    __shared__ __attribute__((aligned(16))) float sAd[2][BN];
    __shared__ __attribute__((aligned(16))) _Float16 sAs[2][Q4 ? BN * 16 : 8];
    // The tile buffers are written by global-to-LDS transfers only; a transfer names the wave's first 16 bytes, so to the compiler
    // most of these arrays is never stored to.  The empty asm makes them memory that unknown code may have written.
    asm volatile("" ::"v"((void *)sAa), "v"((void *)sAb_), "v"((void *)sW1a), "v"((void *)sW1b), "v"((void *)sW0a), "v"((void *)sW0b) : "memory");

    const int per_xcd = n_groups_padded >> 3;
    const int lid = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (lid >= n_groups) return;
    const int64_t row0 = (int64_t)(lid / n_col_tiles) * BM;
    int64_t col0 = (int64_t)(lid % n_col_tiles) * BN;
    int64_t plane_base = 0;
    if constexpr (ID) {
        const int ct = lid % n_col_tiles;
        if (ct >= *route.n_tiles) return;
        plane_base = (int64_t)route.tiles[4 * ct] * N * K;
        col0 = route.tiles[4 * ct + 1];
        B = route.tiles[4 * ct + 2];
    }

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    const int wrow0 = (wave & 1) * 32;    // weight rows of this wave inside the tile
    const int wcol0 = (wave >> 1) * 64;   // activation rows of this wave inside the tile
    const int64_t nsb = K >> 8;
    // split K: group y of gridDim.y walks super-blocks [sb_lo, sb_hi) and writes its sums to its own slice of `dst` (see launch)
    const int64_t sb_per = (nsb + gridDim.y - 1) / gridDim.y;
    const int64_t sb_lo = (int64_t)blockIdx.y * sb_per, sb_hi = sb_lo + sb_per < nsb ? sb_lo + sb_per : nsb;
    if (gridDim.y > 1) {
        dst += (int64_t)blockIdx.y * B * dst_stride;
        residual = nullptr;
    }

    // this thread's weight row, the activation rows of its four transfers, and the column whose scales it copies
    const int64_t wr = row0 + (tid >> 2) < N ? row0 + (tid >> 2) : N - 1;
    const u32 *aux_row = (const u32 *)(planes + 2 * plane_stride) + (plane_base / K + wr) * nsb * 12;   // per-super-block data of the row
    // per-lane byte offsets of this thread's two plane transfers per stage (row * K + swizzled chunk)
    unsigned pofs[2];
#pragma unroll
    for (int it = 0; it < 2; it++) {
        int r, c;
        kp_dma_slot<2>(it, r, c);
        const int64_t gr = row0 + r < N ? row0 + r : N - 1;
        pofs[it] = (unsigned)(gr * K + c * 16);
    }
    const int8_t *plane1 = planes + plane_base, *plane0 = plane1 + plane_stride;
    unsigned aofs[4];
#pragma unroll
    for (int it = 0; it < 4; it++) {
        int r, c;
        kp_dma_slot<4>(it, r, c);
        const int64_t col = col0 + r;
        const int64_t cc = col < B ? col : B - 1;
        aofs[it] = (unsigned)((int64_t)(ID ? route.act_row[cc] : (int)cc) * K + c * 16);
    }
    int srow;
    {
        const int64_t col = col0 + (tid >> 1);
        const int64_t cc = col < B ? col : B - 1;
        srow = ID ? route.act_row[cc] : (int)cc;
    }

    f32x16 acc[2];
#pragma unroll
    for (int tb = 0; tb < 2; tb++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[tb][r] = 0.0f;

    // per super-block scales of the weights come with the piece (Q4_K header / Q6_K d); those of the activations are fetched
    // by two threads per column: 16 bytes of the sub-block sums each, the even thread also the scale
    auto fetch_scales = [&](int64_t sb, float &d8, u32x4 &bs) {
        d8 = ad8[(int64_t)srow * nsb + sb];
        if constexpr (Q4) bs = *(const u32x4 *)(abs_ + ((int64_t)srow * nsb + sb) * 16 + 8 * (tid & 1));
    };
    auto store_scales = [&](int sbuf, float d8, const u32x4 &bs, const pl_h<TYPE> &H) {
        sAd[sbuf][tid >> 1] = d8;   // both threads of the column write the same value: an unconditional use keeps the load where it was issued
        if constexpr (Q4) {
            *(u32x4 *)(sAs[sbuf] + (tid >> 1) * 16 + 8 * (tid & 1)) = bs;
            // the four threads of a row: each writes d, dmin (same values) and the f16 mins of sub-blocks 2p, 2p + 1
            const int r = tid >> 2, p = tid & 3;
            ((u32 *)sWm[sbuf])[r * 8 + p] = H.v[0];
            ((u32 *)sWm[sbuf])[r * 8 + 4 + p] = H.v[1];
            sWd[sbuf][r] = __builtin_bit_cast(float, H.v[2]);
            sWn[sbuf][r] = __builtin_bit_cast(float, H.v[3]);
        } else {
            sWd[sbuf][tid >> 2] = __builtin_bit_cast(float, H.v[0]);   // the four threads of a row write the same value
        }
    };

    pl_h<TYPE> Hc, Hn;   // super-block data in use / of the next super-block
    float d8n = 0.0f;
    u32x4 bsn = {0, 0, 0, 0};
    // both planes of a stage: 64 rows x 128 bytes each, two wave-wide transfers per wave and plane, swizzled like the activations
    auto dma_w = [&](int64_t k0, int8_t *s1, int8_t *s0) {
        kp_dma_a<2>(plane1 + k0, pofs, s1);
        kp_dma_a<2>(plane0 + k0, pofs, s0);
    };
    // prologue: stage 0 into the "a" buffers
    pl_fetch_h<TYPE>(Hc, aux_row, sb_lo);
    kp_dma_a<4>(aq + sb_lo * QKK, aofs, sAa);
    dma_w(sb_lo * QKK, sW1a, sW0a);
    fetch_scales(sb_lo, d8n, bsn);
    store_scales(0, d8n, bsn, Hc);
    Hn = Hc;
    __syncthreads();

    for (int64_t sb = sb_lo; sb < sb_hi; sb++) {
        i32x16 hi[2], lo[2];
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const int8_t *cA = half == 0 ? sAa : sAb_;
            const int8_t *cW1 = half == 0 ? sW1a : sW1b;
            const int8_t *cW0 = half == 0 ? sW0a : sW0b;
            int8_t *nA = half == 0 ? sAb_ : sAa;
            int8_t *nW1 = half == 0 ? sW1b : sW1a;
            int8_t *nW0 = half == 0 ? sW0b : sW0a;
            // Past the end of K the same work is done on the last super-block again and never read: no branches in the stage.
            const int64_t sb1 = sb + 1 < sb_hi ? sb + 1 : sb;
            const int64_t k1 = half == 0 ? sb * QKK + 128 : sb1 * QKK;   // the next stage
            kp_dma_a<4>(aq + k1, aofs, nA);
            dma_w(k1, nW1, nW0);
            if (half == 1) fetch_scales(sb1, d8n, bsn);
            if (half == 0) pl_fetch_h<TYPE>(Hn, aux_row, sb1);   // used from the next stage on
            __builtin_amdgcn_sched_barrier(0);   // the loads stay here, a whole stage ahead of their first use

            i32x4 af[1][2], b1[1], b0[1];
            auto load_frags = [&](int ks, int slot) {
#pragma unroll
                for (int tb = 0; tb < 2; tb++) af[slot][tb] = *(const i32x4 *)(cA + kp_off(wcol0 + tb * 32 + l32, ks * 2 + lhi));
                b1[slot] = *(const i32x4 *)(cW1 + kp_off(wrow0 + l32, ks * 2 + lhi));
                b0[slot] = *(const i32x4 *)(cW0 + kp_off(wrow0 + l32, ks * 2 + lhi));
            };
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                // one set of operand registers: the second resident group covers the LDS latency, and the registers a second set
                // would take are what keeps this kernel from spilling
                const int sl = 0;
                load_frags(ks, 0);
#pragma unroll
                for (int tb = 0; tb < 2; tb++) {
                    if (half == 0 && ks == 0) {
                        i32x16 z;
#pragma unroll
                        for (int r = 0; r < 16; r++) z[r] = 0;
                        hi[tb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[sl][tb], b1[sl], z, 0, 0, 0);
                        lo[tb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[sl][tb], b0[sl], z, 0, 0, 0);
                    } else {
                        hi[tb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[sl][tb], b1[sl], hi[tb], 0, 0, 0);
                        lo[tb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[sl][tb], b0[sl], lo[tb], 0, 0, 0);
                    }
                }
            }

            if (half == 1) {   // end of the super-block: scale the integer sums into the f32 accumulators
                const int sbuf = (int)((sb - sb_lo) & 1);
#pragma unroll
                for (int tb = 0; tb < 2; tb++) {
                    f32x4 d8[4];
#pragma unroll
                    for (int q = 0; q < 4; q++) d8[q] = *(const f32x4 *)(sAd[sbuf] + wcol0 + tb * 32 + 8 * q + 4 * lhi);
                    const int wr_ = wrow0 + l32;
                    const float dw = sWd[sbuf][wr_];
                    if constexpr (Q4) {
                        const float dn = sWn[sbuf][wr_];
                        const f16x8 am = *(const f16x8 *)(sAs[sbuf] + (wcol0 + tb * 32 + l32) * 16 + 8 * lhi);
                        const f16x8 bm = *(const f16x8 *)(sWm[sbuf] + wr_ * 16 + 8 * lhi);
                        f32x16 z;
#pragma unroll
                        for (int r = 0; r < 16; r++) z[r] = 0.0f;
                        const f32x16 M = __builtin_amdgcn_mfma_f32_32x32x16_f16(am, bm, z, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const int t = (hi[tb][r] << RADIX_SHIFT) + lo[tb][r];
                            acc[tb][r] += d8[r >> 2][r & 3] * (dw * (float)t - dn * M[r]);
                        }
                    } else {
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const int t = (hi[tb][r] << RADIX_SHIFT) + lo[tb][r];
                            acc[tb][r] += d8[r >> 2][r & 3] * (dw * (float)t);
                        }
                    }
                }
            }
            if (half == 1) {   // last, so that the loads had the whole stage (the barrier keeps the scheduler from hoisting the wait)
                __builtin_amdgcn_sched_barrier(0);
                store_scales((int)((sb - sb_lo + 1) & 1), d8n, bsn, Hn);
                Hc = Hn;
            }
            __syncthreads();   // also waits for this stage's transfers and loads (issued a whole stage ago)
        }
    }

#pragma unroll
    for (int tb = 0; tb < 2; tb++) {
        const int64_t n = row0 + wrow0 + l32;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int64_t b = col0 + wcol0 + tb * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
            if (n < N && b < B) {
                const int64_t o = (ID ? (int64_t)route.dst_row[b] : b) * dst_stride + n;
                dst[o] = residual ? acc[tb][r] + residual[o] : acc[tb][r];   // residual may be dst itself: one reader and writer per element
            }
        }
    }
}

// ---- split K --------------------------------------------------------------------------------------------------------
// A product with few tiles (wk / wv of a 512-token batch: 64; any matrix at batch 64: N / 64) leaves most of the chip idle
// while each group walks all of K, one dependent stage after the other.  Such launches are cut along K: grid row y takes a
// contiguous range of super-blocks and writes its sums to slice y of a workspace, and k_split_sum adds the slices in fixed
// order (plus the residual).  The same rule serves the kernel that unpacks and the one that reads planes, so they still
// agree bit for bit.  At least two super-blocks per slice, at most eight slices, at most two groups per compute unit.
static int split_k_slices(int64_t N, int64_t K, int64_t B) {
    const int64_t groups = ((N + 63) / 64) * ((B + 127) / 128), nsb = K / QKK;
    if (groups >= 384) return 1;
    if (groups >= 192 && nsb < 32) return 1;   // about a group per compute unit already: the extra pass over the sums pays only for a long K
    int64_t n = 512 / groups;
    if (n > nsb / 2) n = nsb / 2;
    if (n > 8) n = 8;
    if (n < 2) return 1;
    const int64_t per = (nsb + n - 1) / n;
    return (int)((nsb + per - 1) / per);   // no empty slice
}

__global__ void __launch_bounds__(256) k_split_sum(const float *__restrict__ part, float *__restrict__ dst, const float *__restrict__ residual,
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

// slices for this product given the workspace at hand (1 = no split)
static int usable_slices(int64_t N, int64_t K, int64_t B, const void *ws, size_t ws_bytes) {
    const int n = split_k_slices(N, K, B);
    if (n < 2 || ws == nullptr || ((uintptr_t)ws & 15) != 0 || N % 4 != 0) return 1;
    return ws_bytes >= (size_t)n * (size_t)N * (size_t)B * sizeof(float) ? n : 1;
}

static void launch_split_sum(hipStream_t s, const float *part, float *dst, const float *residual, int64_t N, int64_t B, int64_t dst_stride, int n) {
    MI355_LAUNCH(k_split_sum, dim3((unsigned)((N * B / 4 + 255) / 256)), dim3(256), 0, s, part, dst, residual, N, B, dst_stride, n);
}

template <int TYPE>
static void launch_mmq_k(hipStream_t s, const void *W, const void *act, float *dst, const float *residual, int64_t N, int64_t K, int64_t B,
                         int64_t dst_stride, void *ws, size_t ws_bytes) {
    constexpr int BM = 64, BN = 128;
    const row_layout L = make_row_layout(TYPE, K);
    const int8_t *aq = (const int8_t *)act;
    const float *ad8 = (const float *)(aq + q8k_d_offset(K, B));
    const _Float16 *abs_ = (const _Float16 *)(aq + q8k_bs_offset(K, B));
    const int n_row_tiles = (int)((N + BM - 1) / BM);
    const int n_col_tiles = (int)((B + BN - 1) / BN);
    const int n_groups = n_row_tiles * n_col_tiles;
    const int n_groups_padded = (n_groups + 7) & ~7;
    const int n_slices = usable_slices(N, K, B, ws, ws_bytes);
    if (n_slices > 1) {
        MI355_LAUNCH((k_mmq_kp<TYPE, false>), dim3((unsigned)n_groups_padded, (unsigned)n_slices), dim3(256), 0, s, (const uint8_t *)W, aq, ad8, abs_,
                           (float *)ws, nullptr, N, K, B, N, L, n_col_tiles, n_groups, n_groups_padded, mmq_route{});
        launch_split_sum(s, (const float *)ws, dst, residual, N, B, dst_stride, n_slices);
        return;
    }
    MI355_LAUNCH((k_mmq_kp<TYPE, false>), dim3((unsigned)n_groups_padded), dim3(256), 0, s, (const uint8_t *)W, aq, ad8, abs_, dst, residual, N, K,
                       B, dst_stride, L, n_col_tiles, n_groups, n_groups_padded, mmq_route{});
}

// ---- MUL_MAT_ID with many slots: sort the slots by expert, then one tile launch over all experts ----
constexpr int ROUTE_MAX_EXPERTS = 256;

// One 1024-thread group.  Slot s = t * n_used + e reads activation row t * nb1 + e % nb1 and writes dst row s
// (ggml_compute_forward_mul_mat_id, ggml-cpu.c:7717-7895).  The order of the slots inside an expert depends on
// atomic arrival, the result of every slot does not.
__global__ void __launch_bounds__(1024) k_route_slots(const int32_t *__restrict__ ids, int64_t ids_stride, int64_t n_expert, int64_t n_used,
                                                      int64_t nb1, int64_t T, int bn, int32_t *__restrict__ act_row,
                                                      int32_t *__restrict__ dst_row, int32_t *__restrict__ tiles, int32_t *__restrict__ n_tiles) {
    __shared__ int cnt[ROUTE_MAX_EXPERTS], first[ROUTE_MAX_EXPERTS], cursor[ROUTE_MAX_EXPERTS];
    const int tid = threadIdx.x;
    const int64_t S = T * n_used;
    for (int i = tid; i < n_expert; i += 1024) { cnt[i] = 0; cursor[i] = 0; }
    __syncthreads();
    for (int64_t sl = tid; sl < S; sl += 1024) {
        int64_t ex = ids[(sl / n_used) * ids_stride + sl % n_used];
        ex = ex < 0 ? 0 : (ex >= n_expert ? n_expert - 1 : ex);
        atomicAdd(&cnt[ex], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int col = 0, nt = 0;
        for (int ex = 0; ex < n_expert; ex++) {
            first[ex] = col;
            for (int c = 0; c < cnt[ex]; c += bn, nt++) {
                tiles[4 * nt] = ex;
                tiles[4 * nt + 1] = col + c;
                tiles[4 * nt + 2] = col + cnt[ex];
                tiles[4 * nt + 3] = 0;
            }
            col += cnt[ex];
        }
        *n_tiles = nt;
    }
    __syncthreads();
    for (int64_t sl = tid; sl < S; sl += 1024) {
        const int64_t t = sl / n_used, e = sl % n_used;
        int64_t ex = ids[t * ids_stride + e];
        ex = ex < 0 ? 0 : (ex >= n_expert ? n_expert - 1 : ex);
        const int pos = first[ex] + atomicAdd(&cursor[ex], 1);
        act_row[pos] = (int32_t)(t * nb1 + e % nb1);
        dst_row[pos] = (int32_t)sl;
    }
}

// column tile of the routed launch: 64 while the experts see few slots each, 128 beyond
__host__ inline int route_bn(int64_t n_expert, int64_t S) { return S <= 48 * n_expert ? 64 : 128; }
__host__ inline size_t route_max_tiles(int64_t n_expert, int64_t S) { return (size_t)((S + 63) / 64 + n_expert); }
__host__ inline size_t route_bytes(int64_t n_expert, int64_t S) {
    const size_t max_tiles = route_max_tiles(n_expert, S);
    return (2 * (size_t)S + 4 * max_tiles + 4) * sizeof(int32_t);
}

// the routing kernel for launches built elsewhere (the wide-tile kernel's routed form, mmq_w.hip)
void launch_route_slots(hipStream_t s, const int32_t *ids, int64_t ids_stride, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T, int bn,
                        int32_t *act_row, int32_t *dst_row, int32_t *tiles, int32_t *n_tiles) {
    MI355_LAUNCH(k_route_slots, dim3(1), dim3(1024), 0, s, ids, ids_stride, n_expert, n_used, nb1, T, bn, act_row, dst_row, tiles, n_tiles);
}

template <int TYPE>
static void launch_mmq_k_id(hipStream_t s, const void *as, const void *act, int64_t act_rows, const int32_t *ids, int64_t ids_stride,
                            float *dst, int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T, void *route_ws) {
    const int64_t S = T * n_used;
    constexpr bool BOTH = TYPE == MI355_Q4_K || TYPE == MI355_Q6_K;   // the types the 64-column kernel unpacks too
    const int bn = BOTH ? route_bn(n_expert, S) : 128;
    const int max_tiles = (int)((S + bn - 1) / bn + n_expert);
    int32_t *act_row = (int32_t *)route_ws, *dst_row = act_row + S, *tiles = dst_row + S, *n_tiles = tiles + 4 * (int64_t)route_max_tiles(n_expert, S);
    MI355_LAUNCH(k_route_slots, dim3(1), dim3(1024), 0, s, ids, ids_stride, n_expert, n_used, nb1, T, bn, act_row, dst_row, tiles, n_tiles);
    const row_layout L = make_row_layout(TYPE, K);
    const int8_t *aq = (const int8_t *)act;
    const float *ad8 = (const float *)(aq + q8k_d_offset(K, act_rows));
    const _Float16 *abs_ = (const _Float16 *)(aq + q8k_bs_offset(K, act_rows));
    const int n_row_tiles = (int)((N + 63) / 64);
    const int n_groups = n_row_tiles * max_tiles;
    const int n_groups_padded = (n_groups + 7) & ~7;
    const mmq_route route = {act_row, dst_row, tiles, n_tiles, N * L.row_bytes};
    if constexpr (BOTH) {
        if (bn == 64) {
            MI355_LAUNCH((k_mmq_k<TYPE, 1, 1, 2, true>), dim3((unsigned)n_groups_padded), dim3(256), 0, s, (const uint8_t *)as, aq, ad8, abs_,
                               dst, nullptr, N, K, S, N, L, max_tiles, n_groups, n_groups_padded, route);
            return;
        }
    }
    MI355_LAUNCH((k_mmq_kp<TYPE, true>), dim3((unsigned)n_groups_padded), dim3(256), 0, s, (const uint8_t *)as, aq, ad8, abs_, dst, nullptr, N, K,
                           S, N, L, max_tiles, n_groups, n_groups_padded, route);
}

}  // namespace mi355

using namespace mi355;

extern "C" {

size_t mi355_act_q8k_bytes(int64_t k, int64_t nrows) {
    if (k <= 0 || nrows <= 0 || k % QKK != 0) return 0;
    return q8k_bs_offset(k, nrows) + (size_t)nrows * (size_t)(k / QKK) * 32;
}

int mi355_quantize_act_q8k(void *stream, const float *x, void *act, int64_t k, int64_t nrows, int64_t x_stride) {
    MI355_REQUIRE(k > 0 && k % QKK == 0, "quantize_act_q8k: k=%lld is not a multiple of 256", (long long)k);
    MI355_REQUIRE(nrows >= 0 && nrows <= 65535, "quantize_act_q8k: nrows=%lld out of range", (long long)nrows);
    MI355_REQUIRE(x_stride >= k && x_stride % 4 == 0 && ((uintptr_t)x & 15) == 0, "quantize_act_q8k: x must be 16-byte aligned with a row stride that is a multiple of 4 floats");
    MI355_REQUIRE(((uintptr_t)act & 15) == 0, "quantize_act_q8k: workspace must be 16-byte aligned");
    if (nrows == 0) return MI355_OK;
    int8_t *q = (int8_t *)act;
    float *d8 = (float *)(q + q8k_d_offset(k, nrows));
    _Float16 *bs = (_Float16 *)(q + q8k_bs_offset(k, nrows));
    const dim3 grid((unsigned)((k / QKK + 3) / 4), (unsigned)nrows);
    MI355_LAUNCH(k_quantize_q8k, grid, dim3(256), 0, (hipStream_t)stream, x, q, d8, bs, k, x_stride);
    return launch_status("k_quantize_q8k");
}

size_t mi355_mul_mat_id_q8k_route_bytes(int64_t n_expert, int64_t n_used, int64_t T) {
    if (n_expert <= 0 || n_used <= 0 || T <= 0) return 0;
    return (route_bytes(n_expert, T * n_used) + 255) & ~(size_t)255;
}

int mi355_mul_mat_id_q8k(void *stream, int type, const void *as, const void *act, const int32_t *ids, int64_t ids_stride, float *dst,
                         int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T, void *route_ws,
                         size_t route_ws_bytes) {
    MI355_REQUIRE(type == MI355_Q4_K || type == MI355_Q5_K || type == MI355_Q6_K || type == MI355_IQ4_XS, "mul_mat_id_q8k: weight type %d has no super-block tile kernel", type);
    MI355_REQUIRE(N > 0 && K > 0 && n_expert > 0 && n_used > 0 && nb1 > 0 && T > 0, "mul_mat_id_q8k: bad shape");
    MI355_REQUIRE(K % QKK == 0, "mul_mat_id_q8k: K=%lld is not a multiple of 256", (long long)K);
    MI355_REQUIRE(n_expert <= ROUTE_MAX_EXPERTS, "mul_mat_id_q8k: more than %d experts", ROUTE_MAX_EXPERTS);
    MI355_REQUIRE(ids_stride >= n_used, "mul_mat_id_q8k: ids_stride < n_used");
    MI355_REQUIRE(T * n_used < (1 << 24) && nb1 * T < (1 << 24), "mul_mat_id_q8k: too many slots");
    const row_layout L = make_row_layout(type, K);
    MI355_REQUIRE(layout_aligned(as, L) && (N * L.row_bytes) % 16 == 0, "mul_mat_id_q8k: weight rows are not 16-byte aligned (K=%lld)", (long long)K);
    MI355_REQUIRE(((uintptr_t)act & 15) == 0 && (q8k_d_offset(K, nb1 * T) & 15) == 0, "mul_mat_id_q8k: activation workspace is not 16-byte aligned");
    if (route_ws == nullptr || route_ws_bytes < route_bytes(n_expert, T * n_used) || ((uintptr_t)route_ws & 15) != 0) {
        set_error("mul_mat_id_q8k: routing workspace of %zu bytes, need %zu (16-byte aligned)", route_ws_bytes, route_bytes(n_expert, T * n_used));
        return MI355_ERR_WORKSPACE;
    }
    hipStream_t s = (hipStream_t)stream;
    if (type == MI355_Q4_K) launch_mmq_k_id<MI355_Q4_K>(s, as, act, nb1 * T, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, T, route_ws);
    else if (type == MI355_Q5_K) launch_mmq_k_id<MI355_Q5_K>(s, as, act, nb1 * T, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, T, route_ws);
    else if (type == MI355_IQ4_XS) launch_mmq_k_id<MI355_IQ4_XS>(s, as, act, nb1 * T, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, T, route_ws);
    else launch_mmq_k_id<MI355_Q6_K>(s, as, act, nb1 * T, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, T, route_ws);
    return launch_status("k_mmq_k (routed)");
}

size_t mi355_kq_planes_bytes(int64_t rows, int64_t K) {
    if (rows <= 0 || K <= 0 || K % QKK != 0) return 0;
    return 2 * (size_t)rows * (size_t)K + (size_t)rows * (size_t)(K / QKK) * 48;
}

int mi355_kq_unpack_planes(void *stream, int type, const void *W, void *planes, int64_t rows, int64_t K) {
    MI355_REQUIRE(type == MI355_Q4_K || type == MI355_Q6_K, "kq_unpack_planes: weight type %d is not a K-quant", type);
    MI355_REQUIRE(rows > 0 && K > 0 && K % QKK == 0, "kq_unpack_planes: bad shape rows=%lld K=%lld", (long long)rows, (long long)K);
    const row_layout L = make_row_layout(type, K);
    MI355_REQUIRE(layout_aligned(W, L) && ((uintptr_t)planes & 15) == 0, "kq_unpack_planes: rows are not 16-byte aligned (K=%lld)", (long long)K);
    const int64_t pieces = rows * (K >> 8) * 8;
    MI355_REQUIRE((pieces + 255) / 256 < 0x7fffffff, "kq_unpack_planes: too many pieces for one launch");
    const dim3 grid((unsigned)((pieces + 255) / 256)), block(256);
    if (type == MI355_Q4_K) MI355_LAUNCH(k_unpack_planes<MI355_Q4_K>, grid, block, 0, (hipStream_t)stream, (const uint8_t *)W, (int8_t *)planes, rows, K, L);
    else MI355_LAUNCH(k_unpack_planes<MI355_Q6_K>, grid, block, 0, (hipStream_t)stream, (const uint8_t *)W, (int8_t *)planes, rows, K, L);
    return launch_status("k_unpack_planes");
}

size_t mi355_mul_mat_q8k_ws_bytes(int64_t N, int64_t K, int64_t B) {
    if (N <= 0 || K <= 0 || B <= 0 || K % QKK != 0) return 0;
    const int n = split_k_slices(N, K, B);
    return n > 1 && N % 4 == 0 ? (size_t)n * (size_t)N * (size_t)B * sizeof(float) : 0;
}

int mi355_mul_mat_q8k_planes(void *stream, int type, const void *planes, const void *act, float *dst, const float *residual, int64_t N,
                             int64_t K, int64_t B, int64_t dst_stride) {
    return mi355_mul_mat_q8k_planes_ws(stream, type, planes, act, dst, residual, N, K, B, dst_stride, nullptr, 0);
}

int mi355_mul_mat_q8k_planes_ws(void *stream, int type, const void *planes, const void *act, float *dst, const float *residual, int64_t N,
                                int64_t K, int64_t B, int64_t dst_stride, void *ws, size_t ws_bytes) {
    MI355_REQUIRE(type == MI355_Q4_K || type == MI355_Q6_K, "mul_mat_q8k_planes: weight type %d is not a K-quant", type);
    MI355_REQUIRE(N > 0 && K > 0 && B > 0, "mul_mat_q8k_planes: bad shape N=%lld K=%lld B=%lld", (long long)N, (long long)K, (long long)B);
    MI355_REQUIRE(K % QKK == 0, "mul_mat_q8k_planes: K=%lld is not a multiple of 256", (long long)K);
    MI355_REQUIRE(N * K < ((int64_t)1 << 32), "mul_mat_q8k_planes: matrix too large for 32-bit plane offsets");
    MI355_REQUIRE(dst_stride >= N, "mul_mat_q8k_planes: dst_stride < N");
    MI355_REQUIRE(planes != nullptr && ((uintptr_t)planes & 15) == 0, "mul_mat_q8k_planes: planes are not 16-byte aligned");
    MI355_REQUIRE(((uintptr_t)act & 15) == 0 && (q8k_d_offset(K, B) & 15) == 0 && (q8k_bs_offset(K, B) & 15) == 0,
                  "mul_mat_q8k_planes: activation workspace is not 16-byte aligned");
    MI355_REQUIRE((N + 63) / 64 * ((B + 63) / 64) < (1 << 30), "mul_mat_q8k_planes: too many tiles");
    const row_layout L = make_row_layout(type, K);
    const int8_t *aq = (const int8_t *)act;
    const float *ad8 = (const float *)(aq + q8k_d_offset(K, B));
    const _Float16 *abs_ = (const _Float16 *)(aq + q8k_bs_offset(K, B));
    const int n_row_tiles = (int)((N + 63) / 64), n_col_tiles = (int)((B + 127) / 128);
    const int n_groups = n_row_tiles * n_col_tiles, n_groups_padded = (n_groups + 7) & ~7;
    hipStream_t s = (hipStream_t)stream;
    const int n_slices = usable_slices(N, K, B, ws, ws_bytes);
    const dim3 grid((unsigned)n_groups_padded, (unsigned)n_slices);
    float *out = n_slices > 1 ? (float *)ws : dst;
    const float *res = n_slices > 1 ? nullptr : residual;
    const int64_t out_stride = n_slices > 1 ? N : dst_stride;
    if (type == MI355_Q4_K)
        MI355_LAUNCH((k_mmq_pl<MI355_Q4_K, false>), grid, dim3(256), 0, s, (const int8_t *)planes, aq, ad8, abs_, out, res, N, K, B, out_stride, L,
                           n_col_tiles, n_groups, n_groups_padded, mmq_route{}, N * K);
    else
        MI355_LAUNCH((k_mmq_pl<MI355_Q6_K, false>), grid, dim3(256), 0, s, (const int8_t *)planes, aq, ad8, abs_, out, res, N, K, B, out_stride, L,
                           n_col_tiles, n_groups, n_groups_padded, mmq_route{}, N * K);
    if (n_slices > 1) launch_split_sum(s, (const float *)ws, dst, residual, N, B, dst_stride, n_slices);
    return launch_status("k_mmq_pl");
}

int mi355_mul_mat_q8k_add(void *stream, int type, const void *W, const void *act, float *dst, const float *residual, int64_t N, int64_t K,
                          int64_t B, int64_t dst_stride) {
    return mi355_mul_mat_q8k_ws(stream, type, W, act, dst, residual, N, K, B, dst_stride, nullptr, 0);
}

int mi355_mul_mat_q8k_ws(void *stream, int type, const void *W, const void *act, float *dst, const float *residual, int64_t N, int64_t K,
                         int64_t B, int64_t dst_stride, void *ws, size_t ws_bytes) {
    MI355_REQUIRE(type == MI355_Q4_K || type == MI355_Q5_K || type == MI355_Q6_K || type == MI355_IQ4_XS, "mul_mat_q8k: weight type %d has no super-block tile kernel", type);
    MI355_REQUIRE(N > 0 && K > 0 && B > 0, "mul_mat_q8k: bad shape N=%lld K=%lld B=%lld", (long long)N, (long long)K, (long long)B);
    MI355_REQUIRE(K % QKK == 0, "mul_mat_q8k: K=%lld is not a multiple of 256", (long long)K);
    MI355_REQUIRE(dst_stride >= N, "mul_mat_q8k: dst_stride < N");
    const row_layout L = make_row_layout(type, K);
    MI355_REQUIRE(layout_aligned(W, L), "mul_mat_q8k: weight rows are not 16-byte aligned (K=%lld)", (long long)K);
    MI355_REQUIRE(((uintptr_t)act & 15) == 0 && (q8k_d_offset(K, B) & 15) == 0 && (q8k_bs_offset(K, B) & 15) == 0,
                  "mul_mat_q8k: activation workspace is not 16-byte aligned");
    MI355_REQUIRE((N + 63) / 64 * ((B + 63) / 64) < (1 << 30), "mul_mat_q8k: too many tiles");
    hipStream_t s = (hipStream_t)stream;
    if (type == MI355_Q4_K) launch_mmq_k<MI355_Q4_K>(s, W, act, dst, residual, N, K, B, dst_stride, ws, ws_bytes);
    else if (type == MI355_Q5_K) launch_mmq_k<MI355_Q5_K>(s, W, act, dst, residual, N, K, B, dst_stride, ws, ws_bytes);
    else if (type == MI355_IQ4_XS) launch_mmq_k<MI355_IQ4_XS>(s, W, act, dst, residual, N, K, B, dst_stride, ws, ws_bytes);
    else launch_mmq_k<MI355_Q6_K>(s, W, act, dst, residual, N, K, B, dst_stride, ws, ws_bytes);
    return launch_status("k_mmq_k");
}

int mi355_mul_mat_q8k(void *stream, int type, const void *W, const void *act, float *dst, int64_t N, int64_t K, int64_t B,
                      int64_t dst_stride) {
    return mi355_mul_mat_q8k_add(stream, type, W, act, dst, nullptr, N, K, B, dst_stride);
}

}  // extern "C"
