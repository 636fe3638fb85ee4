// FLASH_ATTN_EXT for many query rows (prefill) on the f16 matrix cores.
// Semantics: ggml_compute_forward_flash_attn_ext_f16, ggml/src/ggml-cpu/ggml-cpu.c:10916-11129
// (q rounded to f16, scores scale * q.k [+ softcap] + slope * mask, online softmax in f32,
// -inf mask entries contribute nothing, GQA by head index division).
//
// A 256-thread group serves one kv head: its 4 waves are HPW query heads of that kv head times
// 4 / HPW tiles of 32 queries, so every K/V tile staged in LDS is used by all four waves.
// Per wave and 64-cell kv tile, with v_mfma_f32_32x32x16_f16 (D[i][j], lane l supplies row /
// column l % 32 and k slots [8*(l/32), +8); D register r is i = 8*(r/4) + 4*(l/32) + r%4, j = l%32):
//   S^T = K Q^T   A = K rows (i = kv cell), B = Q rows (j = query)  -> a lane holds ONE query's
//                 scores for 16 cells, so softmax row reductions are in-lane plus one xor-32 step
//   O^T += V^T P^T  A = V^T rows (i = head dim), B = P^T (j = query) -> the B operand is the lane's
//                 own score registers 8t..8t+7 rounded to f16: no cross-lane data movement.  The
//                 kv cells those registers stand for, 16t + 8*(s/4) + 4*(l/32) + s%4, fix which
//                 cells the A operand must supply in k slot s: four cells at one element of the head, twice -
//                 two transposing reads (ds_read_b64_tr_b16) of the row-major V tile.
// Rescaling by exp(m_old - m_new) is one multiply per accumulator register because both
// accumulators are indexed by query along the lanes.
#include "fattn.hpp"


#include <float.h>

namespace mi355 {

namespace {

constexpr int FM_BC = 64;            // kv cells per tile
constexpr float FM_NEG = -FLT_MAX / 2;

// ---- staging of one 64-cell K tile and the matching V tile through registers, both row-major ----
template <int D, int NTH, int BC = FM_BC> struct kv_stage {
    static constexpr int KP = D + 8;        // f16 pitch of a K row in LDS (16 bytes of padding spread the banks)
    static constexpr int VP = D + 16;       // f16 pitch of a V row in LDS: rows 8 banks apart, so the four rows of a transposing read miss each other
    static constexpr int KCH = D / 8;       // 16-byte chunks per K/V row
    static constexpr int KIT = BC * KCH / NTH;            // chunks per thread per tile, K and V each
    static_assert(D % 32 == 0 && KIT >= 1, "head size not served by this kernel");
    static_assert(NTH % KCH == 0, "a thread keeps its chunk position over the rows it loads");
    u32x4 k[KIT], v[KIT];

    // A tile that lies inside the cache is addressed as (uniform base of the tile and of the thread's it-th row block) + (one
    // 32-bit offset per thread, the same for every tile): thread tid loads rows tid / KCH + it * (NTH / KCH), chunk tid % KCH.
    // The uniform part is scalar arithmetic; per-row 64-bit products in vector registers cost as many instructions per tile
    // step as the soft-max.  The launcher checks that a tile's span fits 32 bits.  The last, partial tile clamps row by row.
    __device__ __forceinline__ void fetch(const fattn_args &a, int64_t hk, int64_t kv0, int tid) {
        if (kv0 + BC <= a.Nkv) {   // uniform
            const unsigned r0 = (unsigned)(tid / KCH), ch16 = (unsigned)(tid % KCH) * 16;
            const unsigned ko = r0 * (unsigned)a.k_nb1 + ch16, vo = r0 * (unsigned)a.v_nb1 + ch16;
            const uint8_t *kb = a.k + kv0 * a.k_nb1 + hk * a.k_nb2, *vb = a.v + kv0 * a.v_nb1 + hk * a.v_nb2;
#pragma unroll
            for (int it = 0; it < KIT; it++) {
                k[it] = load16(kb + (size_t)it * (NTH / KCH) * a.k_nb1 + ko);
                v[it] = load16(vb + (size_t)it * (NTH / KCH) * a.v_nb1 + vo);
            }
            return;
        }
        const int64_t last = a.Nkv - 1;
#pragma unroll
        for (int it = 0; it < KIT; it++) {
            const int unit = tid + it * NTH;
            const int row = unit / KCH, ch = unit % KCH;
            const int64_t c = kv0 + row < last ? kv0 + row : last;   // rows past the end repeat the last cell; their scores are dropped
            k[it] = load16(a.k + c * a.k_nb1 + hk * a.k_nb2 + ch * 16);
            v[it] = load16(a.v + c * a.v_nb1 + hk * a.v_nb2 + ch * 16);
        }
    }
    __device__ __forceinline__ void commit(_Float16 *sK, _Float16 *sV, int tid) const {
#pragma unroll
        for (int it = 0; it < KIT; it++) {
            const int unit = tid + it * NTH;
            const int row = unit / KCH, ch = unit % KCH;
            *(u32x4 *)(sK + row * KP + ch * 8) = k[it];
            *(u32x4 *)(sV + row * VP + ch * 8) = v[it];
        }
    }
};

// f16 bits of the mask entries of NG groups of 4 consecutive cells, first cell c0 + 8*g.  Loads are
// unconditional (clamped), so they can be issued with the K/V prefetch and never force a wait.
template <int NG>
__device__ __forceinline__ void fetch_mask(u32x2 (&out)[NG], const unsigned short *mrow, bool vec_ok, int64_t c0, int64_t Nkv) {
    if (mrow == nullptr) {
#pragma unroll
        for (int g = 0; g < NG; g++) out[g] = u32x2{0, 0};
    } else if (vec_ok) {   // uniform: aligned rows and a full tile
#pragma unroll
        for (int g = 0; g < NG; g++) out[g] = *(const u32x2 *)(mrow + c0 + 8 * g);
    } else {
        const int64_t last = Nkv - 1;
#pragma unroll
        for (int g = 0; g < NG; g++) {
            u32 h[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int64_t c = c0 + 8 * g + i;
                h[i] = mrow[c < last ? c : last];
            }
            out[g] = u32x2{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
        }
    }
}
__device__ __forceinline__ float mask_value(const u32x2 &w, int i) {
    return half_bits_to_float((unsigned short)((i < 2 ? w[0] : w[1]) >> (16 * (i & 1))));
}

// max / sum of a value over a lane and its partner in the other half of the wave (lane ^ 32), in every lane: one
// v_permlane32_swap (both halves of one register handed to the other half of a second) instead of a trip through the LDS
// crossbar, whose latency a wave that is alone on its SIMD waits out.
__device__ __forceinline__ float half_pair_max(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_pair_sum(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Running maximum of the prefill kernels.  The reference point of a column's exponentials moves only when the tile's largest
// score exceeds it by more than FM_LAZY: any reference point gives the same quotient sum(p v) / sum(p), and while it stays put
// the 64 output registers are not rescaled (with an exact running maximum some query of a 32-query tile raises its maximum
// in most tiles of a few thousand cells; this way it happens in the first tiles only).  Probabilities then reach e^FM_LAZY at
// most, far inside the f16 range of the matrix operand.
constexpr float FM_LAZY = 8.0f;
constexpr float FM_LOG2E = 1.4426950408889634f;
__device__ __forceinline__ float lazy_max(float m, float mx) { return mx > m + FM_LAZY ? mx : m; }
// exp(s - m) as one multiply-add and one exponential: 2^(s log2(e) - m log2(e)); m2 = m log2(e)
__device__ __forceinline__ float exp_rel(float s, float m2) { return __builtin_amdgcn_exp2f(fmaf(s, FM_LOG2E, -m2)); }

// scale [+ softcap], add the mask, mark dropped cells with FM_NEG; returns the largest surviving score.
// A masked cell (-inf; slopes are positive) and a NaN score of a stale cell both end as FM_NEG in fmaxf(s, FM_NEG); the test against
// the end of the range is made only in a tile that reaches past it (uniform over the group), on 32-bit offsets.
__device__ __forceinline__ float finish_scores(f32x16 &S, const u32x2 (&mw)[4], const fattn_args &a, float scale, float slope,
                                                int64_t c_first, int lhi, int64_t c_end) {
    float mx = FM_NEG;
    const int64_t room = c_end - c_first;
    if (a.softcap == 0.0f && slope == 1.0f && room >= 32) {   // the common case in one multiply-add per score: scale * s + mask
#pragma unroll
        for (int g = 0; g < 4; g++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float s = fmaf(S[4 * g + i], scale, mask_value(mw[g], i));
                s = fmaxf(s, FM_NEG);   // -inf and NaN become FM_NEG
                S[4 * g + i] = s;
                mx = fmaxf(mx, s);
            }
        return mx;
    }
    if (a.softcap != 0.0f) {
#pragma unroll
        for (int r = 0; r < 16; r++) S[r] = a.softcap * tanhf(S[r] * scale);
    } else {
#pragma unroll
        for (int r = 0; r < 16; r++) S[r] *= scale;
    }
    if (room >= 32) {   // every cell of this half tile lies inside the range
#pragma unroll
        for (int g = 0; g < 4; g++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float s = S[4 * g + i] + slope * mask_value(mw[g], i);
                s = fmaxf(s, FM_NEG);   // -inf and NaN become FM_NEG
                S[4 * g + i] = s;
                mx = fmaxf(mx, s);
            }
    } else {
        const int left = (int)room - 4 * lhi;   // cells of the range from this lane's first one on (may be <= 0)
#pragma unroll
        for (int g = 0; g < 4; g++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float s = S[4 * g + i] + slope * mask_value(mw[g], i);
                s = 8 * g + i < left ? fmaxf(s, FM_NEG) : FM_NEG;
                S[4 * g + i] = s;
                mx = fmaxf(mx, s);
            }
    }
    return mx;
}

// The decode kernel keeps the plain form (every score tested against the end of its kv range): with its two tile bodies the
// split into a full-tile and an end-of-range variant cost it 10 % at 131072 cells (115 -> 127 us) for 2 % gained at 32768.
__device__ __forceinline__ float finish_scores_dec(f32x16 &S, const u32x2 (&mw)[4], const fattn_args &a, float scale, float slope,
                                                    int64_t c_first, int lhi, int64_t c_end) {
    if (a.softcap != 0.0f) {
#pragma unroll
        for (int r = 0; r < 16; r++) S[r] = a.softcap * tanhf(S[r] * scale);
    } else {
#pragma unroll
        for (int r = 0; r < 16; r++) S[r] *= scale;
    }
    float mx = FM_NEG;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const int64_t c = c_first + 8 * g + 4 * lhi;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float mv = mask_value(mw[g], i);
            float s = S[4 * g + i] + slope * mv;
            const bool valid = c + i < c_end && mv != -INFINITY && s > FM_NEG;   // NaN scores of stale cells drop out too
            s = valid ? s : FM_NEG;
            S[4 * g + i] = s;
            mx = fmaxf(mx, s);
        }
    }
    return mx;
}

template <int D>
__device__ __forceinline__ void load_q(f16x8 (&qf)[D / 16], const float *qp, int lhi) {
#pragma unroll
    for (int kk = 0; kk < D / 16; kk++) {   // rounded to f16 (ggml-cpu.c:11037-11040)
        const f32x4 x0 = *(const f32x4 *)(qp + 16 * kk + 8 * lhi);
        const f32x4 x1 = *(const f32x4 *)(qp + 16 * kk + 8 * lhi + 4);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            qf[kk][i] = (_Float16)x0[i];
            qf[kk][4 + i] = (_Float16)x1[i];
        }
    }
}
__device__ __forceinline__ float alibi_slope(const fattn_args &a, int64_t head) {   // ggml-cpu.c:10998-11003
    if (a.max_bias <= 0.0f) return 1.0f;
    const unsigned h = (unsigned)head;
    return h < a.n_head_log2 ? powf(a.m0, (float)(h + 1)) : powf(a.m1, (float)(2 * (h - a.n_head_log2) + 1));
}

// O^T tiles [DT0, DT0 + NDT) += V^T P^T for the 32 cells of half u whose probabilities sit in S.  The A operand of a lane -
// element 32 dt + l32 of cells c .. c + 3 and c + 8 .. c + 11, c = 32 u + 16 t + 4 lhi - comes from the row-major V tile by two
// transposing reads: in each group of 16 lanes, lane i receives element i % 4 of the four rows that lanes i / 4, i / 4 + 4, + 8 and
// + 12 point at, so lane 4 r + q of a group points at row c + r, elements 16 (group % 2) + 4 q .. + 3 of the tile's 32.
template <int D, int NDT>
__device__ __forceinline__ void accumulate_pv(f32x16 (&o)[NDT], const f32x16 &S, const _Float16 *sV, int dt0, int u, int l32, int lhi) {
    constexpr int VP = D + 16;
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    const int li = l32 & 15;
    const _Float16 *lane_base = sV + (32 * u + 4 * lhi + (li >> 2)) * VP + 16 * (l32 >> 4) + 4 * (li & 3);
#pragma unroll
    for (int t = 0; t < 2; t++) {
        f16x8 pf;
#pragma unroll
        for (int i = 0; i < 8; i++) pf[i] = (_Float16)S[8 * t + i];
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) {
            const _Float16 *vp = lane_base + 16 * t * VP + 32 * (dt0 + dt);
            const s16x4 v0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)vp);
            const s16x4 v1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)(vp + 8 * VP));
            const f16x4 h0 = __builtin_bit_cast(f16x4, v0), h1 = __builtin_bit_cast(f16x4, v1);
            f16x8 vf;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                vf[i] = h0[i];
                vf[4 + i] = h1[i];
            }
            o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf, o[dt], 0, 0, 0);
        }
    }
}

// EAGER: all of the row's fragments are requested before the first matrix instruction (D / 2 more registers), so the chain of
// dependent instructions does not stop for an LDS round trip after every second one.
template <int D, bool EAGER = false>
__device__ __forceinline__ f32x16 scores(const f16x8 (&qf)[D / 16], const _Float16 *sK, int u, int l32, int lhi) {
    constexpr int KP = D + 8;
    f32x16 S;
#pragma unroll
    for (int r = 0; r < 16; r++) S[r] = 0.0f;
    if constexpr (EAGER) {
        f16x8 kf[D / 16];
#pragma unroll
        for (int kk = 0; kk < D / 16; kk++) kf[kk] = *(const f16x8 *)(sK + (32 * u + l32) * KP + 16 * kk + 8 * lhi);
#pragma unroll
        for (int kk = 0; kk < D / 16; kk++) asm volatile("" : "+v"(kf[kk]));   // keeps the loads ahead of the chain
#pragma unroll
        for (int kk = 0; kk < D / 16; kk++) S = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[kk], qf[kk], S, 0, 0, 0);
        return S;
    }
#pragma unroll
    for (int kk = 0; kk < D / 16; kk++) {
        const f16x8 kf = *(const f16x8 *)(sK + (32 * u + l32) * KP + 16 * kk + 8 * lhi);
        S = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[kk], S, 0, 0, 0);
    }
    return S;
}

// ---- prefill --------------------------------------------------------------------------------
// How far each tile of 32 queries can see: extent[t] = 1 + the last cell whose mask entry is not -inf in any of the tile's
// rows (0 when there is none).  With llama.cpp's causal mask the tiles of a prompt see a growing prefix of the cache, and the
// prefill kernel stops staging K/V tiles at that point instead of loading, scoring and then discarding them.  One group
// per tile; threads take 8 cells (16 bytes) of each row at a time.  Needs 16-byte aligned mask rows and Nkv % 8 == 0.
__global__ void __launch_bounds__(256) k_mask_extent(const uint8_t *__restrict__ mask, size_t mask_nb1, int64_t Nq, int64_t Nkv,
                                                     int32_t *__restrict__ extent) {
    __shared__ int s_max[4];
    const int64_t q0 = (int64_t)blockIdx.x * 32;
    int last = -1;
    for (int64_t c = (int64_t)threadIdx.x * 8; c < Nkv; c += 256 * 8) {
        u32x4 any = {0, 0, 0, 0};   // per 16-bit field: non-zero when some row's entry differs from -inf (0xFC00)
        for (int r = 0; r < 32; r++) {
            const int64_t iq = q0 + r < Nq ? q0 + r : Nq - 1;
            const u32x4 m = load16(mask + iq * mask_nb1 + c * 2);
#pragma unroll
            for (int i = 0; i < 4; i++) any[i] |= m[i] ^ 0xFC00FC00u;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {   // c grows, so the last assignment is the largest visible cell
            const u32 w = any[i];
            if (w & 0x0000FFFFu) last = (int)c + 2 * i;
            if (w & 0xFFFF0000u) last = (int)c + 2 * i + 1;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) last = max(last, __shfl_xor(last, off, 64));
    if ((threadIdx.x & 63) == 0) s_max[threadIdx.x >> 6] = last;
    __syncthreads();
    if (threadIdx.x == 0) extent[blockIdx.x] = max(max(s_max[0], s_max[1]), max(s_max[2], s_max[3])) + 1;
}

// Groups go to the eight XCDs round-robin by linear index and each XCD has its own L2.  Renumbered so that XCD x works through the
// x-th eighth of the grid in (head, query tile) order, the groups that read one kv head's K and V run on one XCD and find in its
// L2 what their neighbours loaded (with 8 kv heads: one head per XCD).  Query tiles are taken from the last one down: under a
// causal mask the last tile sees the most cells, and groups are started in index order, so the long groups start first and the
// short ones fill the gaps at the end (in ascending order the launch ends with the longest groups running alone: 64 slots
// and 128 tiles of 1 .. 128 half-steps finish after 96 steps instead of 64.5).  Returns the group's place (x, y) in the grid.
struct grid_pos { unsigned x, y; };
__device__ __forceinline__ grid_pos xcd_grid_pos() {
    const unsigned nx = gridDim.x;
    const uint64_t total = (uint64_t)nx * gridDim.y;
    uint64_t L = blockIdx.x + (uint64_t)nx * blockIdx.y;
    if (total % 8 == 0) L = (L % 8) * (total / 8) + L / 8;
    return grid_pos{nx - 1 - (unsigned)(L % nx), (unsigned)(L / nx)};
}

template <int D, int HPW>
__global__ void __launch_bounds__(256, 2) k_fattn_mma(fattn_args a) {
    typedef kv_stage<D, 256> stage_t;
    constexpr int QTW = 4 / HPW;   // query tiles per group
    __shared__ __attribute__((aligned(16))) _Float16 sK[FM_BC * stage_t::KP];
    __shared__ __attribute__((aligned(16))) _Float16 sVt[FM_BC * stage_t::VP];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    const int groups = (int)(a.Hq / a.Hkv) / HPW;
    const grid_pos gp = xcd_grid_pos();
    const int64_t hk = gp.y / groups, hg = gp.y % groups;
    const int64_t head = (hk * groups + hg) * HPW + (wave % HPW);
    const int64_t q0 = ((int64_t)gp.x * QTW + wave / HPW) * 32;
    const int64_t iq = q0 + l32 < a.Nq ? q0 + l32 : a.Nq - 1;   // clamped: rows past Nq are computed and dropped

    f16x8 qf[D / 16];
    load_q<D>(qf, (const float *)(a.q + iq * a.q_nb1 + head * a.q_nb2), lhi);
    float slope = alibi_slope(a, head);
    asm volatile("" : "+v"(slope));   // kept in a vector register also where the head is uniform over the group: a scalar slope makes
                                      // the compiler build a second copy of the tile loop around "slope == 1", which then spills
    const float scale = a.softcap != 0.0f ? a.scale / a.softcap : a.scale;
    const unsigned short *mrow = a.mask ? (const unsigned short *)(a.mask + iq * a.mask_nb1) : nullptr;
    const bool mask_aligned = (((uintptr_t)a.mask | a.mask_nb1) & 7) == 0;

    f32x16 o[D / 32];
#pragma unroll
    for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[dt][r] = 0.0f;
    float m = FM_NEG, l = 0.0f;

    // cells past kv_limit are masked for every query of this group
    int64_t kv_limit = a.Nkv;
    if (a.kv_extent) {
        int e = 0;
#pragma unroll
        for (int j = 0; j < QTW; j++) {
            const int64_t t = (int64_t)gp.x * QTW + j;
            if (t * 32 < a.Nq) e = max(e, a.kv_extent[t]);
        }
        kv_limit = e < a.Nkv ? e : a.Nkv;
    }

    stage_t st;
    u32x2 mnext[2][4];
    auto prefetch = [&](int64_t kv0) {
        st.fetch(a, hk, kv0, tid);
        const bool vec_ok = mask_aligned && kv0 + FM_BC <= a.Nkv;
        fetch_mask<4>(mnext[0], mrow, vec_ok, kv0 + 4 * lhi, a.Nkv);
        fetch_mask<4>(mnext[1], mrow, vec_ok, kv0 + 32 + 4 * lhi, a.Nkv);
    };
    if (kv_limit > 0) prefetch(0);
    for (int64_t kv0 = 0; kv0 < kv_limit; kv0 += FM_BC) {
        __syncthreads();   // the previous tile has been consumed
        st.commit(sK, sVt, tid);
        u32x2 mcur[2][4];
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int g = 0; g < 4; g++) mcur[u][g] = mnext[u][g];
        __syncthreads();
        if (kv0 + FM_BC < kv_limit) prefetch(kv0 + FM_BC);

        // scores of 64 cells for this lane's query: S[u][r] <-> cell kv0 + 32u + 8*(r/4) + 4*lhi + r%4
        f32x16 S[2];
        float mx = FM_NEG;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            S[u] = scores<D>(qf, sK, u, l32, lhi);
            mx = fmaxf(mx, finish_scores(S[u], mcur[u], a, scale, slope, kv0 + 32 * u, lhi, a.Nkv));
        }
        mx = half_pair_max(mx);
        if (__ballot(mx > FM_NEG) == 0) continue;   // every cell of the tile is masked for all 32 queries (wave-uniform)
        const float m_new = lazy_max(m, mx);
        const float alpha = __builtin_amdgcn_exp2f((m - m_new) * FM_LOG2E);   // exactly 1 while the reference point stays
        // dropped scores are exactly FM_NEG: exp(FM_NEG - m) is 0 for any real maximum; a column that has seen no cell yet
        // (maximum still FM_NEG) subtracts 0 instead, so its dropped scores give 0 as well and not exp(0)
        const float m2 = m_new > FM_NEG ? m_new * FM_LOG2E : 0.0f;
        float rs = 0.0f;
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float p = exp_rel(S[u][r], m2);
                S[u][r] = p;
                rs += p;
            }
        rs = half_pair_sum(rs);
        l = l * alpha + rs;
        m = m_new;
        if (__ballot(alpha != 1.0f) != 0) {   // wave-uniform
#pragma unroll
            for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[dt][r] *= alpha;
        }
#pragma unroll
        for (int u = 0; u < 2; u++) accumulate_pv<D, D / 32>(o, S[u], sVt, 0, u, l32, lhi);
    }

    if (q0 + l32 < a.Nq) {
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
        float *dp = a.dst + ((q0 + l32) * a.Hq + head) * D;
#pragma unroll
        for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                f32x4 w;
#pragma unroll
                for (int i = 0; i < 4; i++) w[i] = o[dt][4 * g + i] * inv;
                *(f32x4 *)(dp + 32 * dt + 8 * g + 4 * lhi) = w;
            }
    }
}

// ---- prefill with few query tiles: the 32-cell parts of every K/V tile go to different waves -----------------------------------
// k_fattn_mma gives a wave 32 queries of one head and the whole 64-cell tile; a batch of a few hundred rows is then fewer groups
// than compute units, each a serial chain of tiles.  Here a group is two query heads of one kv head x the NU 32-cell parts of a
// tile of 32 NU cells: wave (hp, u) scores and accumulates cells [32u, 32u + 32) of each tile for head hp with its own soft-max
// state, and the states of a head's waves are joined pairwise through LDS at the end.  NU = 2: twice the groups of k_fattn_mma
// with half the work per wave and tile; NU = 4 (eight waves, 128-cell tiles) when even those leave one group per compute
// unit: two waves per SIMD, so that one wave's matrix instructions run under the other's soft-max arithmetic, and half the
// tile steps.
template <int D, int NU>
__global__ void __launch_bounds__(128 * NU, NU == 2 ? 2 : 1) k_fattn_mma_half(fattn_args a) {
    constexpr int NTH = 128 * NU, BC = 32 * NU;
    typedef kv_stage<D, NTH, BC> stage_t;
    constexpr int NDT = D / 32;
    constexpr int KV_HALVES = BC * stage_t::KP + BC * stage_t::VP;                    // f16 elements of the K tile and the V tile
    constexpr int MERGE_FLOATS = NU * (D + 2) * 32;                                   // per (head, pair of waves): O^T [D][32], max, sum
    constexpr int SMEM_BYTES = KV_HALVES * 2 > MERGE_FLOATS * 4 ? KV_HALVES * 2 : MERGE_FLOATS * 4;
    __shared__ __attribute__((aligned(16))) uint8_t smem[SMEM_BYTES];
    _Float16 *sK = (_Float16 *)smem, *sVt = sK + BC * stage_t::KP;
    float *s_merge = (float *)smem;   // reused after the last tile

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    const int u = wave % NU, hp = wave / NU;
    const int pairs = (int)(a.Hq / a.Hkv) / 2;   // head pairs per kv head
    const grid_pos gp = xcd_grid_pos();
    const int64_t hk = gp.y / pairs, hg = gp.y % pairs;
    const int64_t head = (hk * pairs + hg) * 2 + hp;
    const int64_t q0 = (int64_t)gp.x * 32;
    const int64_t iq = q0 + l32 < a.Nq ? q0 + l32 : a.Nq - 1;   // clamped: rows past Nq are computed and dropped

    f16x8 qf[D / 16];
    load_q<D>(qf, (const float *)(a.q + iq * a.q_nb1 + head * a.q_nb2), lhi);
    const float slope = alibi_slope(a, head);
    const float scale = a.softcap != 0.0f ? a.scale / a.softcap : a.scale;
    const unsigned short *mrow = a.mask ? (const unsigned short *)(a.mask + iq * a.mask_nb1) : nullptr;
    const bool mask_aligned = (((uintptr_t)a.mask | a.mask_nb1) & 7) == 0;

    f32x16 o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[dt][r] = 0.0f;
    float m = FM_NEG, l = 0.0f;

    stage_t st;
    u32x2 mnext[4];
    auto prefetch = [&](int64_t kv0) {
        st.fetch(a, hk, kv0, tid);
        fetch_mask<4>(mnext, mrow, mask_aligned && kv0 + BC <= a.Nkv, kv0 + 32 * u + 4 * lhi, a.Nkv);
    };
    prefetch(0);
    for (int64_t kv0 = 0; kv0 < a.Nkv; kv0 += BC) {
        __syncthreads();   // the previous tile has been consumed
        st.commit(sK, sVt, tid);
        u32x2 mcur[4];
#pragma unroll
        for (int g = 0; g < 4; g++) mcur[g] = mnext[g];
        __syncthreads();
        if (kv0 + BC < a.Nkv) prefetch(kv0 + BC);
        f32x16 S = scores<D, true>(qf, sK, u, l32, lhi);
        float mx = finish_scores(S, mcur, a, scale, slope, kv0 + 32 * u, lhi, a.Nkv);
        mx = half_pair_max(mx);
        if (__ballot(mx > FM_NEG) == 0) continue;   // all 32 cells masked for all 32 queries (wave-uniform; barriers are at the loop head)
        const float m_new = lazy_max(m, mx);
        const float alpha = __builtin_amdgcn_exp2f((m - m_new) * FM_LOG2E);   // exactly 1 while the reference point stays
        // dropped scores are exactly FM_NEG: exp(FM_NEG - m) is 0 for any real maximum; a column that has seen no cell yet
        // (maximum still FM_NEG) subtracts 0 instead, so its dropped scores give 0 as well and not exp(0)
        const float m2 = m_new > FM_NEG ? m_new * FM_LOG2E : 0.0f;
        float rs = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float p = exp_rel(S[r], m2);
            S[r] = p;
            rs += p;
        }
        rs = half_pair_sum(rs);
        l = l * alpha + rs;
        m = m_new;
        if (__ballot(alpha != 1.0f) != 0) {   // wave-uniform
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[dt][r] *= alpha;
        }
        accumulate_pv<D, NDT>(o, S, sVt, 0, u, l32, lhi);
    }

    // ---- the states of a head's waves are joined pairwise: u + step hands its state to u (step = 1, then 2)
#pragma unroll
    for (int step = 1; step < NU; step *= 2) {
        float *mg = s_merge + (hp * (NU / 2) + (u >> 1) / step) * (D + 2) * 32;   // [d][query], then max, sum
        __syncthreads();
        if ((u & (2 * step - 1)) == step) {
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) mg[(32 * dt + 8 * (r >> 2) + 4 * lhi + (r & 3)) * 32 + l32] = o[dt][r];
            if (lhi == 0) {
                mg[D * 32 + l32] = m;
                mg[(D + 1) * 32 + l32] = l;
            }
        }
        __syncthreads();
        if ((u & (2 * step - 1)) == 0) {
            const float m1 = mg[D * 32 + l32], l1 = mg[(D + 1) * 32 + l32];
            const float M = fmaxf(m, m1);
            const float f0 = __expf(m - M), f1 = __expf(m1 - M);
            l = l * f0 + l1 * f1;
            m = M;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[dt][r] = o[dt][r] * f0 + mg[(32 * dt + 8 * (r >> 2) + 4 * lhi + (r & 3)) * 32 + l32] * f1;
        }
    }
    if (u != 0 || q0 + l32 >= a.Nq) return;
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    float *dp = a.dst + ((q0 + l32) * a.Hq + head) * D;
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            f32x4 w;
#pragma unroll
            for (int i = 0; i < 4; i++) w[i] = o[dt][4 * g + i] * inv;
            *(f32x4 *)(dp + 32 * dt + 8 * g + 4 * lhi) = w;
        }
}

template <int D>
int launch_half(hipStream_t s, const fattn_args &a) {
    const int64_t pairs = (a.Hq / a.Hkv) / 2;
    const dim3 grid((unsigned)((a.Nq + 31) / 32), (unsigned)(a.Hkv * pairs));
    // at most one group per compute unit and a long cache: eight waves on 128-cell tiles (512 rows: 4096 cells 112 -> 103 us,
    // 512 cells 24.8 -> 26.2 us)
    if ((int64_t)grid.x * grid.y <= 256 && a.Nkv >= 1024) MI355_LAUNCH((k_fattn_mma_half<D, 4>), grid, dim3(512), 0, s, a);
    else MI355_LAUNCH((k_fattn_mma_half<D, 2>), grid, dim3(256), 0, s, a);
    return launch_status("k_fattn_mma_half");
}

template <int D, int HPW>
int launch(hipStream_t s, const fattn_args &a) {
    constexpr int QTW = 4 / HPW;
    const int64_t groups = (a.Hq / a.Hkv) / HPW;
    const dim3 grid((unsigned)((a.Nq + 32 * QTW - 1) / (32 * QTW)), (unsigned)(a.Hkv * groups));
    MI355_LAUNCH((k_fattn_mma<D, HPW>), grid, dim3(256), 0, s, a);
    return launch_status("k_fattn_mma");
}

template <int D>
int launch_hpw(hipStream_t s, const fattn_args &a) {
    const int64_t R = a.Hq / a.Hkv;
    if (R % 4 == 0) return launch<D, 4>(s, a);
    if (R % 2 == 0) return launch<D, 2>(s, a);
    return launch<D, 1>(s, a);
}

// ---- decode / small batches: the 32 MFMA columns are (token, head of the GQA group) pairs -------
// A 256-thread group owns one kv head, NT = 32 / R tokens and one kv split, so the K/V bytes of
// a kv head are read once for all R query heads.  Its four waves are (u, h): u picks the 32-cell
// half of each 64-cell tile the wave scores, h the half of the head dimension it accumulates.
// States are merged through LDS; a split writes (O, max, sum) partials for k_fattn_combine.
template <int D>
__global__ void __launch_bounds__(256, 2) k_fattn_mma_dec(fattn_args a, int R, int NT) {
    typedef kv_stage<D, 256> stage_t;
    constexpr int NDT = D / 64;   // 32-row O^T tiles per wave
    __shared__ __attribute__((aligned(16))) _Float16 sK[FM_BC * stage_t::KP];
    __shared__ __attribute__((aligned(16))) _Float16 sVt[FM_BC * stage_t::VP];
    float *s_merge = (float *)sK;   // reused after the last tile: per h, [D/2 + 2][32] floats of the u = 1 wave
    static_assert(sizeof(_Float16) * FM_BC * stage_t::KP >= sizeof(float) * (D + 4) * 32, "merge buffer does not fit the K tile");

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    const int u = wave & 1, h = wave >> 1;
    const int split = blockIdx.x;
    const int64_t hk = blockIdx.y;
    const int col_tok = l32 / R, col_head = l32 % R;
    const bool col_live = col_tok < NT && (int64_t)blockIdx.z * NT + col_tok < a.Nq;
    const int64_t iq = col_live ? (int64_t)blockIdx.z * NT + col_tok : a.Nq - 1;
    const int64_t head = hk * R + (col_live ? col_head : 0);

    f16x8 qf[D / 16];
    load_q<D>(qf, (const float *)(a.q + iq * a.q_nb1 + head * a.q_nb2), lhi);
    const float slope = alibi_slope(a, head);
    const float scale = a.softcap != 0.0f ? a.scale / a.softcap : a.scale;
    const unsigned short *mrow = a.mask ? (const unsigned short *)(a.mask + iq * a.mask_nb1) : nullptr;
    const bool mask_aligned = (((uintptr_t)a.mask | a.mask_nb1) & 7) == 0;

    f32x16 o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[dt][r] = 0.0f;
    float m = FM_NEG, l = 0.0f;

    const int64_t c_begin = (int64_t)split * a.cells_per_split;
    const int64_t c_end = c_begin + a.cells_per_split < a.Nkv ? c_begin + a.cells_per_split : a.Nkv;

    // two tiles of K/V (and their mask entries) are always in flight: tile i + 2 is requested as soon as the
    // registers of tile i have been written to LDS
    stage_t st0, st1;
    u32x2 mn0[4], mn1[4];
    auto prefetch = [&](stage_t &st, u32x2 (&mn)[4], int64_t kv0) {
        st.fetch(a, hk, kv0, tid);
        fetch_mask<4>(mn, mrow, mask_aligned && kv0 + FM_BC <= a.Nkv, kv0 + 32 * u + 4 * lhi, a.Nkv);
    };
    auto tile = [&](stage_t &st, u32x2 (&mn)[4], int64_t kv0) {
        __syncthreads();   // the previous tile has been consumed
        st.commit(sK, sVt, tid);
        u32x2 mcur[4];
#pragma unroll
        for (int g = 0; g < 4; g++) mcur[g] = mn[g];
        __syncthreads();
        if (kv0 + 2 * FM_BC < c_end) prefetch(st, mn, kv0 + 2 * FM_BC);
        f32x16 S = scores<D>(qf, sK, u, l32, lhi);
        float mx = finish_scores_dec(S, mcur, a, scale, slope, kv0 + 32 * u, lhi, c_end);
        mx = half_pair_max(mx);
        if (__ballot(mx > FM_NEG) == 0) return;   // all 32 cells masked for every column (wave-uniform)
        const float m_new = fmaxf(m, mx);
        const float alpha = __expf(m - m_new);
        float rs = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float p = S[r] > FM_NEG ? __expf(S[r] - m_new) : 0.0f;
            S[r] = p;
            rs += p;
        }
        rs = half_pair_sum(rs);
        l = l * alpha + rs;
        m = m_new;
        if (__ballot(alpha != 1.0f) != 0) {   // wave-uniform: most tiles do not raise any column's maximum
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[dt][r] *= alpha;
        }
        accumulate_pv<D, NDT>(o, S, sVt, h * NDT, u, l32, lhi);
    };
    if (c_begin < c_end) prefetch(st0, mn0, c_begin);
    if (c_begin + FM_BC < c_end) prefetch(st1, mn1, c_begin + FM_BC);
    for (int64_t kv0 = c_begin; kv0 < c_end; kv0 += 2 * FM_BC) {
        tile(st0, mn0, kv0);
        if (kv0 + FM_BC < c_end) tile(st1, mn1, kv0 + FM_BC);   // uniform over the group
    }

    // ---- merge the u = 1 wave into the u = 0 wave of the same h
    float *mg = s_merge + h * (D / 2 + 2) * 32;   // [d_local][col], then max, sum
    __syncthreads();
    if (u == 1) {
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) mg[(32 * dt + 8 * (r >> 2) + 4 * lhi + (r & 3)) * 32 + l32] = o[dt][r];
        if (lhi == 0) {
            mg[(D / 2) * 32 + l32] = m;
            mg[(D / 2 + 1) * 32 + l32] = l;
        }
    }
    __syncthreads();
    if (u != 0 || !col_live) return;
    {
        const float m1 = mg[(D / 2) * 32 + l32], l1 = mg[(D / 2 + 1) * 32 + l32];
        const float M = fmaxf(m, m1);
        const float f0 = __expf(m - M), f1 = __expf(m1 - M);
        l = l * f0 + l1 * f1;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[dt][r] = o[dt][r] * f0 + mg[(32 * dt + 8 * (r >> 2) + 4 * lhi + (r & 3)) * 32 + l32] * f1;
        m = M;
    }
    const int d_first = h * (D / 2);   // this wave's slice of the head
    if (a.n_splits == 1) {
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
        float *dp = a.dst + (iq * a.Hq + head) * D + d_first;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) {
            float w[16];
            float amax = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                w[r] = o[dt][r] * inv;
                amax = fmaxf(amax, fabsf(w[r]));
            }
#pragma unroll
            for (int g = 0; g < 4; g++) *(f32x4 *)(dp + 32 * dt + 8 * g + 4 * lhi) = f32x4{w[4 * g], w[4 * g + 1], w[4 * g + 2], w[4 * g + 3]};
            if (a.act_q) {   // Q8_1 of this 32-element block of the head (quantize_row_q8_1_ref, ggml-quants.c:220-253)
                amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
                const float d = amax / 127.0f;
                const float id = d != 0.0f ? 1.0f / d : 0.0f;
                int sum = 0;
                const int64_t e0 = head * D + d_first + 32 * dt;   // first element of the block inside the activation row
                int8_t *qrow = a.act_q + iq * a.Hq * D + e0;
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    u32 packed = 0;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int q = (int)roundf(w[4 * g + i] * id);
                        sum += q;
                        packed |= (u32)(q & 0xFF) << (8 * i);
                    }
                    *(u32 *)(qrow + 8 * g + 4 * lhi) = packed;
                }
                sum += __shfl_xor(sum, 32, 64);
                if (lhi == 0) {
                    act_ds e;
                    e.d = half_bits_to_float(float_to_half_bits(d));
                    e.sum = sum;
                    a.act_s[iq * (a.Hq * D / 32) + e0 / 32] = e;
                }
            }
        }
    } else {
        float *p = a.ws + ((iq * a.Hq + head) * a.n_splits + split) * (D + 2);
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
                for (int i = 0; i < 4; i++) p[d_first + 32 * dt + 8 * g + 4 * lhi + i] = o[dt][4 * g + i];
        if (h == 0 && lhi == 0) {
            p[D] = m;
            p[D + 1] = l;
        }
    }
}

template <int D>
int launch_dec(hipStream_t s, const fattn_args &a) {
    const int R = (int)(a.Hq / a.Hkv);
    const int NT = 32 / R;
    const dim3 grid((unsigned)a.n_splits, (unsigned)a.Hkv, (unsigned)((a.Nq + NT - 1) / NT));
    MI355_LAUNCH(k_fattn_mma_dec<D>, grid, dim3(256), 0, s, a, R, NT);
    return launch_status("k_fattn_mma_dec");
}

}  // namespace

int launch_fattn_mma(hipStream_t s, fattn_args &a, int64_t D, size_t ws_bytes) {
    if (a.Hkv * (a.Hq / a.Hkv) > 65535 || (a.Nq + 31) / 32 > 0x7fffffff) return 1;
    if ((a.q_nb1 % 16) != 0 || (a.q_nb2 % 16) != 0) return 1;
    if (D != 64 && D != 128) return 1;
    if (a.k_nb1 >= (size_t(1) << 24) || a.v_nb1 >= (size_t(1) << 24)) return 1;   // kv_stage: a tile's rows within 32-bit offsets
    a.kv_extent = nullptr;
    const int64_t n_tiles = (a.Nq + 31) / 32;
    // The pre-pass pays when there are more groups than the chip holds at once (two per compute unit): then a group that stops
    // early makes room for the next one.  With fewer groups the launch takes as long as its longest group either way.
    const int64_t n_groups = n_tiles * a.Hq / 4;
    if (n_groups > 512 && a.mask && a.ws && ws_bytes >= (size_t)n_tiles * sizeof(int32_t) && (((uintptr_t)a.mask | a.mask_nb1) & 15) == 0 &&
        a.Nkv % 8 == 0 && a.Nkv >= 2 * FM_BC && a.Nkv < 0x7fffffff) {
        MI355_LAUNCH(k_mask_extent, dim3((unsigned)n_tiles), dim3(256), 0, s, a.mask, a.mask_nb1, a.Nq, a.Nkv, (int32_t *)a.ws);
        const int rc = launch_status("k_mask_extent");
        if (rc != MI355_OK) return rc;
        a.kv_extent = (const int32_t *)a.ws;
    }
    // few query tiles (a batch of a few hundred rows): twice the groups with half a K/V tile per wave, while the chip is not full
    const int64_t R = a.Hq / a.Hkv;
    if (R % 2 == 0 && n_tiles * a.Hkv * (R / 2) <= 512) {
        switch (D) {
            case 64: return launch_half<64>(s, a);
            case 128: return launch_half<128>(s, a);
        }
    }
    switch (D) {
        case 64: return launch_hpw<64>(s, a);
        case 128: return launch_hpw<128>(s, a);
        default: return 1;   // other head sizes stay on the vector kernel
    }
}

// Few query rows: returns 1 when the shape is not served.  a.n_splits / a.cells_per_split (a multiple of 64) are set by the caller.
int launch_fattn_mma_dec(hipStream_t s, fattn_args &a, int64_t D) {
    const int64_t R = a.Hq / a.Hkv;
    if (R > 32 || a.Hkv > 65535 || (a.q_nb1 % 16) != 0 || (a.q_nb2 % 16) != 0 || a.cells_per_split % FM_BC != 0) return 1;
    if ((a.Nq + (32 / R) - 1) / (32 / R) > 65535) return 1;
    if (a.k_nb1 >= (size_t(1) << 24) || a.v_nb1 >= (size_t(1) << 24)) return 1;   // kv_stage: a tile's rows within 32-bit offsets
    switch (D) {
        case 64: return launch_dec<64>(s, a);
        case 128: return launch_dec<128>(s, a);
        default: return 1;
    }
}

}  // namespace mi355
