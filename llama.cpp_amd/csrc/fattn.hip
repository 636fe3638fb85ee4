// FLASH_ATTN_EXT with grouped-query heads over an f16 KV cache; the vector kernel also reads Q8_0 / Q4_0 caches where they lie.
//
// k_fattn_vec: the HBM-bound form (decode, and any query count as a fallback).  A group
// works on one (kv head, query token, kv split).  A K or V row of D halves is read by
// D/8 neighbouring lanes with one 16-byte load each, so a wave streams 64/LPR cache cells
// per step and all R = Hq/Hkv query heads that share the kv head are served from the same
// bytes (each K/V byte leaves HBM once per query token).  q.k uses v_dot2_f32_f16 on q
// rounded to f16 (as the reference does before its f16 dot), the LPR partial sums are
// folded with DPP row operations, and every lane group keeps its own online-softmax state
// (running max, sum, R x 8 output slice); the states are merged through LDS, and across kv
// splits by k_fattn_combine.  -inf mask entries are skipped, as in the reference.
#include "common.hpp"
#include "fattn.hpp"

#include <float.h>
#include <type_traits>
#include <stdlib.h>

namespace mi355 {

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// sum over aligned groups of LPR lanes (8, 16 or 32); every lane of the group gets the sum
template <int LPR>
__device__ __forceinline__ float group_sum(float v) {
    v += dpp_mov<0xB1>(v);    // quad_perm [1,0,3,2]
    v += dpp_mov<0x4E>(v);    // quad_perm [2,3,0,1]
    v += dpp_mov<0x141>(v);   // row_half_mirror: 8 lanes
    if constexpr (LPR >= 16) v += dpp_mov<0x140>(v);   // row_mirror: 16 lanes
    if constexpr (LPR >= 32) v += __shfl_xor(v, 16, 64);
    return v;
}

__device__ __forceinline__ float dot8_f16(const u32x4 &a, const u32x4 &b) {
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        // copy the lanes out first: bit-casting a vector element expression directly reads element 0
        const u32 ai = a[i], bi = b[i];
        s = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, ai), __builtin_bit_cast(f16x2, bi), s, false);
    }
    return s;
}



// Where this lane's eight elements d0 .. d0 + 7 of the (cell 0, kv head hk) row of a quantized operand lie: their levels (Q4_0: the
// eight bytes whose low or high nibbles - shift 0 or 4 - they are) and the block's f16 scale; a cell further on they are lv_step /
// sc_step bytes further on.
struct kv_lane {
    const uint8_t *lv, *sc;
    int shift;
    int64_t lv_step, sc_step;
};
__device__ __forceinline__ kv_lane kv_lane_of(const kv_src &s, int type, int64_t hk, int d0) {
    const int BB = type == MI355_Q8_0 ? Q8_0_BYTES : Q4_0_BYTES, LB = type == MI355_Q8_0 ? 32 : 16;
    const int64_t g = s.first_block + hk * s.head_blocks + (d0 >> 5);
    const int j = d0 & 31;
    kv_lane o;
    const uint8_t *lv;
    if (s.row_blocks == 0) {
        o.sc = s.base + g * BB;
        lv = o.sc + 2;
    } else {   // cell 0's blocks lie in the owner's row that starts at s.base (kv_in_place): g < row_blocks
        lv = s.base + g * LB;
        o.sc = s.base + s.row_blocks * LB + g * 2;
    }
    o.lv = lv + (type == MI355_Q8_0 ? j : (j & 15));
    o.shift = (type == MI355_Q4_0 && j >= 16) ? 4 : 0;
    o.lv_step = s.cell_lv;
    o.sc_step = s.cell_sc;
    return o;
}
// the raw bytes of one cell's eight elements: levels in words 0 and 1, the scale's bits in word 2 (plain blocks are 2-byte aligned)
__device__ __forceinline__ u32x4 kv_load8(const kv_lane &p, int64_t cell) {
    u32x2 w;
    __builtin_memcpy(&w, p.lv + cell * p.lv_step, 8);
    return u32x4{w[0], w[1], (u32)*(const unsigned short *)(p.sc + cell * p.sc_step), 0u};
}
// d * level of the eight elements (dequantize_row_q8_0 / dequantize_row_q4_0, ggml-quants.c:255-273, 365-380)
__device__ __forceinline__ void kv_values8(int type, const u32x4 &raw, int shift, float (&f)[8]) {
    const float d = half_bits_to_float((unsigned short)raw[2]);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const u32 w = raw[i >> 2] >> (8 * (i & 3));
        f[i] = type == MI355_Q8_0 ? (float)(int8_t)(w & 0xFF) * d : (float)((int)((w >> shift) & 0xF) - 8) * d;
    }
}
// The eight levels as f16 pairs, exact: byte u in the low byte of a half whose high byte is 0x64 reads 1024 + u, and one packed
// subtraction brings it to the level (Q8_0: u = level + 128 after the sign bit is flipped; Q4_0: u = nibble, level = u - 8).
// Returns the block's scale; the dot of these levels with q is multiplied by it afterwards.
__device__ __forceinline__ float kv_levels8_f16(int type, const u32x4 &raw, int shift, u32x4 &out) {
    const bool q8 = type == MI355_Q8_0;
    const f16x2 bias = q8 ? f16x2{(_Float16)-1152.0f, (_Float16)-1152.0f} : f16x2{(_Float16)-1032.0f, (_Float16)-1032.0f};
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const u32 w = q8 ? raw[h] ^ 0x80808080u : (raw[h] >> shift) & 0x0F0F0F0Fu;
        // v_perm_b32 picks bytes of {0x64646464, w}: selector bytes 0..3 = w's bytes, 4..7 = the constant's
        const u32 lo = __builtin_amdgcn_perm(0x64646464u, w, 0x04010400u);   // halves (0x64, byte 0), (0x64, byte 1)
        const u32 hi = __builtin_amdgcn_perm(0x64646464u, w, 0x04030402u);   // halves (0x64, byte 2), (0x64, byte 3)
        const f16x2 a = __builtin_bit_cast(f16x2, lo) + bias, b = __builtin_bit_cast(f16x2, hi) + bias;
        out[2 * h] = __builtin_bit_cast(u32, a);
        out[2 * h + 1] = __builtin_bit_cast(u32, b);
    }
    return half_bits_to_float((unsigned short)raw[2]);
}

// NW: waves per group; KV: 0 = f16 K and V; 1 = K and / or V are Q8_0 / Q4_0 read in place, the types taken from a.type_k, a.type_v
// (every use of a type is then a branch, uniform but in the way of the scheduler: 10.3 us at 256 cells against 7.1 us for f16);
// 2 = both Q8_0, 3 = both Q4_0, known to the compiler
template <int D, int R, int NW = 4, int KV = 0>
__global__ void __launch_bounds__(NW * 64) k_fattn_vec(fattn_args a) {
    constexpr bool QUANT = KV != 0;
    const int type_k = KV == 2 ? MI355_Q8_0 : KV == 3 ? MI355_Q4_0 : a.type_k;
    const int type_v = KV == 2 ? MI355_Q8_0 : KV == 3 ? MI355_Q4_0 : a.type_v;
    constexpr int LPR = D <= 64 ? 8 : (D <= 128 ? 16 : 32);   // lanes per K/V row
    constexpr int CPW = 64 / LPR;                               // cells per wave step
    constexpr int SLOTS = NW * CPW;                             // independent softmax states per group
    constexpr int NT = NW * 64;
    constexpr float NEG = -FLT_MAX / 2;

    __shared__ float s_m[NW][R], s_l[NW][R];
    __shared__ float s_o[NW][R][D];

    const int split = blockIdx.x;
    const int64_t hk = blockIdx.y / a.groups, hg = blockIdx.y % a.groups, iq = blockIdx.z;
    const int64_t head0 = (hk * a.groups + hg) * R;   // first of this group's R query heads
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane % LPR, slot = wave * CPW + lane / LPR;
    const int d0 = sub * 8;
    const bool active = d0 < D;

    // q slices, rounded to f16 (ggml-cpu.c:11037-11040 converts q to the K type before the dot)
    u32x4 qh[R];
    float slope[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int64_t head = head0 + r;
        const float *qp = (const float *)(a.q + iq * a.q_nb1 + head * a.q_nb2) + d0;
        f32x4 x0 = {0, 0, 0, 0}, x1 = {0, 0, 0, 0};
        if (active) {
            x0 = *(const f32x4 *)qp;
            x1 = *(const f32x4 *)(qp + 4);
        }
#pragma unroll
        for (int i = 0; i < 2; i++) {
            f16x2 p0 = {(_Float16)x0[2 * i], (_Float16)x0[2 * i + 1]};
            f16x2 p1 = {(_Float16)x1[2 * i], (_Float16)x1[2 * i + 1]};
            qh[r][i] = __builtin_bit_cast(u32, p0);
            qh[r][2 + i] = __builtin_bit_cast(u32, p1);
        }
        // ALiBi slope of this head (ggml-cpu.c:10998-11003)
        slope[r] = 1.0f;
        if (a.max_bias > 0.0f) {
            const unsigned h = (unsigned)head;
            slope[r] = h < a.n_head_log2 ? powf(a.m0, (float)(h + 1)) : powf(a.m1, (float)(2 * (h - a.n_head_log2) + 1));
        }
    }

    float m[R], l[R], acc[R][8];
#pragma unroll
    for (int r = 0; r < R; r++) {
        m[r] = NEG;
        l[r] = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) acc[r][i] = 0.0f;
    }

    const int64_t c_begin = (int64_t)split * a.cells_per_split;
    const int64_t c_end = c_begin + a.cells_per_split < a.Nkv ? c_begin + a.cells_per_split : a.Nkv;
    const unsigned short *mrow = a.mask ? (const unsigned short *)(a.mask + iq * a.mask_nb1) : nullptr;
    const float scale = a.softcap != 0.0f ? a.scale / a.softcap : a.scale;
    // quantized operands (wave-uniform choice): this lane's place in the rows of kv head hk
    const bool k_f16 = !QUANT || type_k == MI355_F16, v_f16 = !QUANT || type_v == MI355_F16;
    kv_lane kl = {nullptr, nullptr, 0, 0, 0}, vl = {nullptr, nullptr, 0, 0, 0};
    if (!k_f16 && active) kl = kv_lane_of(a.kq, type_k, hk, d0);
    if (!v_f16 && active) vl = kv_lane_of(a.vq, type_v, hk, d0);

    // U steps of SLOTS cells at a time: all mask entries, then all K/V rows of the U steps are requested before the first
    // is used, so a short context costs one round trip to memory instead of one per step.  Cells are still folded into a
    // slot's state in ascending order.
    constexpr int U = 4;
    for (int64_t cb = c_begin; cb < c_end; cb += U * SLOTS) {
        float mv[U];
        bool valid[U];
        {
            // the U mask entries are requested together, from clamped addresses and without a branch per entry (a branch per entry
            // makes each load wait for the one before it: U round trips instead of one)
            unsigned mraw[U];   // (32-bit each: halves packed in pairs would be merged load by load, with a wait for each)
#pragma unroll
            for (int j = 0; j < U; j++) mraw[j] = 0;
            if (mrow) {   // uniform
#pragma unroll
                for (int j = 0; j < U; j++) {
                    const int64_t c = cb + j * SLOTS + slot;
                    mraw[j] = mrow[c < c_end ? c : c_end - 1];
                }
            }
            __builtin_amdgcn_sched_barrier(0);   // (or each load is moved down to its first use, and waited for there)
#pragma unroll
            for (int j = 0; j < U; j++) {
                const int64_t c = cb + j * SLOTS + slot;
                mv[j] = half_bits_to_float((unsigned short)mraw[j]);
                valid[j] = c < c_end && mv[j] != -INFINITY;
                if (c >= c_end) mv[j] = 0.0f;
            }
        }
        u32x4 kk[U], vv[U];
        if constexpr (!QUANT) {
#pragma unroll
            for (int j = 0; j < U; j++) {
                const int64_t c = cb + j * SLOTS + slot;
                kk[j] = u32x4{0, 0, 0, 0};
                vv[j] = u32x4{0, 0, 0, 0};
                if (valid[j] && active) {   // masked cells cost no K/V traffic
                    kk[j] = load16(a.k + c * a.k_nb1 + hk * a.k_nb2 + d0 * 2);
                    vv[j] = load16(a.v + c * a.v_nb1 + hk * a.v_nb2 + d0 * 2);
                }
            }
        } else if (!active) {
#pragma unroll
            for (int j = 0; j < U; j++) {
                kk[j] = u32x4{0, 0, 0, 0};
                vv[j] = u32x4{0, 0, 0, 0};
            }
        } else {
            // Quantized operands take two or three loads per row; under a branch per step the narrow ones (the scales) are waited
            // for inside it, a round trip per step (9.1 us at 256 cells of a Q8_0 cache, 7.6 without).  So no branch: a masked cell
            // reads the split's first cell instead - a row that is in use, not one that may never have been written and would come
            // from memory cold - and is zeroed afterwards.
#pragma unroll
            for (int j = 0; j < U; j++) {
                const int64_t c = valid[j] ? cb + j * SLOTS + slot : c_begin;
                kk[j] = k_f16 ? load16(a.k + c * a.k_nb1 + hk * a.k_nb2 + d0 * 2) : kv_load8(kl, c);
                vv[j] = v_f16 ? load16(a.v + c * a.v_nb1 + hk * a.v_nb2 + d0 * 2) : kv_load8(vl, c);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < U; j++) {
                if (!valid[j]) {
                    kk[j] = u32x4{0, 0, 0, 0};
                    vv[j] = u32x4{0, 0, 0, 0};
                }
            }
        }
        float kd[U];   // quantized K: the levels as exact f16 values; their dot with q takes the block's scale afterwards
#pragma unroll
        for (int j = 0; j < U; j++) {
            kd[j] = 1.0f;
            if (!k_f16) {
                const u32x4 raw = kk[j];
                kd[j] = kv_levels8_f16(type_k, raw, kl.shift, kk[j]);
            }
        }
        // V rows as floats, then per head: the U scores (independent of each other), ONE new maximum and ONE rescale of the state,
        // and the U weighted rows - the dependent chain per step is a fraction of folding the cells one by one
        float vf[U][8];
#pragma unroll
        for (int j = 0; j < U; j++) {
            if (v_f16) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const u32 vi = vv[j][i];
                    const f16x2 h2 = __builtin_bit_cast(f16x2, vi);
                    vf[j][2 * i] = (float)h2[0];
                    vf[j][2 * i + 1] = (float)h2[1];
                }
            } else {
                kv_values8(type_v, vv[j], vl.shift, vf[j]);
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            float sj[U];
            float mn = m[r];
#pragma unroll
            for (int j = 0; j < U; j++) {
                float sc = group_sum<LPR>(k_f16 ? dot8_f16(qh[r], kk[j]) : dot8_f16(qh[r], kk[j]) * kd[j]) * scale;
                if (a.softcap != 0.0f) sc = a.softcap * tanhf(sc);
                sc += slope[r] * mv[j];
                sj[j] = valid[j] ? sc : NEG;
                mn = fmaxf(mn, sj[j]);
            }
            const float f = __expf(m[r] - mn);   // 1 when nothing changed (also while the state is still empty)
            m[r] = mn;
            l[r] *= f;
#pragma unroll
            for (int i = 0; i < 8; i++) acc[r][i] *= f;
#pragma unroll
            for (int j = 0; j < U; j++) {
                const float p = valid[j] ? __expf(sj[j] - mn) : 0.0f;
                l[r] += p;
#pragma unroll
                for (int i = 0; i < 8; i++) acc[r][i] += p * vf[j][i];
            }
        }
    }

    // merge the states: first the CPW lane groups of a wave (cross-lane), then the NW waves through LDS
#pragma unroll
    for (int r = 0; r < R; r++) {
        // (a lane and its partner end up with the same merged state: the pair is taken in one order by both)
        auto merge_step = [&](auto off_c) {
            constexpr int OFF = decltype(off_c)::value;
            if constexpr (OFF >= LPR) {
                const lane_pair pm = lanes_pair<OFF>(m[r]), pl = lanes_pair<OFF>(l[r]);
                const float M = fmaxf(pm.a, pm.b);
                const float fa = __expf(pm.a - M), fb = __expf(pm.b - M);
                l[r] = pl.a * fa + pl.b * fb;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const lane_pair pa = lanes_pair<OFF>(acc[r][i]);
                    acc[r][i] = pa.a * fa + pa.b * fb;
                }
                m[r] = M;
            }
        };
        merge_step(std::integral_constant<int, 8>{});
        merge_step(std::integral_constant<int, 16>{});
        merge_step(std::integral_constant<int, 32>{});
        if (lane == 0) {
            s_m[wave][r] = m[r];
            s_l[wave][r] = l[r];
        }
        if (active && lane < LPR) {
#pragma unroll
            for (int i = 0; i < 8; i++) s_o[wave][r][d0 + i] = acc[r][i];
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < R * D; idx += NT) {
        const int r = idx / D, d = idx % D;
        float M = NEG;
#pragma unroll
        for (int s = 0; s < NW; s++) M = fmaxf(M, s_m[s][r]);
        float L = 0.0f, O = 0.0f;
#pragma unroll
        for (int s = 0; s < NW; s++) {
            const float f = __expf(s_m[s][r] - M);
            L += s_l[s][r] * f;
            O += s_o[s][r][d] * f;
        }
        const int64_t head = head0 + r;
        if (a.n_splits == 1) {
            const float o = O / L;
            a.dst[(iq * a.Hq + head) * D + d] = o;
            if (a.act_q) quantize_lane32(o, a.act_q + iq * a.Hq * D, a.act_s + iq * (a.Hq * D / 32), head * D + d);
        } else {
            float *p = a.ws + ((iq * a.Hq + head) * a.n_splits + split) * (D + 2);
            p[d] = O;
            if (d == 0) {
                p[D] = M;
                p[D + 1] = L;
            }
        }
    }
}

// Merge of the kv splits, one 512-thread group per (token, head).  The partial results were written by other compute units a
// moment ago, so every load is a trip to memory: a thread asks for its split's (max, sum) pair and for the first sixteen partial
// outputs of its element before it uses any of them.  Thread tid owns element tid % D and the splits tid / D, tid / D + PARTS, ...
// (PARTS = 512 / D); the parts are added through LDS.
template <int D>
__global__ void __launch_bounds__(512) k_fattn_combine(const float *__restrict__ ws, float *__restrict__ dst, int n_splits, int8_t *__restrict__ act_q,
                                                       act_ds *__restrict__ act_s, int64_t Hq) {
    constexpr int PARTS = 512 / D, U = 16;
    __shared__ float s_w[256];
    __shared__ float s_red[16];
    __shared__ float s_o[PARTS][D];
    const int64_t row = blockIdx.x;   // iq * Hq + head
    const float *p = ws + row * n_splits * (D + 2);
    const int tid = threadIdx.x, d = tid % D, part = tid / D;
    const bool live = part < PARTS;   // head sizes that do not divide 512 leave the last threads without an element
    float ms = -FLT_MAX / 2, ls = 0.0f;
    if (tid < n_splits) {
        ms = p[tid * (D + 2) + D];
        ls = p[tid * (D + 2) + D + 1];
    }
    float v[U];
#pragma unroll
    for (int i = 0; i < U; i++) {
        const int sidx = part + PARTS * i;
        v[i] = live && sidx < n_splits ? p[sidx * (D + 2) + d] : 0.0f;
    }
    float M = wave_max_dpp(ms);
    if ((tid & 63) == 0) s_red[tid >> 6] = M;
    __syncthreads();
    M = s_red[0];
#pragma unroll
    for (int i = 1; i < 8; i++) M = fmaxf(M, s_red[i]);
    const float w = tid < n_splits ? __expf(ms - M) : 0.0f;
    if (tid < 256) s_w[tid] = w;
    float L = wave_sum_dpp(ls * w);
    if ((tid & 63) == 0) s_red[8 + (tid >> 6)] = L;
    __syncthreads();
    L = s_red[8];
#pragma unroll
    for (int i = 1; i < 8; i++) L += s_red[8 + i];
    float O = 0.0f;
#pragma unroll
    for (int i = 0; i < U; i++) {
        const int sidx = part + PARTS * i;
        if (sidx < n_splits) O += v[i] * s_w[sidx];
    }
    for (int s0 = PARTS * U; s0 < n_splits; s0 += PARTS * U) {   // more than PARTS * 16 splits
#pragma unroll
        for (int i = 0; i < U; i++) {
            const int sidx = s0 + part + PARTS * i;
            v[i] = live && sidx < n_splits ? p[sidx * (D + 2) + d] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < U; i++) {
            const int sidx = s0 + part + PARTS * i;
            if (sidx < n_splits) O += v[i] * s_w[sidx];
        }
    }
    if (live) s_o[part][d] = O;
    __syncthreads();
    if (part == 0) {   // threads 0 .. D - 1: whole 32-lane runs where the output is also quantized (D % 32 == 0 then)
#pragma unroll
        for (int i = 1; i < PARTS; i++) O += s_o[i][d];
        const float o = O / L;
        dst[row * D + d] = o;
        if (act_q) {
            const int64_t iq = row / Hq, head = row % Hq;
            quantize_lane32(o, act_q + iq * Hq * D, act_s + iq * (Hq * D / 32), head * D + d);
        }
    }
}

static int pick_splits(int64_t Nkv, int64_t Hkv, int64_t Nq) {
    int64_t by_len = (Nkv + 255) / 256;
    int64_t by_fill = 2048 / (Hkv * Nq > 0 ? Hkv * Nq : 1);
    int64_t n = by_len < by_fill ? by_len : by_fill;
    if (n < 1) n = 1;
    if (n > 256) n = 256;
    return (int)n;
}

template <int D, int R, int NW = 4>
static int launch_vec(hipStream_t s, fattn_args &a) {
    const bool quant = a.type_k != MI355_F16 || a.type_v != MI355_F16;
    a.groups = (int)(a.Hq / a.Hkv) / R;
    const dim3 grid((unsigned)a.n_splits, (unsigned)(a.Hkv * a.groups), (unsigned)a.Nq);
    if constexpr (D % 32 == 0) {
        const bool same = a.type_k == a.type_v && D == 128;   // the caches llama.cpp builds with -ctk / -ctv of one type
        if (quant && same && a.type_k == MI355_Q8_0) MI355_LAUNCH((k_fattn_vec<D, R, NW, D == 128 ? 2 : 1>), grid, dim3(NW * 64), 0, s, a);
        else if (quant && same && a.type_k == MI355_Q4_0) MI355_LAUNCH((k_fattn_vec<D, R, NW, D == 128 ? 3 : 1>), grid, dim3(NW * 64), 0, s, a);
        else if (quant) MI355_LAUNCH((k_fattn_vec<D, R, NW, 1>), grid, dim3(NW * 64), 0, s, a);
        else MI355_LAUNCH((k_fattn_vec<D, R, NW, 0>), grid, dim3(NW * 64), 0, s, a);
    } else {
        if (quant) {
            set_error("flash_attn: head size %d is not a whole number of quantization blocks", D);
            return MI355_ERR_ARG;
        }
        MI355_LAUNCH((k_fattn_vec<D, R, NW, 0>), grid, dim3(NW * 64), 0, s, a);
    }
    int rc = launch_status("k_fattn_vec");
    if (rc != MI355_OK) return rc;
    if (a.n_splits > 1) {
        MI355_LAUNCH(k_fattn_combine<D>, dim3((unsigned)(a.Nq * a.Hq)), dim3(512), 0, s, a.ws, a.dst, a.n_splits, a.act_q,
                           a.act_s, a.Hq);
        rc = launch_status("k_fattn_combine");
    }
    return rc;
}

template <int D>
static int launch_vec_r(hipStream_t s, fattn_args &a, int R) {
    // R = query heads served per group from one pass over the kv head's bytes.  A short context is not bandwidth-bound but
    // a serial chain of soft-max updates per (step, head): one head per group then spreads it over R times as many waves.
    // Up to 1024 cells and few (token, head) pairs: one head per group, eight waves per group (32 cells of a D = 128 head per step,
    // four steps' loads in flight) and no split of the cells over groups, so no second launch.  Measured per decoded token of
    // the 8B model at 256 cells: 4 waves 1.897 ms, 8 waves 1.856 ms, 16 waves 1.875 ms; requesting K and V together with the mask
    // instead of after it (one round trip less per step, but masked cells - rows of the cache that may never have been written - then
    // come from memory cold, and every lane waits for them) 1.91-1.96 ms; measured again with the mask entries requested together:
    // 6.6 us for 256 cells that are all in use, but a decoded token 1.87 ms against 1.83.
    constexpr int64_t one_head_max = 1024;
    // (quantized operands cost more arithmetic per cell: from 257 cells on their cells are split over groups)
    const bool quantized = a.type_k != MI355_F16 || a.type_v != MI355_F16;
    if (a.Nkv <= one_head_max && !(quantized && a.Nkv > 256 && a.n_splits > 1)) {
        if (a.Nq * a.Hq <= 512) {   // few (token, head) pairs: the chip is far from full
            a.n_splits = 1;
            a.cells_per_split = a.Nkv;
            return launch_vec<D, 1, 8>(s, a);
        }
        return launch_vec<D, 1>(s, a);
    }
    if (R % 4 == 0) return launch_vec<D, 4>(s, a);
    if (R % 2 == 0) return launch_vec<D, 2>(s, a);
    return launch_vec<D, 1>(s, a);
}

// checks shared by the entry points and the argument block of the kernels; quantized operands skip the f16 row checks
static int fattn_fill(fattn_args &a, const float *q, const void *k, const void *v, const void *mask, float *dst, int64_t D, int64_t Nq, int64_t Nkv,
                      int64_t Hq, int64_t Hkv, size_t q_nb1, size_t q_nb2, size_t k_nb1, size_t k_nb2, size_t v_nb1, size_t v_nb2, size_t mask_nb1,
                      float scale, float max_bias, float logit_softcap, void *ws, size_t ws_bytes, void *act, bool k_f16, bool v_f16) {
    MI355_REQUIRE(D > 0 && D % 8 == 0 && D <= 256, "flash_attn: head size %lld not supported", (long long)D);
    MI355_REQUIRE(Nq > 0 && Nkv > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0, "flash_attn: bad shape");
    MI355_REQUIRE(Nq <= 65535 && Hq <= 65535, "flash_attn: too many query rows or heads for one launch");
    MI355_REQUIRE(((uintptr_t)q & 15) == 0 && q_nb1 % 16 == 0 && q_nb2 % 16 == 0, "flash_attn: q rows must be 16-byte aligned");
    MI355_REQUIRE(!k_f16 || (((uintptr_t)k & 15) == 0 && k_nb1 % 16 == 0 && k_nb2 % 16 == 0), "flash_attn: k rows must be 16-byte aligned");
    MI355_REQUIRE(!v_f16 || (((uintptr_t)v & 15) == 0 && v_nb1 % 16 == 0 && v_nb2 % 16 == 0), "flash_attn: v rows must be 16-byte aligned");
    MI355_REQUIRE(max_bias <= 0.0f || mask != nullptr, "flash_attn: max_bias needs a mask");
    MI355_REQUIRE(act == nullptr || (D % 32 == 0 && ((uintptr_t)act & 15) == 0), "flash_attn: quantized output needs head size %% 32 == 0 and a 16-byte aligned buffer");
    a.kv_extent = nullptr;
    a.act_q = (int8_t *)act;
    a.act_s = act ? (act_ds *)((int8_t *)act + Nq * Hq * D) : nullptr;
    a.q = (const uint8_t *)q; a.k = (const uint8_t *)k; a.v = (const uint8_t *)v; a.mask = (const uint8_t *)mask;
    a.dst = dst; a.ws = (float *)ws;
    a.Nq = Nq; a.Nkv = Nkv; a.Hq = Hq; a.Hkv = Hkv;
    a.q_nb1 = q_nb1; a.q_nb2 = q_nb2; a.k_nb1 = k_nb1; a.k_nb2 = k_nb2; a.v_nb1 = v_nb1; a.v_nb2 = v_nb2; a.mask_nb1 = mask_nb1;
    a.scale = scale; a.max_bias = max_bias; a.softcap = logit_softcap;
    // ALiBi base slopes, ggml-cpu.c:10986-10990
    unsigned n2 = 1;
    while (n2 * 2 <= (unsigned)Hq) n2 *= 2;
    a.n_head_log2 = n2;
    a.m0 = powf(2.0f, -(max_bias) / n2);
    a.m1 = powf(2.0f, -(max_bias / 2.0f) / n2);
    a.n_splits = pick_splits(Nkv, Hkv, Nq);
    if (a.n_splits > 1) {
        const size_t need = (size_t)Nq * (size_t)Hq * (size_t)a.n_splits * (size_t)(D + 2) * sizeof(float);
        if (ws == nullptr || ws_bytes < need) a.n_splits = 1;   // no scratch: run unsplit
    }
    a.cells_per_split = (Nkv + a.n_splits - 1) / a.n_splits;
    return MI355_OK;
}

int fattn_vec_kv(hipStream_t s, const float *q, const void *k, int type_k, const kv_src &kq, const void *v, int type_v, const kv_src &vq,
                 const void *mask, float *dst, int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv, size_t q_nb1, size_t q_nb2, size_t k_nb1,
                 size_t k_nb2, size_t v_nb1, size_t v_nb2, size_t mask_nb1, float scale, float max_bias, float logit_softcap, void *ws,
                 size_t ws_bytes, void *act) {
    fattn_args a;
    const int frc = fattn_fill(a, q, k, v, mask, dst, D, Nq, Nkv, Hq, Hkv, q_nb1, q_nb2, k_nb1, k_nb2, v_nb1, v_nb2, mask_nb1, scale, max_bias, logit_softcap,
                               ws, ws_bytes, act, type_k == MI355_F16, type_v == MI355_F16);
    if (frc != MI355_OK) return frc;
    a.type_k = type_k;
    a.type_v = type_v;
    a.kq = kq;
    a.vq = vq;
    // One token over a long cache with both operands quantized: the streaming kernel (at 1024 cells the 512 waves have two tiles
    // each; below that the vector kernel's splits are as quick)
    constexpr int64_t stream_q_min = 1024;
    if (Nq == 1 && Nkv >= stream_q_min && type_k != MI355_F16 && type_v != MI355_F16) {
        fattn_args b = a;
        const int rc = launch_fattn_dec_stream_q(s, b, D, ws_bytes);
        if (rc < 0) return rc;
        if (rc == 0) {
            MI355_LAUNCH(k_fattn_combine<128>, dim3((unsigned)(Nq * Hq)), dim3(512), 0, s, b.ws, b.dst, b.n_splits, b.act_q, b.act_s, b.Hq);
            return launch_status("k_fattn_combine");
        }
    }
    return launch_fattn_vec_any(s, a, D);
}

int launch_fattn_vec_any(hipStream_t s, fattn_args &a, int64_t D) {
    const int R = (int)(a.Hq / a.Hkv);
    switch (D) {
        case 64: return launch_vec_r<64>(s, a, R);
        case 80: return launch_vec_r<80>(s, a, R);
        case 96: return launch_vec_r<96>(s, a, R);
        case 112: return launch_vec_r<112>(s, a, R);
        case 128: return launch_vec_r<128>(s, a, R);
        case 256: return launch_vec_r<256>(s, a, R);
        default: set_error("flash_attn: head size %lld not supported", (long long)D); return MI355_ERR_ARG;
    }
}

}  // namespace mi355

using namespace mi355;

extern "C" {

size_t mi355_flash_attn_ws_bytes(int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq) {
    // worst case: 256 kv splits
    (void)Nkv;
    return (size_t)Nq * (size_t)Hq * 256 * (size_t)(D + 2) * sizeof(float);
}

int mi355_flash_attn_ext_quant(void *stream, const float *q, const void *k, const void *v, const void *mask, float *dst,
                               int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv, size_t q_nb1, size_t q_nb2,
                               size_t k_nb1, size_t k_nb2, size_t v_nb1, size_t v_nb2, size_t mask_nb1, float scale,
                               float max_bias, float logit_softcap, void *ws, size_t ws_bytes, void *act) {
    fattn_args a;
    const int frc = fattn_fill(a, q, k, v, mask, dst, D, Nq, Nkv, Hq, Hkv, q_nb1, q_nb2, k_nb1, k_nb2, v_nb1, v_nb2, mask_nb1, scale, max_bias, logit_softcap,
                               ws, ws_bytes, act, true, true);
    if (frc != MI355_OK) return frc;
    const int R = (int)(Hq / Hkv);
    hipStream_t s = (hipStream_t)stream;
    if (Nq >= 16 && act == nullptr) {   // prefill: f16 matrix cores
        const int rc = launch_fattn_mma(s, a, D, ws_bytes);
        if (rc <= 0) return rc;
    }
    // Decode and small batches over a long context: matrix cores with (token, head) columns, which read a kv head's
    // bytes once for its whole GQA group.  Short contexts are latency-bound and mostly padding (-inf mask): the
    // vector kernel, which skips masked cells before touching K/V, is quicker there.
    constexpr int64_t dec_min = 256;
    // One token over a long cache (head size 128, up to four query heads per kv head): the per-wave streaming kernel.  Measured on
    // the 32-over-8-head shape: 12.2 us against 13.7 at 4096 cells, 36 against 41 at 32768, 105 against 117 at 131072; below about
    // 3000 cells fewer than 512 of its 64-cell tiles exist and the kernel below is ahead (10.2 against 11.2 us at 2048).
    constexpr int64_t stream_min = 3072;
    // 257 .. 512 cells: one launch with a wave per 64 cells (8.4 / 8.6 us at 384 / 512 cells against 9.0 for the split form below
    // with its merge launch; up to 256 cells the vector kernel further down is ahead, 6.8 against 7.1 us)
    constexpr int64_t short_min = 256;
    constexpr int64_t short_max = 512;
    if (Nq == 1 && Nkv > short_min && Nkv <= short_max && D == 128 && R <= 4) {
        const int rc = launch_fattn_dec_short(s, a, D);
        if (rc <= 0) return rc;
    }
    if (Nq == 1 && Nkv > stream_min && D == 128 && R <= 4 && ws != nullptr) {
        fattn_args b = a;
        const int rc = launch_fattn_dec_stream(s, b, D, ws_bytes);
        if (rc < 0) return rc;
        if (rc == 0) {
            MI355_LAUNCH(k_fattn_combine<128>, dim3((unsigned)(Nq * Hq)), dim3(512), 0, s, b.ws, b.dst, b.n_splits, b.act_q, b.act_s, b.Hq);
            return launch_status("k_fattn_combine");
        }
    }
    if (Nq < 16 && Nkv > dec_min && (D == 64 || D == 128) && R <= 32) {
        fattn_args b = a;
        // enough splits to put about two groups on every CU; a split is a whole number of 64-cell tiles
        const int64_t tiles = (Nkv + 63) / 64;
        const int64_t nt = 32 / R, base = Hkv * ((Nq + nt - 1) / nt);
        constexpr int64_t target_groups = 512;
        int64_t n = target_groups / base;
        if (n > tiles) n = tiles;
        if (n > 256) n = 256;
        if (n < 1) n = 1;
        if (n > 1 && (ws == nullptr || ws_bytes < (size_t)Nq * (size_t)Hq * (size_t)n * (size_t)(D + 2) * sizeof(float))) n = 1;
        const int64_t tiles_per_split = (tiles + n - 1) / n;
        b.cells_per_split = tiles_per_split * 64;
        b.n_splits = (int)((tiles + tiles_per_split - 1) / tiles_per_split);
        int rc = launch_fattn_mma_dec(s, b, D);
        if (rc < 0) return rc;
        if (rc == 0) {
            if (b.n_splits > 1) {
                switch (D) {
                    case 64: MI355_LAUNCH(k_fattn_combine<64>, dim3((unsigned)(Nq * Hq)), dim3(512), 0, s, b.ws, b.dst, b.n_splits, b.act_q, b.act_s, b.Hq); break;
                    default: MI355_LAUNCH(k_fattn_combine<128>, dim3((unsigned)(Nq * Hq)), dim3(512), 0, s, b.ws, b.dst, b.n_splits, b.act_q, b.act_s, b.Hq); break;
                }
                return launch_status("k_fattn_combine");
            }
            return MI355_OK;
        }
    }
    return launch_fattn_vec_any(s, a, D);
}

int mi355_flash_attn_ext(void *stream, const float *q, const void *k, const void *v, const void *mask, float *dst,
                         int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv, size_t q_nb1, size_t q_nb2,
                         size_t k_nb1, size_t k_nb2, size_t v_nb1, size_t v_nb2, size_t mask_nb1, float scale,
                         float max_bias, float logit_softcap, void *ws, size_t ws_bytes) {
    return mi355_flash_attn_ext_quant(stream, q, k, v, mask, dst, D, Nq, Nkv, Hq, Hkv, q_nb1, q_nb2, k_nb1, k_nb2, v_nb1, v_nb2, mask_nb1,
                                      scale, max_bias, logit_softcap, ws, ws_bytes, nullptr);
}

}  // extern "C"
