// Bandwidth-bound quantized GEMV (batch 1..8): dst[b][n] = sum_k W[n][k] * x[b][k] (+ residual).
//
// One wave owns RPW consecutive weight rows and walks them in steps of 64 chunks: every lane
// issues 16-byte streaming loads to consecutive addresses across the wave, so HBM sees long
// linear bursts.  The activation chunk (already Q8_1-quantized, L2 resident) is loaded once
// per step and reused for all RPW rows and all NCOLS activation rows.  Integer dots use
// v_dot4_i32_i8; scales are applied in f32; the wave reduces with cross-lane shuffles.
//
// One launch can serve up to four weight matrices that share the activation (Q/K/V, gate/up):
// the groups of all matrices are laid end to end in the grid, which turns three short launches
// into one long enough to fill the chip.  An optional residual is added in the epilogue.
#include "common.hpp"
#include "kv_blocks.hpp"
#include "qdot.hpp"
#include "norm_quant.hpp"
#include "ffn.hpp"

#include <math.h>
#include <stdlib.h>

namespace mi355 {

struct gemv_item {
    const uint8_t *W;
    float *dst;
    const float *residual;   // may be null; same shape/stride as dst; may alias dst
    int64_t N;
    int64_t dst_stride;
    int type;
    int first_group;         // index of this matrix's first group in the launch
    int epi;                 // EPI_*: what happens to a finished row
    int64_t nb1, nb2;        // EPI_*_CACHE: byte strides of a cache cell and of a head inside it (dst = cache base)
                             // EPI_*_QCACHE: block index of cell 0 within the tensor that owns the cache memory (dst = its data) and
                             // that tensor's blocks per row in the device row layout (0: plain ggml blocks)
    int ctype;               // EPI_*_QCACHE: MI355_Q8_0 or MI355_Q4_0
};
enum { EPI_STORE = 0, EPI_ROPE = 1, EPI_ROPE_CACHE = 2, EPI_CACHE = 3, EPI_ROPE_QCACHE = 4, EPI_QCACHE = 5 };

// rotary embedding of the Q/K rows produced by the fused QKV launch (mode 0: adjacent pairs)
struct gemv_rope {
    const int32_t *pos;      // [B] rope position of each activation row
    const int32_t *cells;    // [B] cache cell of each activation row
    const float *ff;         // frequency factors [n_dims/2] or null
    int D, n_dims;
    float theta_scale, freq_scale, ext_factor, attn_factor, corr0, corr1;
    const float *nx, *nw;    // NORM: the f32 row to normalise and the norm weights (the group quantizes it into its LDS copy itself)
    float neps;
};

// rope_yarn, same roundings as k_rope (glue.hip) and k_rope_kv_store (fused.hip); ggml-cpu.c:9268-9306
__device__ __forceinline__ void rope_coeffs(const gemv_rope &a, int pos, int pair, float &c, float &s) {
    const float theta_extrap = (float)pos * powf(a.theta_scale, (float)pair) / (a.ff ? a.ff[pair] : 1.0f);
    const float theta_interp = a.freq_scale * theta_extrap;
    float theta = theta_interp, mscale = a.attn_factor;
    if (a.ext_factor != 0.0f) {
        const float yv = ((float)pair - a.corr0) / fmaxf(0.001f, a.corr1 - a.corr0);
        const float ramp = (1.0f - fminf(1.0f, fmaxf(0.0f, yv))) * a.ext_factor;
        theta = theta_interp * (1.0f - ramp) + theta_extrap * ramp;
        mscale *= 1.0f + 0.1f * logf(1.0f / a.freq_scale);
    }
    c = cosf(theta) * mscale;
    s = sinf(theta) * mscale;
}
__device__ __forceinline__ void rope_apply(float c, float s, float x0, float x1, float &y0, float &y1) {
    y0 = sub_rn(mul_rn(x0, c), mul_rn(x1, s));
    y1 = add_rn(mul_rn(x0, s), mul_rn(x1, c));
}
struct gemv_batch {
    gemv_item it[4];
    int n;
};

// COH: results are stored with device scope (written through to where every XCD sees them), for launches whose last
// group reads rows produced by other groups
// LDSA: the group copies the quantized activation (NCOLS rows of K levels, then their scales) into s_act once and its four
// waves read it from there; otherwise every wave reads it from memory.  On the 14336 x 4096 Q4_K product the activation
// reads of the 7168 waves (36 MB from L2) outweighed the 33 MB of weights and competed with them: 8.7 -> 7.9 us with the
// copy in LDS.  The first step's weight loads are issued before the copy, so the copy's round trip hides behind them.
template <int TYPE, int NCOLS, int RPW, bool QKV = false, bool COH = false, bool LDSA = false, bool NORM = false>
__device__ __forceinline__ void gemv_body(const gemv_item &m, int group, const int8_t *__restrict__ aq,
                                          const act_ds *__restrict__ ads, int K, const gemv_rope *rp = nullptr, uint8_t *s_act = nullptr) {
    typedef wq<TYPE> T;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t row0 = ((int64_t)group * 4 + wave) * RPW;
    const bool wave_live = row0 < m.N;   // uniform over the wave
    if (!LDSA && !wave_live) return;     // with the copy in LDS a wave without rows still takes its share of the copy

    const row_layout L = make_row_layout(TYPE, K);
    const int nchunks = K / T::CHUNK;
    const int nblk = K >> 5;   // Q8_1 blocks per activation row

    const uint8_t *rows[RPW];
#pragma unroll
    for (int r = 0; r < RPW; r++) {
        const int64_t row = row0 + r < m.N ? row0 + r : m.N - 1;   // clamp: tail rows recompute the last row, never stored
        rows[r] = m.W + row * L.row_bytes;
    }

    float acc[RPW][NCOLS];
#pragma unroll
    for (int r = 0; r < RPW; r++)
#pragma unroll
        for (int c = 0; c < NCOLS; c++) acc[r][c] = 0.0f;

    // QKV: lane c finishes activation row c.  Its rotation and cache cell depend on nothing the product computes, so they are
    // worked out here, while the weight loads of the first step are in flight (the empty asm keeps them from being moved
    // behind the loop, next to their use).
    float rope_c = 1.0f, rope_s = 0.0f;
    int cell = 0;
    bool rotate = false;
    if constexpr (QKV) {
        if (lane < NCOLS) {
            const gemv_rope &R = *rp;
            const int d = (int)(row0 % R.D);
            rotate = (m.epi == EPI_ROPE || m.epi == EPI_ROPE_CACHE) && d < R.n_dims;
            if (rotate) rope_coeffs(R, R.pos[lane], d >> 1, rope_c, rope_s);
            if (m.epi == EPI_ROPE_CACHE || m.epi == EPI_CACHE) cell = R.cells[lane];
        }
        asm volatile("" : "+v"(rope_c), "+v"(rope_s), "+v"(cell));
    }

    typename T::chunk w_first[RPW];
    if constexpr (LDSA) {
        const int c = lane < nchunks ? lane : nchunks - 1;
#pragma unroll
        for (int r = 0; r < RPW; r++) w_first[r] = T::load_w(rows[r], L, c);
        int8_t *s_q = (int8_t *)s_act;
        act_ds *s_ds = (act_ds *)(s_act + NCOLS * K);
        if constexpr (NORM) {   // RMS_NORM -> MUL -> Q8_1 of the one activation row straight into the group's LDS copy
            __shared__ float s_norm[4];
            rms_norm_quant_row<4, false, false>(rp->nx, rp->nw, nullptr, s_act, 0, K, 1, rp->neps, s_norm);
        } else {
            for (int i = threadIdx.x * 16; i < NCOLS * K; i += 256 * 16) *(u32x4 *)(s_q + i) = load16(aq + i);
            for (int i = threadIdx.x; i < NCOLS * nblk; i += 256) s_ds[i] = ads[i];
        }
        __syncthreads();
        if (!wave_live) return;
        aq = s_q;
        ads = s_ds;
    }

    for (int c0 = 0; c0 < nchunks; c0 += 64) {
        const int c = c0 + lane;
        if (c < nchunks) {
            typename T::chunk w[RPW];
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                if (LDSA && c0 == 0) w[r] = w_first[r];
                else w[r] = T::load_w(rows[r], L, c);
            }
#pragma unroll
            for (int col = 0; col < NCOLS; col++) {
                const typename T::act A = T::load_a(aq + (int64_t)col * K, ads + col * nblk, c);
#pragma unroll
                for (int r = 0; r < RPW; r++) {
                    const chunk_dots d = T::dots(w[r], A);
                    acc[r][col] = T::accumulate(acc[r][col], w[r], A, d);
                }
            }
        }
    }

    if constexpr (QKV) {
        // RPW == 2: the wave owns the adjacent rows (row0, row0 + 1) = one rotation pair of one head.
        // Every lane gets all sums; lane c finishes activation row c.
        static_assert(RPW == 2, "the rope epilogue pairs the two rows of a wave");
        float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
        for (int c = 0; c < NCOLS; c++) {
            const float a0 = wave_sum_dpp(acc[0][c]), a1 = wave_sum_dpp(acc[1][c]);
            if (lane == c) { s0 = a0; s1 = a1; }
        }
        if (lane < NCOLS && row0 + 1 < m.N) {
            const gemv_rope &R = *rp;
            const int64_t head = row0 / R.D;
            const int d = (int)(row0 % R.D);
            float y0 = s0, y1 = s1;
            if (rotate) rope_apply(rope_c, rope_s, s0, s1, y0, y1);
            if (m.epi == EPI_ROPE || m.epi == EPI_STORE) {
                float *o = m.dst + lane * m.dst_stride + row0;
                o[0] = y0;
                o[1] = y1;
            } else {
                _Float16 *o = (_Float16 *)((uint8_t *)m.dst + (int64_t)cell * m.nb1 + head * m.nb2) + d;
                o[0] = (_Float16)y0;
                o[1] = (_Float16)y1;
            }
        }
    } else {
#pragma unroll
        for (int r = 0; r < RPW; r++)
#pragma unroll
            for (int c = 0; c < NCOLS; c++) {
                const float s = wave_sum_dpp(acc[r][c]);
                if (lane == 0 && row0 + r < m.N) {
                    const int64_t o = c * m.dst_stride + row0 + r;
                    const float v = m.residual ? s + m.residual[o] : s;
                    if constexpr (COH) __hip_atomic_store(m.dst + o, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    else m.dst[o] = v;
                }
            }
    }
}

// The Q/K/V launch when K and / or V go to a Q8_0 / Q4_0 cache: groups of EIGHT waves.  QUANT: the group's 32 rows (four per wave)
// are one block of a cache row; the finished, rotated values meet in LDS and wave c quantizes the block of activation row c
// (quantize_row_q8_0_ref / quantize_row_q4_0_ref, as the cache copies of kv_quant.hip do); m.N is a multiple of 32, so every wave is
// live.  !QUANT: 16 rows per group (two per wave) with the epilogues of gemv_body.  Every row sum is formed exactly as in gemv_body.
// (Groups of four waves that took their eight rows each in two passes of four were measured first: 14.6 us against 10.3 us for the
// launch with f16 stores on the Llama-8B shapes - the groups of 32 rows ran twice as long as the others.)
template <int TYPE, int NCOLS, bool NORM, bool QUANT>
__device__ __forceinline__ void gemv_body_qc(const gemv_item &m, int group, const int8_t *__restrict__ aq, const act_ds *__restrict__ ads, int K,
                                             const gemv_rope &R, uint8_t *s_act) {
    typedef wq<TYPE> T;
    constexpr int NW = 8, RPW = QUANT ? 4 : 2, NP = RPW / 2;
    static_assert(NCOLS <= 4, "wave c quantizes activation row c");
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t row0 = ((int64_t)group * NW + wave) * RPW;
    const bool wave_live = row0 < m.N;   // uniform over the wave; always true with QUANT
    if (!NORM && !wave_live) return;     // with NORM a wave without rows still takes its share of the norm and its barriers
    const row_layout L = make_row_layout(TYPE, K);
    const int nchunks = K / T::CHUNK;
    const int nblk = K >> 5;

    const uint8_t *rows[RPW];
#pragma unroll
    for (int r = 0; r < RPW; r++) {
        const int64_t row = row0 + r < m.N ? row0 + r : m.N - 1;   // clamp: tail rows recompute the last row, never stored
        rows[r] = m.W + row * L.row_bytes;
    }

    float rope_c[NP], rope_s[NP];
    bool rotate[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) {
        rope_c[p] = 1.0f;
        rope_s[p] = 0.0f;
        rotate[p] = false;
    }
    int cell = 0;
    if (lane < NCOLS) {
        const bool rope_epi = m.epi == EPI_ROPE || m.epi == EPI_ROPE_CACHE || m.epi == EPI_ROPE_QCACHE;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int d = (int)((row0 + 2 * p) % R.D);
            rotate[p] = rope_epi && d < R.n_dims;
            if (rotate[p]) rope_coeffs(R, R.pos[lane], d >> 1, rope_c[p], rope_s[p]);
        }
        if (m.epi == EPI_ROPE_CACHE || m.epi == EPI_CACHE) cell = R.cells[lane];
    }
#pragma unroll
    for (int p = 0; p < NP; p++) asm volatile("" : "+v"(rope_c[p]), "+v"(rope_s[p]));
    asm volatile("" : "+v"(cell));

    typename T::chunk w_first[RPW];
    if constexpr (NORM) {   // as in gemv_body: the first step's weights are on their way while the group normalises and quantizes the row
        const int c = lane < nchunks ? lane : nchunks - 1;
#pragma unroll
        for (int r = 0; r < RPW; r++) w_first[r] = T::load_w(rows[r], L, c);
        __shared__ float s_norm[4];
        if (threadIdx.x < 256) rms_norm_quant_row<4, false, false>(R.nx, R.nw, nullptr, s_act, 0, K, 1, R.neps, s_norm);
        else __syncthreads();   // the one barrier inside the norm
        __syncthreads();
        if (!wave_live) return;
        aq = (const int8_t *)s_act;
        ads = (const act_ds *)(s_act + NCOLS * K);
    }

    float acc[RPW][NCOLS];
#pragma unroll
    for (int r = 0; r < RPW; r++)
#pragma unroll
        for (int c = 0; c < NCOLS; c++) acc[r][c] = 0.0f;
    for (int c0 = 0; c0 < nchunks; c0 += 64) {
        const int c = c0 + lane;
        if (c < nchunks) {
            typename T::chunk w[RPW];
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                if (NORM && c0 == 0) w[r] = w_first[r];
                else w[r] = T::load_w(rows[r], L, c);
            }
#pragma unroll
            for (int col = 0; col < NCOLS; col++) {
                const typename T::act A = T::load_a(aq + (int64_t)col * K, ads + col * nblk, c);
#pragma unroll
                for (int r = 0; r < RPW; r++) {
                    const chunk_dots d = T::dots(w[r], A);
                    acc[r][col] = T::accumulate(acc[r][col], w[r], A, d);
                }
            }
        }
    }
    float sv[RPW];
#pragma unroll
    for (int r = 0; r < RPW; r++) sv[r] = 0.0f;
#pragma unroll
    for (int r = 0; r < RPW; r++)
#pragma unroll
        for (int c = 0; c < NCOLS; c++) {
            const float a = wave_sum_dpp(acc[r][c]);
            if (lane == c) sv[r] = a;
        }
    if constexpr (QUANT) {
        __shared__ float s_blk[NCOLS][32];
        if (lane < NCOLS) {
#pragma unroll
            for (int p = 0; p < NP; p++) {
                float y0 = sv[2 * p], y1 = sv[2 * p + 1];
                if (rotate[p]) rope_apply(rope_c[p], rope_s[p], sv[2 * p], sv[2 * p + 1], y0, y1);
                s_blk[lane][wave * RPW + 2 * p] = y0;
                s_blk[lane][wave * RPW + 2 * p + 1] = y1;
            }
        }
        __syncthreads();
        if (wave < NCOLS) {
            const int j = lane & 31;
            const float v = s_blk[wave][j];
            const int64_t g = m.nb1 + (int64_t)R.cells[wave] * (m.N >> 5) + group;
            const kv_place pl = {0, m.nb2};
            int64_t lv, sc;
            if (m.ctype == MI355_Q8_0) {
                kv_block_offsets<MI355_Q8_0>(pl, g, lv, sc);
                kv_store_q8_0_lane32(v, j, (uint8_t *)m.dst, lv, sc, lane < 32);
            } else {
                kv_block_offsets<MI355_Q4_0>(pl, g, lv, sc);
                kv_store_q4_0_lane32(v, j, (uint8_t *)m.dst, lv, sc, lane < 32);
            }
        }
    } else if (lane < NCOLS && row0 + 1 < m.N) {
        const int64_t head = row0 / R.D;
        const int d = (int)(row0 % R.D);
        float y0 = sv[0], y1 = sv[1];
        if (rotate[0]) rope_apply(rope_c[0], rope_s[0], sv[0], sv[1], y0, y1);
        if (m.epi == EPI_ROPE || m.epi == EPI_STORE) {
            float *o = m.dst + lane * m.dst_stride + row0;
            o[0] = y0;
            o[1] = y1;
        } else {
            _Float16 *o = (_Float16 *)((uint8_t *)m.dst + (int64_t)cell * m.nb1 + head * m.nb2) + d;
            o[0] = (_Float16)y0;
            o[1] = (_Float16)y1;
        }
    }
}

// dynamic LDS of the launches below: the group's copy of the activation (LDSA), act_lds_bytes() bytes
extern __shared__ __attribute__((aligned(16))) uint8_t s_act_dyn[];

template <int NCOLS, int RPW, bool COH = false, bool LDSA = false>
__device__ __forceinline__ void gemv_dispatch(const gemv_item &m, int group, const int8_t *__restrict__ aq,
                                              const act_ds *__restrict__ ads, int K) {
#define MI355_BODY(TY) gemv_body<TY, NCOLS, RPW, false, COH, LDSA>(m, group, aq, ads, K, nullptr, s_act_dyn);
    MI355_WEIGHT_TYPE_SWITCH(m.type, MI355_BODY)   // uniform over the group
#undef MI355_BODY
}

// Q, K and V projections in one launch; finished rows are rotated and land in q (f32) or in the f16 KV cache
template <int NCOLS, bool LDSA>
__global__ void __launch_bounds__(256) k_gemv_qkv(gemv_batch b, const int8_t *__restrict__ aq, const act_ds *__restrict__ ads, int K, gemv_rope rp) {
    const int g = blockIdx.x;
    int i = 0;
#pragma unroll
    for (int j = 1; j < 3; j++)
        if (g >= b.it[j].first_group) i = j;   // unused items start at INT_MAX
    const gemv_item &m = b.it[i];
    const int group = g - m.first_group;
#define MI355_BODY(TY) gemv_body<TY, NCOLS, 2, true, false, LDSA>(m, group, aq, ads, K, &rp, s_act_dyn);
    MI355_WEIGHT_TYPE_SWITCH(m.type, MI355_BODY)   // uniform over the group
#undef MI355_BODY
}

// single matrix, type known at compile time (smallest code, used by mi355_mul_mat_vec_q)
template <int TYPE, int NCOLS, int RPW, bool LDSA>
__global__ void __launch_bounds__(256) k_gemv_q(gemv_item m, const int8_t *__restrict__ aq, const act_ds *__restrict__ ads, int K) {
    gemv_body<TYPE, NCOLS, RPW, false, false, LDSA>(m, blockIdx.x, aq, ads, K, nullptr, s_act_dyn);
}

// ... with the RMS norm of the layer input computed by every group for itself (one activation row)
__global__ void __launch_bounds__(256) k_gemv_qkv_norm(gemv_batch b, int K, gemv_rope rp) {
    const int g = blockIdx.x;
    int i = 0;
#pragma unroll
    for (int j = 1; j < 3; j++)
        if (g >= b.it[j].first_group) i = j;
    const gemv_item &m = b.it[i];
    const int group = g - m.first_group;
#define MI355_BODY(TY) gemv_body<TY, 1, 2, true, false, true, true>(m, group, nullptr, nullptr, K, &rp, s_act_dyn);
    MI355_WEIGHT_TYPE_SWITCH(m.type, MI355_BODY)
#undef MI355_BODY
}

// The same two launches with K and / or V going to a Q8_0 / Q4_0 cache (gemv_body_qc): 512 threads per group; the matrices with a
// quantized destination have groups of 32 rows, one cache block per group, the others groups of 16.  The host lists the groups
// of 32 rows first in the grid.  (With f16 caches these groups of eight waves decode the 8B model at 536 tokens/s against 542 for
// the groups of four of k_gemv_qkv_norm, which therefore keeps them.)
__device__ __forceinline__ int qkv_item_of(const gemv_batch &b, int g) {
    int i = 0, best = -1;
#pragma unroll
    for (int j = 0; j < 3; j++)
        if (g >= b.it[j].first_group && b.it[j].first_group > best) {   // unused items start at INT_MAX
            i = j;
            best = b.it[j].first_group;
        }
    return i;
}

template <int NCOLS>
__global__ void __launch_bounds__(512, (NCOLS == 1 ? 4 : 2)) k_gemv_qkv_qc(gemv_batch b, const int8_t *__restrict__ aq, const act_ds *__restrict__ ads, int K, gemv_rope rp) {
    const gemv_item &m = b.it[qkv_item_of(b, blockIdx.x)];
    const int group = blockIdx.x - m.first_group;
    if (m.epi >= EPI_ROPE_QCACHE) {   // uniform over the group
#define MI355_BODY(TY) gemv_body_qc<TY, NCOLS, false, true>(m, group, aq, ads, K, rp, nullptr);
        MI355_WEIGHT_TYPE_SWITCH(m.type, MI355_BODY)
#undef MI355_BODY
    } else {
#define MI355_BODY(TY) gemv_body_qc<TY, NCOLS, false, false>(m, group, aq, ads, K, rp, nullptr);
        MI355_WEIGHT_TYPE_SWITCH(m.type, MI355_BODY)
#undef MI355_BODY
    }
}

__global__ void __launch_bounds__(512, 4) k_gemv_qkv_norm_qc(gemv_batch b, int K, gemv_rope rp) {
    const gemv_item &m = b.it[qkv_item_of(b, blockIdx.x)];
    const int group = blockIdx.x - m.first_group;
    if (m.epi >= EPI_ROPE_QCACHE) {
#define MI355_BODY(TY) gemv_body_qc<TY, 1, true, true>(m, group, nullptr, nullptr, K, rp, s_act_dyn);
        MI355_WEIGHT_TYPE_SWITCH(m.type, MI355_BODY)
#undef MI355_BODY
    } else {
#define MI355_BODY(TY) gemv_body_qc<TY, 1, true, false>(m, group, nullptr, nullptr, K, rp, s_act_dyn);
        MI355_WEIGHT_TYPE_SWITCH(m.type, MI355_BODY)
#undef MI355_BODY
    }
}

// several matrices sharing one activation
template <int NCOLS, int RPW, bool LDSA>
__global__ void __launch_bounds__(256) k_gemv_multi(gemv_batch b, const int8_t *__restrict__ aq, const act_ds *__restrict__ ads, int K) {
    const int g = blockIdx.x;
    int i = 0;
#pragma unroll
    for (int j = 1; j < 4; j++)
        if (j < b.n && g >= b.it[j].first_group) i = j;
    gemv_dispatch<NCOLS, RPW, false, LDSA>(b.it[i], g - b.it[i].first_group, aq, ads, K);
}

// ---- a launch whose last-arriving groups also do the nodes that follow the product ------------
// Every group stores its rows with device scope and waits for those stores (an explicit vmcnt wait), then
// one thread takes a ticket from the counter of its 32-row block.  The group that draws the last
// ticket of a block knows that all of the block's rows have been written, reads them back with
// device-scope loads, finishes the follow-up nodes and re-arms the counter for the next launch.  No
// cache-wide fence is involved (a device-scope fence per group writes back and invalidates the
// whole L2 and made a decoded token 10x slower), counters are shared by 8 groups only (one counter
// for a whole launch serialises ~1000 device-scope atomics), and nobody waits for anybody, so
// there is nothing that could hang.
// The same scheme for the RMS norm that follows wo / ffn_down (last group of the whole launch normalises the row; tickets on
// two levels) was measured and dropped: store acknowledgement, two dependent device-scope atomics and the device-scope
// read-back are ~2 us each and all on the critical path of a 4-10 us launch, 12 us in total against 5.8 us for the separate
// norm launch.  Here the block tails overlap with the other blocks' products and only the last one is exposed.
struct gemv_tail {
    unsigned *counters;     // one per 32-row block; zero before the first launch, left zero by every launch
    int8_t *act_q;          // quantized output, split activation layout
    act_ds *act_s;
    const float *x2;        // rows of the second matrix (up), same stride as the first
    int n;                  // elements per output row (N of the matrices)
};

__device__ __forceinline__ float load_coherent(const float *p) {   // bypasses caches that other XCDs cannot invalidate
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// gate and up projections (llm_build_ffn, src/llama.cpp:280-320) with UNARY(SILU), MUL and the Q8_1 quantization of
// the product done per 32-row block by whichever of the block's 8 groups (4 per matrix, 8 rows each) finishes last
template <int NCOLS, bool LDSA>
__global__ void __launch_bounds__(256) k_gemv_gate_up(gemv_batch b, const int8_t *__restrict__ aq, const act_ds *__restrict__ ads, int K, gemv_tail t) {
    __shared__ unsigned s_ticket;
    const int g = blockIdx.x;
    const int i = g >= b.it[1].first_group ? 1 : 0;
    const int group = g - b.it[i].first_group;
    gemv_dispatch<NCOLS, 2, true, LDSA>(b.it[i], group, aq, ads, K);
    // Every wave waits until its device-scope stores have been acknowledged before it reaches the barrier: the
    // barrier's own wait covers LDS and scalar loads only, and a ticket that overtakes a row store would let the
    // last group read that row too early.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const int block = group >> 2;   // 8 rows per group, 32 rows per quantization block
    if (threadIdx.x == 0) s_ticket = atomicAdd(t.counters + block, 1u);
    __syncthreads();
    if (s_ticket != 7u) return;   // uniform over the group
    if (threadIdx.x == 0) t.counters[block] = 0;
    const int tid = threadIdx.x;
    for (int idx = tid; idx < 32 * NCOLS; idx += 256) {   // NCOLS <= 4: whole waves, aligned groups of 32 lanes
        const int col = idx >> 5, j = idx & 31;
        const int64_t row = (int64_t)block * 32 + j;
        const float gv = load_coherent(b.it[0].dst + col * b.it[0].dst_stride + row);
        const float uv = load_coherent(t.x2 + col * b.it[0].dst_stride + row);
        const float h = silu_fast(gv) * uv;
        quantize_lane32<false>(h, t.act_q + (int64_t)col * t.n, t.act_s + (int64_t)col * (t.n >> 5), row);
    }
}

// MUL_MAT_ID, one activation row per expert slot: blockIdx.y = slot = t * n_used + e.  The
// expert id is read on the device, so no host synchronisation is needed to route tokens.
template <int TYPE, int RPW, bool LDSA>
__global__ void __launch_bounds__(256) k_gemv_id(const uint8_t *__restrict__ as, const int8_t *__restrict__ aq,
                                                 const act_ds *__restrict__ ads, const int32_t *__restrict__ ids,
                                                 int64_t ids_stride, float *__restrict__ dst, int64_t N, int K,
                                                 int64_t n_expert, int64_t n_used, int64_t nb1) {
    const int64_t slot = blockIdx.y, t = slot / n_used, e = slot % n_used;
    int64_t ex = ids[t * ids_stride + e];
    ex = ex < 0 ? 0 : (ex >= n_expert ? n_expert - 1 : ex);   // never index outside the expert stack
    const int64_t arow = t * nb1 + e % nb1;
    const row_layout L = make_row_layout(TYPE, K);
    gemv_item m;
    m.W = as + ex * N * L.row_bytes;
    m.dst = dst + slot * N;
    m.residual = nullptr;
    m.N = N;
    m.dst_stride = N;
    m.type = TYPE;
    m.first_group = 0;
    gemv_body<TYPE, 1, RPW, false, false, LDSA>(m, blockIdx.x, aq + arow * K, ads + arow * (K >> 5), K, nullptr, s_act_dyn);
}

// Same routing for weight rows that are not 16-byte aligned (byte loads): one wave per (row, slot).
template <int TYPE>
__global__ void __launch_bounds__(64) k_gemv_id_unaligned(const uint8_t *__restrict__ as, const int8_t *__restrict__ aq,
                                                          const act_ds *__restrict__ ads, const int32_t *__restrict__ ids,
                                                          int64_t ids_stride, float *__restrict__ dst, int64_t N, int64_t K,
                                                          int64_t n_expert, int64_t n_used, int64_t nb1, row_layout L) {
    const int64_t row = blockIdx.x, slot = blockIdx.y, t = slot / n_used, e = slot % n_used;
    int64_t ex = ids[t * ids_stride + e];
    ex = ex < 0 ? 0 : (ex >= n_expert ? n_expert - 1 : ex);
    const int64_t arow = t * nb1 + e % nb1;
    const uint8_t *wrow = as + (ex * N + row) * L.row_bytes;
    const int8_t *q = aq + arow * K;
    const act_ds *ds = ads + arow * (K >> 5);
    float acc = 0.0f;
    for (int64_t i = threadIdx.x; i < K; i += 64) acc += weight_value<TYPE>(wrow, L, i) * (ds[i >> 5].d * (float)q[i]);
    acc = wave_sum(acc);
    if (threadIdx.x == 0) dst[slot * N + row] = acc;
}

// Parity dump of the integer granule dots (one wave per row, activation row 0).
template <int TYPE>
__global__ void __launch_bounds__(64) k_block_dots(const uint8_t *__restrict__ W, const int8_t *__restrict__ aq,
                                                   const act_ds *__restrict__ ads, int32_t *__restrict__ out, int64_t N, int K) {
    typedef wq<TYPE> T;
    const int lane = threadIdx.x;
    const int64_t row = blockIdx.x;
    const row_layout L = make_row_layout(TYPE, K);
    const int nchunks = K / T::CHUNK;
    const int ngran = TYPE == MI355_Q6_K ? K / 16 : K / 32;
    const uint8_t *wrow = W + row * L.row_bytes;
    for (int c0 = 0; c0 < nchunks; c0 += 64) {
        const int c = c0 + lane;
        const bool live = c < nchunks;
        const int cc = live ? c : 0;
        const typename T::chunk w = T::load_w(wrow, L, cc);
        const typename T::act A = T::load_a(aq, ads, cc);
        const chunk_dots d = T::dots(w, A);
        if (!live) continue;
        if constexpr (T::CHUNK == 32 && TYPE != MI355_Q6_K) {   // one 32-element block per chunk
            out[row * ngran + c] = d.i0;
        } else if constexpr (TYPE == MI355_Q4_K || TYPE == MI355_Q5_K) {   // chunk c = sub-blocks 2c and 2c+1 of the row
            out[row * ngran + 2 * c] = d.i0;
            out[row * ngran + 2 * c + 1] = d.i1;
        } else {   // Q6_K: 16 granules per super-block
            const int sb = c >> 3, ccc = c & 7, hf = ccc >> 2, r = ccc & 3;
            const int gi = 8 * hf + 2 * (r >> 1) + (r & 1);
            out[row * ngran + sb * 16 + gi] = d.i0;
            out[row * ngran + sb * 16 + gi + 4] = d.i1;
        }
    }
}

// rows per wave: enough waves to cover every SIMD a few times over, then amortise the
// activation reads over more rows.
static int pick_rpw(int64_t total_rows) {
    if (total_rows >= 32768) return 4;
    if (total_rows >= 8192) return 2;
    return 1;
}

// bytes of LDS for the group's copy of the activation, or 0 when every wave reads it from memory.  The copy pays when the
// launch has several generations of groups per compute unit (its round trip then hides behind other groups' loads, and the
// activation reads it saves are the larger part of the launch's L2 traffic): output projection 98.9 -> 77.5 us (6.8 TB/s),
// 14336 x 4096 8.6 -> 8.0 us.  A launch whose groups are all resident at once (wo, ffn_down, Q/K/V: ~1000 groups) is one
// dependent chain per wave, and the copy's barrier lengthens it (+0.3 to +0.7 us measured).  Up to four activation rows, and
// small enough that eight groups still fit a compute unit.
// Measured and not adopted: splitting K over the four waves of a group (each wave reads a quarter of the activation, partial
// sums meet in LDS at the end) - Q4_K 4096 x 4096 4.9 -> 4.3 us and 14336 x 4096 8.2 -> 7.9 us, but Q6_K slower throughout
// (4096 x 14336 11.2 -> 14.0 us, output projection 80 -> 87 us): its 16-byte pieces per lane then form 256-byte runs.
// Also measured and not adopted: the next step's weights requested before the current step's are used (one step of look-ahead in
// the loop below) - Q4_K 4096 x 14336 10.9 -> 10.7 us, but norm + Q/K/V 10.0 -> 10.8, Q6_K 4096 x 14336 11.9 -> 13.9, wo 4.85 -> 5.1
// and the output projection 70 -> 123 us (decode 557 -> 521 tokens/s).
// Also measured and not adopted: a fixed number of groups (512..1536) that walk the matrix, activation copied to LDS once per
// group, the next block's weights requested before the current one is contracted - bit-identical sums, but 14336 x 4096 Q4_K
// 8.3 -> 9.9..10.9 us and the output projection 50.6 -> 61..77 us: many short-lived waves keep more loads in flight than few
// long-lived ones with one block of look-ahead.
static size_t act_lds_bytes(int ncols, int64_t K, int64_t groups) {
    const int64_t bytes = (int64_t)ncols * (K + K / 4);
    return (groups >= 1536 && ncols <= 4 && bytes <= 20480) ? (size_t)bytes : 0;
}

template <int NCOLS>
static void launch_multi(int rpw, hipStream_t s, const gemv_batch &b, unsigned grid, const int8_t *aq, const act_ds *ads, int K) {
    if constexpr (NCOLS <= 4) {
        if (const size_t lds = act_lds_bytes(NCOLS, K, grid)) {
            if (rpw == 1) MI355_LAUNCH((k_gemv_multi<NCOLS, 1, true>), dim3(grid), dim3(256), lds, s, b, aq, ads, K);
            else if (rpw == 2) MI355_LAUNCH((k_gemv_multi<NCOLS, 2, true>), dim3(grid), dim3(256), lds, s, b, aq, ads, K);
            else MI355_LAUNCH((k_gemv_multi<NCOLS, 4, true>), dim3(grid), dim3(256), lds, s, b, aq, ads, K);
            return;
        }
    }
    if (rpw == 1) MI355_LAUNCH((k_gemv_multi<NCOLS, 1, false>), dim3(grid), dim3(256), 0, s, b, aq, ads, K);
    else if (rpw == 2) MI355_LAUNCH((k_gemv_multi<NCOLS, 2, false>), dim3(grid), dim3(256), 0, s, b, aq, ads, K);
    else MI355_LAUNCH((k_gemv_multi<NCOLS, 4, false>), dim3(grid), dim3(256), 0, s, b, aq, ads, K);
}

template <int TYPE, int NCOLS>
static void launch_single(int rpw, hipStream_t s, const gemv_item &m, unsigned grid, const int8_t *aq, const act_ds *ads, int K) {
    if constexpr (NCOLS <= 4) {
        if (const size_t lds = act_lds_bytes(NCOLS, K, grid)) {
            if (rpw == 1) MI355_LAUNCH((k_gemv_q<TYPE, NCOLS, 1, true>), dim3(grid), dim3(256), lds, s, m, aq, ads, K);
            else if (rpw == 2) MI355_LAUNCH((k_gemv_q<TYPE, NCOLS, 2, true>), dim3(grid), dim3(256), lds, s, m, aq, ads, K);
            else MI355_LAUNCH((k_gemv_q<TYPE, NCOLS, 4, true>), dim3(grid), dim3(256), lds, s, m, aq, ads, K);
            return;
        }
    }
    if (rpw == 1) MI355_LAUNCH((k_gemv_q<TYPE, NCOLS, 1, false>), dim3(grid), dim3(256), 0, s, m, aq, ads, K);
    else if (rpw == 2) MI355_LAUNCH((k_gemv_q<TYPE, NCOLS, 2, false>), dim3(grid), dim3(256), 0, s, m, aq, ads, K);
    else MI355_LAUNCH((k_gemv_q<TYPE, NCOLS, 4, false>), dim3(grid), dim3(256), 0, s, m, aq, ads, K);
}

template <int TYPE>
static void launch_single_cols(int rpw, int64_t B, hipStream_t s, const gemv_item &m, unsigned grid, const int8_t *aq, const act_ds *ads, int K) {
    switch (B) {
        case 1: launch_single<TYPE, 1>(rpw, s, m, grid, aq, ads, K); break;
        case 2: launch_single<TYPE, 2>(rpw, s, m, grid, aq, ads, K); break;
        case 3: launch_single<TYPE, 3>(rpw, s, m, grid, aq, ads, K); break;
        case 4: launch_single<TYPE, 4>(rpw, s, m, grid, aq, ads, K); break;
        case 5: launch_single<TYPE, 5>(rpw, s, m, grid, aq, ads, K); break;
        case 6: launch_single<TYPE, 6>(rpw, s, m, grid, aq, ads, K); break;
        case 7: launch_single<TYPE, 7>(rpw, s, m, grid, aq, ads, K); break;
        default: launch_single<TYPE, 8>(rpw, s, m, grid, aq, ads, K); break;
    }
}

static int check_gemv_args(const char *who, int type, const void *W, int64_t N, int64_t K, int64_t dst_stride) {
    MI355_REQUIRE(is_weight_type(type), "%s: unsupported weight type %d", who, type);
    MI355_REQUIRE(N > 0 && K > 0 && K < (int64_t(1) << 30), "%s: bad shape N=%lld K=%lld", who, (long long)N, (long long)K);
    MI355_REQUIRE(K % type_block_elems(type) == 0, "%s: K=%lld is not a multiple of the block size", who, (long long)K);
    MI355_REQUIRE(dst_stride >= N, "%s: dst_stride < N", who);
    MI355_REQUIRE(layout_aligned(W, make_row_layout(type, K)), "%s: weight rows are not 16-byte aligned (K=%lld)", who, (long long)K);
    return MI355_OK;
}

}  // namespace mi355

using namespace mi355;

extern "C" {

int mi355_mul_mat_vec_q(void *stream, int type, const void *W, const void *act, float *dst, int64_t N, int64_t K,
                        int64_t B, int64_t dst_stride) {
    mi355_gemv_mat m = {type, W, N, dst, dst_stride, nullptr};
    return mi355_mul_mat_vec_q_multi(stream, 1, &m, act, K, B);
}

int mi355_mul_mat_vec_q_multi(void *stream, int n_mats, const mi355_gemv_mat *mats, const void *act, int64_t K, int64_t B) {
    MI355_REQUIRE(n_mats >= 1 && n_mats <= 4, "mul_mat_vec_q_multi: 1..4 matrices per launch, got %d", n_mats);
    MI355_REQUIRE(B >= 1 && B <= 32, "mul_mat_vec_q: batch %lld outside 1..32", (long long)B);
    MI355_REQUIRE(((uintptr_t)act & 15) == 0, "mul_mat_vec_q: activation workspace is not 16-byte aligned");
    int64_t total_rows = 0;
    bool aligned = true;
    for (int i = 0; i < n_mats; i++) {
        MI355_REQUIRE(is_weight_type(mats[i].type) && K > 0 && K % type_block_elems(mats[i].type) == 0, "mul_mat_vec_q: unsupported type %d or K=%lld not a multiple of its block size", mats[i].type, (long long)K);
        aligned = aligned && layout_aligned(mats[i].W, make_row_layout(mats[i].type, K));
    }
    if (!aligned) {   // tiny / odd shapes only: byte-load kernel, one matrix at a time
        for (int i = 0; i < n_mats; i++) {
            MI355_REQUIRE(mats[i].N > 0 && mats[i].dst_stride >= mats[i].N, "mul_mat_vec_q: bad shape");
            int rc = gemv_unaligned((hipStream_t)stream, mats[i].type, mats[i].W, act, mats[i].dst, mats[i].residual, mats[i].N, K, B, mats[i].dst_stride);
            if (rc != MI355_OK) return rc;
        }
        return MI355_OK;
    }
    for (int i = 0; i < n_mats; i++) {
        int rc = check_gemv_args("mul_mat_vec_q", mats[i].type, mats[i].W, mats[i].N, K, mats[i].dst_stride);
        if (rc != MI355_OK) return rc;
        total_rows += mats[i].N;
    }
    // From five activation rows on the matrix-core kernel (skinny.hip) is ahead wherever it supports the product; a single
    // Q4_0/Q8_0/Q4_K matrix already at four (14336 x 4096 Q4_K: 14.3 -> 12.0 us, 4096 x 14336: 18.0 -> 14.6 us).
    if (B >= 5 || (B == 4 && n_mats == 1 && mats[0].type != MI355_Q6_K)) {
        bool ok = true;
        for (int i = 0; i < n_mats; i++) ok = ok && mi355_mul_mat_skinny_supported(mats[i].type, mats[i].W, K, B);
        if (ok) {
            for (int i = 0; i < n_mats; i++) {
                int rc = mi355_mul_mat_skinny(stream, mats[i].type, mats[i].W, act, mats[i].dst, mats[i].residual, mats[i].N, K, B, mats[i].dst_stride, nullptr, 0);
                if (rc != MI355_OK) return rc;
            }
            return MI355_OK;
        }
    }
    MI355_REQUIRE(B <= 8, "mul_mat_vec_q: batch %lld needs the matrix-core kernel, which does not support this product (K a multiple of 256, aligned rows)", (long long)B);
    int rpw = pick_rpw(total_rows);
    if (B > 4 && rpw > 2) rpw = 2;   // keep the accumulator tile in registers
    {   // per-type corrections, measured on the 8B shapes
        bool any_q6 = false, all_q4k = true;
        for (int i = 0; i < n_mats; i++) {
            any_q6 = any_q6 || mats[i].type == MI355_Q6_K;
            all_q4k = all_q4k && mats[i].type == MI355_Q4_K;
        }
        if (any_q6 && rpw > 2) rpw = 2;                   // 128256 x 4096 Q6_K: 79.5 -> 69.3 us with two rows per wave
        if (all_q4k && rpw == 1 && K >= 8192) rpw = 2;    // 4096 x 14336 Q4_K: 11.4 -> 10.6 us (half the activation reads)
    }
    gemv_batch b;
    b.n = n_mats;
    int64_t groups = 0;
    for (int i = 0; i < 4; i++) {
        const mi355_gemv_mat &src = mats[i < n_mats ? i : 0];
        b.it[i].W = (const uint8_t *)src.W;
        b.it[i].dst = src.dst;
        b.it[i].residual = src.residual;
        b.it[i].N = src.N;
        b.it[i].dst_stride = src.dst_stride;
        b.it[i].type = src.type;
        b.it[i].first_group = (int)groups;
        b.it[i].epi = EPI_STORE;
        b.it[i].nb1 = b.it[i].nb2 = 0;
        if (i < n_mats) groups += (src.N + 4 * rpw - 1) / (4 * rpw);
    }
    MI355_REQUIRE(groups < 0x7fffffff, "mul_mat_vec_q: too many rows for one launch");
    hipStream_t s = (hipStream_t)stream;
    const int8_t *aq = (const int8_t *)act;
    const act_ds *ads = (const act_ds *)(aq + B * K);
    if (n_mats == 1) {
#define MI355_SINGLE_LAUNCH(TY) launch_single_cols<TY>(rpw, B, s, b.it[0], (unsigned)groups, aq, ads, (int)K);
        MI355_WEIGHT_TYPE_SWITCH(mats[0].type, MI355_SINGLE_LAUNCH)
#undef MI355_SINGLE_LAUNCH
        return launch_status("k_gemv_q");
    }
    switch (B) {
        case 1: launch_multi<1>(rpw, s, b, (unsigned)groups, aq, ads, (int)K); break;
        case 2: launch_multi<2>(rpw, s, b, (unsigned)groups, aq, ads, (int)K); break;
        case 3: launch_multi<3>(rpw, s, b, (unsigned)groups, aq, ads, (int)K); break;
        case 4: launch_multi<4>(rpw, s, b, (unsigned)groups, aq, ads, (int)K); break;
        default:
            // wider batches: one launch per matrix (register budget of the type switch)
            for (int i = 0; i < n_mats; i++) {
                mi355_gemv_mat one = mats[i];
                int rc = mi355_mul_mat_vec_q_multi(stream, 1, &one, act, K, B);
                if (rc != MI355_OK) return rc;
            }
            return MI355_OK;
    }
    return launch_status("k_gemv_multi");
}

// nx != null: one activation row that every group normalises and quantizes for itself (act is not read)
static int vec_q_rope_impl(void *stream, int n_mats, const mi355_gemv_rope_mat *mats, const void *act, int64_t K, int64_t B,
                             const mi355_rope_desc *rope, const float *nx, const float *nw, float neps) {
    MI355_REQUIRE(n_mats >= 1 && n_mats <= 3 && mats != nullptr && rope != nullptr, "mul_mat_vec_q_rope: 1..3 matrices per launch");
    MI355_REQUIRE(B >= 1 && B <= 4, "mul_mat_vec_q_rope: batch %lld outside 1..4", (long long)B);
    const int64_t D = rope->head_dim;
    const int n_dims = rope->n_dims;
    MI355_REQUIRE(D > 0 && D % 2 == 0 && n_dims > 0 && n_dims <= D && n_dims % 2 == 0, "mul_mat_vec_q_rope: bad head geometry");
    MI355_REQUIRE(rope->mode == 0, "mul_mat_vec_q_rope: only the adjacent-pair rope mode is fused (mode %d)", rope->mode);
    MI355_REQUIRE(nx != nullptr || ((uintptr_t)act & 15) == 0, "mul_mat_vec_q_rope: activation workspace is not 16-byte aligned");
    MI355_REQUIRE(nx == nullptr || (B == 1 && K <= 4096 && K % 1024 == 0 && ((uintptr_t)nx & 15) == 0 && ((uintptr_t)nw & 15) == 0),
                  "rms_norm_qkv_rope_store: one row of K <= 4096 (a multiple of 1024), 16-byte aligned x and weights");
    gemv_batch b;
    b.n = n_mats;
    int64_t groups = 0;
    bool needs_pos = false, needs_cells = false, any_qc = false;
    for (int i = 0; i < n_mats; i++) any_qc = any_qc || mats[i].epilogue == MI355_EPI_ROPE_QCACHE || mats[i].epilogue == MI355_EPI_QCACHE;
    // groups of 32 rows (quantized-cache epilogues) first in the grid, then the groups of 8: pass 0 places the former
    for (int pass = 0; pass < 2; pass++) {
        for (int i = 0; i < 4; i++) {
            const mi355_gemv_rope_mat &m = mats[i < n_mats ? i : 0];
            const bool qc = m.epilogue == MI355_EPI_ROPE_QCACHE || m.epilogue == MI355_EPI_QCACHE;
            if (i < n_mats && qc != (pass == 0)) continue;
            if (i >= n_mats && pass == 0) continue;
            if (i < n_mats) {
                int rc = check_gemv_args("mul_mat_vec_q_rope", m.type, m.W, m.N, K, m.N);
                if (rc != MI355_OK) return rc;
                MI355_REQUIRE(m.epilogue >= MI355_EPI_STORE && m.epilogue <= MI355_EPI_QCACHE && m.dst != nullptr && m.N % 2 == 0,
                              "mul_mat_vec_q_rope: bad epilogue %d, missing destination or odd row count", m.epilogue);
                if (m.epilogue == MI355_EPI_STORE || m.epilogue == MI355_EPI_ROPE)
                    MI355_REQUIRE(m.dst_stride >= m.N, "mul_mat_vec_q_rope: dst_stride < N");
                else if (qc)
                    MI355_REQUIRE(((uintptr_t)m.dst & 1) == 0 && (m.dst_stride == MI355_Q8_0 || m.dst_stride == MI355_Q4_0) && m.nb1 >= 0 && m.nb2 >= 0 &&
                                      m.N % 32 == 0,
                                  "mul_mat_vec_q_rope: a quantized cache takes whole Q8_0 / Q4_0 blocks (N a multiple of 32)");
                else
                    MI355_REQUIRE(((uintptr_t)m.dst & 1) == 0 && m.nb1 % 2 == 0 && m.nb2 % 2 == 0, "mul_mat_vec_q_rope: misaligned f16 destination");
                if (m.epilogue != MI355_EPI_STORE) MI355_REQUIRE(m.N % D == 0, "mul_mat_vec_q_rope: N=%lld is not a whole number of heads", (long long)m.N);
                needs_pos = needs_pos || m.epilogue == MI355_EPI_ROPE || m.epilogue == MI355_EPI_ROPE_CACHE || m.epilogue == MI355_EPI_ROPE_QCACHE;
                needs_cells = needs_cells || m.epilogue == MI355_EPI_ROPE_CACHE || m.epilogue == MI355_EPI_CACHE || qc;
            }
            b.it[i].W = (const uint8_t *)m.W;
            b.it[i].residual = nullptr;
            b.it[i].N = m.N;
            b.it[i].type = m.type;
            b.it[i].dst = (float *)m.dst;
            b.it[i].dst_stride = m.dst_stride;
            b.it[i].nb1 = m.nb1;
            b.it[i].nb2 = m.nb2;
            b.it[i].ctype = qc ? (int)m.dst_stride : 0;
            // the kernel's epilogue codes: plain rows take the rope path with no rotation applied to them
            b.it[i].epi = m.epilogue == MI355_EPI_STORE        ? EPI_STORE
                          : m.epilogue == MI355_EPI_ROPE       ? EPI_ROPE
                          : m.epilogue == MI355_EPI_ROPE_CACHE ? EPI_ROPE_CACHE
                          : m.epilogue == MI355_EPI_CACHE      ? EPI_CACHE
                          : m.epilogue == MI355_EPI_ROPE_QCACHE ? EPI_ROPE_QCACHE
                                                               : EPI_QCACHE;
            b.it[i].first_group = i < n_mats ? (int)groups : 0x7fffffff;
            if (i < n_mats) groups += any_qc ? (qc ? m.N / 32 : (m.N + 15) / 16) : (m.N + 7) / 8;   // 8 waves x 4 or 2 rows; without quantized stores 4 waves x 2 rows
        }
    }
    MI355_REQUIRE(!needs_pos || rope->pos != nullptr, "mul_mat_vec_q_rope: rope positions missing");
    MI355_REQUIRE(!needs_cells || rope->cells != nullptr, "mul_mat_vec_q_rope: cache cells missing");
    MI355_REQUIRE(groups < 0x7fffffff, "mul_mat_vec_q_rope: too many rows for one launch");
    gemv_rope rp;
    rp.pos = rope->pos; rp.cells = rope->cells; rp.ff = rope->freq_factors;
    rp.D = (int)D; rp.n_dims = n_dims;
    rp.theta_scale = powf(rope->freq_base, -2.0f / n_dims);
    rp.freq_scale = rope->freq_scale; rp.ext_factor = rope->ext_factor; rp.attn_factor = rope->attn_factor;
    const float pi = 3.14159265358979323846f;   // ggml_rope_yarn_corr_dims, ggml/src/ggml.c:3695-3707
    const float c0 = floorf(n_dims * logf(rope->n_ctx_orig / (rope->beta_fast * 2 * pi)) / (2 * logf(rope->freq_base)));
    const float c1 = ceilf(n_dims * logf(rope->n_ctx_orig / (rope->beta_slow * 2 * pi)) / (2 * logf(rope->freq_base)));
    rp.corr0 = c0 > 0 ? c0 : 0;
    rp.corr1 = c1 < n_dims - 1 ? c1 : (float)(n_dims - 1);
    hipStream_t s = (hipStream_t)stream;
    const int8_t *aq = (const int8_t *)act;
    const act_ds *ads = (const act_ds *)(aq + B * K);
    const size_t lds = act_lds_bytes((int)B, K, groups);
    if (nx != nullptr) {
        rp.nx = nx; rp.nw = nw; rp.neps = neps;
        if (any_qc) {
            MI355_LAUNCH(k_gemv_qkv_norm_qc, dim3((unsigned)groups), dim3(512), (size_t)K + K / 4, s, b, (int)K, rp);
            return launch_status("k_gemv_qkv_norm_qc");
        }
        MI355_LAUNCH(k_gemv_qkv_norm, dim3((unsigned)groups), dim3(256), (size_t)K + K / 4, s, b, (int)K, rp);
        return launch_status("k_gemv_qkv_norm");
    }
    rp.nx = rp.nw = nullptr; rp.neps = 0.0f;
    if (any_qc) {   // every wave reads the activation from memory (L2): these launches have too few groups for the copy in LDS to pay
        switch (B) {
            case 1: MI355_LAUNCH((k_gemv_qkv_qc<1>), dim3((unsigned)groups), dim3(512), 0, s, b, aq, ads, (int)K, rp); break;
            case 2: MI355_LAUNCH((k_gemv_qkv_qc<2>), dim3((unsigned)groups), dim3(512), 0, s, b, aq, ads, (int)K, rp); break;
            case 3: MI355_LAUNCH((k_gemv_qkv_qc<3>), dim3((unsigned)groups), dim3(512), 0, s, b, aq, ads, (int)K, rp); break;
            default: MI355_LAUNCH((k_gemv_qkv_qc<4>), dim3((unsigned)groups), dim3(512), 0, s, b, aq, ads, (int)K, rp); break;
        }
        return launch_status("k_gemv_qkv_qc");
    }
    switch (B) {
        case 1:
            if (lds) MI355_LAUNCH((k_gemv_qkv<1, true>), dim3((unsigned)groups), dim3(256), lds, s, b, aq, ads, (int)K, rp);
            else MI355_LAUNCH((k_gemv_qkv<1, false>), dim3((unsigned)groups), dim3(256), 0, s, b, aq, ads, (int)K, rp);
            break;
        case 2:
            if (lds) MI355_LAUNCH((k_gemv_qkv<2, true>), dim3((unsigned)groups), dim3(256), lds, s, b, aq, ads, (int)K, rp);
            else MI355_LAUNCH((k_gemv_qkv<2, false>), dim3((unsigned)groups), dim3(256), 0, s, b, aq, ads, (int)K, rp);
            break;
        case 3:
            if (lds) MI355_LAUNCH((k_gemv_qkv<3, true>), dim3((unsigned)groups), dim3(256), lds, s, b, aq, ads, (int)K, rp);
            else MI355_LAUNCH((k_gemv_qkv<3, false>), dim3((unsigned)groups), dim3(256), 0, s, b, aq, ads, (int)K, rp);
            break;
        default:
            if (lds) MI355_LAUNCH((k_gemv_qkv<4, true>), dim3((unsigned)groups), dim3(256), lds, s, b, aq, ads, (int)K, rp);
            else MI355_LAUNCH((k_gemv_qkv<4, false>), dim3((unsigned)groups), dim3(256), 0, s, b, aq, ads, (int)K, rp);
            break;
    }
    return launch_status("k_gemv_qkv");
}

int mi355_mul_mat_vec_q_rope(void *stream, int n_mats, const mi355_gemv_rope_mat *mats, const void *act, int64_t K, int64_t B,
                             const mi355_rope_desc *rope) {
    return vec_q_rope_impl(stream, n_mats, mats, act, K, B, rope, nullptr, nullptr, 0.0f);
}

int mi355_rms_norm_mul_mat_vec_q_rope(void *stream, const float *x, const float *norm_w, float eps, int n_mats, const mi355_gemv_rope_mat *mats,
                                      int64_t K, const mi355_rope_desc *rope) {
    MI355_REQUIRE(x != nullptr && norm_w != nullptr, "rms_norm_mul_mat_vec_q_rope: missing operands");
    return vec_q_rope_impl(stream, n_mats, mats, nullptr, K, 1, rope, x, norm_w, eps);
}

int mi355_rms_norm_qkv_rope_store(void *stream, const float *x, const float *norm_w, float eps, int type_q, const void *wq, int type_k,
                                  const void *wk, int type_v, const void *wv, float *q, void *kcache, void *vcache, const int32_t *pos,
                                  const int32_t *cells, const float *freq_factors, int64_t K, int64_t H, int64_t HK, int64_t D, size_t k_nb1,
                                  size_t k_nb2, size_t v_nb1, size_t v_nb2, int n_dims, int mode, int n_ctx_orig, float freq_base,
                                  float freq_scale, float ext_factor, float attn_factor, float beta_fast, float beta_slow) {
    MI355_REQUIRE(H > 0 && HK > 0 && D > 0 && x != nullptr && norm_w != nullptr, "rms_norm_qkv_rope_store: bad head geometry or missing operands");
    mi355_gemv_rope_mat m[3];
    m[0] = mi355_gemv_rope_mat{type_q, wq, H * D, MI355_EPI_ROPE, q, H * D, 0, 0};
    m[1] = mi355_gemv_rope_mat{type_k, wk, HK * D, MI355_EPI_ROPE_CACHE, kcache, 0, (int64_t)k_nb1, (int64_t)k_nb2};
    m[2] = mi355_gemv_rope_mat{type_v, wv, HK * D, MI355_EPI_CACHE, vcache, 0, (int64_t)v_nb1, (int64_t)v_nb2};
    mi355_rope_desc r = {pos, cells, freq_factors, D, n_dims, mode, n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow};
    return vec_q_rope_impl(stream, 3, m, nullptr, K, 1, &r, x, norm_w, eps);
}

int mi355_qkv_rope_store(void *stream, int type_q, const void *wq, int type_k, const void *wk, int type_v, const void *wv, const void *act,
                         float *q, void *kcache, void *vcache, const int32_t *pos, const int32_t *cells, const float *freq_factors,
                         int64_t K, int64_t B, int64_t H, int64_t HK, int64_t D, size_t k_nb1, size_t k_nb2, size_t v_nb1, size_t v_nb2,
                         int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale, float ext_factor, float attn_factor,
                         float beta_fast, float beta_slow) {
    MI355_REQUIRE(H > 0 && HK > 0 && D > 0, "qkv_rope_store: bad head geometry");
    mi355_gemv_rope_mat m[3];
    m[0] = mi355_gemv_rope_mat{type_q, wq, H * D, MI355_EPI_ROPE, q, H * D, 0, 0};
    m[1] = mi355_gemv_rope_mat{type_k, wk, HK * D, MI355_EPI_ROPE_CACHE, kcache, 0, (int64_t)k_nb1, (int64_t)k_nb2};
    m[2] = mi355_gemv_rope_mat{type_v, wv, HK * D, MI355_EPI_CACHE, vcache, 0, (int64_t)v_nb1, (int64_t)v_nb2};
    mi355_rope_desc r = {pos, cells, freq_factors, D, n_dims, mode, n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow};
    return mi355_mul_mat_vec_q_rope(stream, 3, m, act, K, B, &r);
}

int mi355_ffn_gate_up_swiglu(void *stream, int type_gate, const void *w_gate, int type_up, const void *w_up, const void *act, float *gate,
                             float *up, int64_t out_stride, void *act_out, unsigned *counters, int64_t N, int64_t K, int64_t B) {
    MI355_REQUIRE(B >= 1 && B <= 4, "ffn_gate_up_swiglu: batch %lld outside 1..4", (long long)B);
    MI355_REQUIRE(N > 0 && N % 32 == 0 && out_stride >= N, "ffn_gate_up_swiglu: N=%lld must be a positive multiple of 32 and fit the row stride", (long long)N);
    MI355_REQUIRE(((uintptr_t)act & 15) == 0 && ((uintptr_t)act_out & 15) == 0 && counters != nullptr, "ffn_gate_up_swiglu: misaligned or missing operands");
    int rc = check_gemv_args("ffn_gate_up_swiglu", type_gate, w_gate, N, K, out_stride);
    if (rc != MI355_OK) return rc;
    rc = check_gemv_args("ffn_gate_up_swiglu", type_up, w_up, N, K, out_stride);
    if (rc != MI355_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    const int8_t *aq = (const int8_t *)act;
    const act_ds *ads = (const act_ds *)(aq + B * K);
    // both matrices of one type, the activation rows fit in LDS: the launch whose groups own whole Q8_1 blocks (ffn.hip; no counters used)
    if (type_gate == type_up && B * (K + K / 4) <= 40960 && N / 32 < 0x7fffffff)
        return launch_gate_up_blk(s, type_gate, w_gate, w_up, aq, ads, K, B, gate, up, out_stride, act_out, N);
    const int64_t per = N / 8;   // groups per matrix: 4 waves x 2 rows
    MI355_REQUIRE(2 * per < 0x7fffffff, "ffn_gate_up_swiglu: too many rows for one launch");
    gemv_batch b;
    b.n = 2;
    for (int i = 0; i < 4; i++) {
        const int j = i & 1;
        b.it[i].W = (const uint8_t *)(j ? w_up : w_gate);
        b.it[i].dst = j ? up : gate;
        b.it[i].residual = nullptr;
        b.it[i].N = N;
        b.it[i].dst_stride = out_stride;
        b.it[i].type = j ? type_up : type_gate;
        b.it[i].first_group = (int)(j * per);
        b.it[i].epi = EPI_STORE;
        b.it[i].nb1 = b.it[i].nb2 = 0;
    }
    gemv_tail t;
    t.counters = counters; t.x2 = up; t.n = (int)N;
    t.act_q = (int8_t *)act_out;
    t.act_s = (act_ds *)(t.act_q + B * N);
    const dim3 grid((unsigned)(2 * per));
    const size_t lds = act_lds_bytes((int)B, K, 2 * per);
    switch (B) {
        case 1:
            if (lds) MI355_LAUNCH((k_gemv_gate_up<1, true>), grid, dim3(256), lds, s, b, aq, ads, (int)K, t);
            else MI355_LAUNCH((k_gemv_gate_up<1, false>), grid, dim3(256), 0, s, b, aq, ads, (int)K, t);
            break;
        case 2:
            if (lds) MI355_LAUNCH((k_gemv_gate_up<2, true>), grid, dim3(256), lds, s, b, aq, ads, (int)K, t);
            else MI355_LAUNCH((k_gemv_gate_up<2, false>), grid, dim3(256), 0, s, b, aq, ads, (int)K, t);
            break;
        case 3:
            if (lds) MI355_LAUNCH((k_gemv_gate_up<3, true>), grid, dim3(256), lds, s, b, aq, ads, (int)K, t);
            else MI355_LAUNCH((k_gemv_gate_up<3, false>), grid, dim3(256), 0, s, b, aq, ads, (int)K, t);
            break;
        default:
            if (lds) MI355_LAUNCH((k_gemv_gate_up<4, true>), grid, dim3(256), lds, s, b, aq, ads, (int)K, t);
            else MI355_LAUNCH((k_gemv_gate_up<4, false>), grid, dim3(256), 0, s, b, aq, ads, (int)K, t);
            break;
    }
    return launch_status("k_gemv_gate_up");
}

// act: split layout of nb1*T quantized rows of b.  dst [N, n_used, T] contiguous.
int mi355_mul_mat_id_vec(void *stream, int type, const void *as, const void *act, const int32_t *ids, int64_t ids_stride,
                         float *dst, int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T) {
    MI355_REQUIRE(is_weight_type(type), "mul_mat_id: unsupported weight type %d", type);
    MI355_REQUIRE(N > 0 && K > 0 && K < (int64_t(1) << 30) && n_expert > 0 && n_used > 0 && nb1 > 0 && T > 0, "mul_mat_id: bad shape");
    MI355_REQUIRE(K % type_block_elems(type) == 0, "mul_mat_id: K=%lld is not a multiple of the block size", (long long)K);
    MI355_REQUIRE(n_used * T <= 65535, "mul_mat_id: too many expert slots for one launch");
    const row_layout L = make_row_layout(type, K);
    hipStream_t s = (hipStream_t)stream;
    const int8_t *aq = (const int8_t *)act;
    const act_ds *ads = (const act_ds *)(aq + nb1 * T * K);
    if (!layout_aligned(as, L)) {
        const dim3 ugrid((unsigned)N, (unsigned)(n_used * T));
#define MI355_ID_UNALIGNED_LAUNCH(TY) MI355_LAUNCH(k_gemv_id_unaligned<TY>, ugrid, dim3(64), 0, s, (const uint8_t *)as, aq, ads, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, L);
        MI355_WEIGHT_TYPE_SWITCH(type, MI355_ID_UNALIGNED_LAUNCH)
#undef MI355_ID_UNALIGNED_LAUNCH
        return launch_status("k_gemv_id_unaligned");
    }
    const int rpw = pick_rpw(N * n_used) > 2 ? 2 : pick_rpw(N * n_used);
    const dim3 grid((unsigned)((N + 4 * rpw - 1) / (4 * rpw)), (unsigned)(n_used * T));
    // an activation row of the split layout is 16-byte aligned inside the workspace when K % 64 == 0 (levels and scales)
    const size_t lds = K % 64 == 0 ? act_lds_bytes(1, K, (int64_t)grid.x * grid.y) : 0;
#define MI355_ID_LAUNCH(TY)                                                                                           \
    if (lds && rpw == 1) MI355_LAUNCH((k_gemv_id<TY, 1, true>), grid, dim3(256), lds, s, (const uint8_t *)as, aq, ads, ids, ids_stride, dst, N, (int)K, n_expert, n_used, nb1); \
    else if (lds) MI355_LAUNCH((k_gemv_id<TY, 2, true>), grid, dim3(256), lds, s, (const uint8_t *)as, aq, ads, ids, ids_stride, dst, N, (int)K, n_expert, n_used, nb1); \
    else if (rpw == 1) MI355_LAUNCH((k_gemv_id<TY, 1, false>), grid, dim3(256), 0, s, (const uint8_t *)as, aq, ads, ids, ids_stride, dst, N, (int)K, n_expert, n_used, nb1); \
    else MI355_LAUNCH((k_gemv_id<TY, 2, false>), grid, dim3(256), 0, s, (const uint8_t *)as, aq, ads, ids, ids_stride, dst, N, (int)K, n_expert, n_used, nb1);
    MI355_WEIGHT_TYPE_SWITCH(type, MI355_ID_LAUNCH)
#undef MI355_ID_LAUNCH
    return launch_status("k_gemv_id");
}

int mi355_moe_gate_up_swiglu_supported(int type, const void *as_gate, const void *as_up, int64_t N, int64_t K) {
    if (!is_weight_type(type) || N <= 0 || N % 32 != 0 || N / 32 >= 0x7fffffff || K <= 0 || K > 32768 || K % 64 != 0 || K % type_block_elems(type) != 0) return 0;
    const row_layout L = make_row_layout(type, K);
    return layout_aligned(as_gate, L) && layout_aligned(as_up, L) ? 1 : 0;
}

int mi355_moe_gate_up_swiglu(void *stream, int type, const void *as_gate, const void *as_up, const void *act, const int32_t *ids, int64_t ids_stride,
                             float *gate, float *up, void *act_out, int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T) {
    MI355_REQUIRE(is_weight_type(type), "moe_gate_up_swiglu: unsupported weight type %d", type);
    MI355_REQUIRE(N > 0 && N % 32 == 0 && N / 32 < 0x7fffffff && K > 0 && K <= 32768 && n_expert > 0 && n_used > 0 && nb1 > 0 && T > 0,
                  "moe_gate_up_swiglu: bad shape (N must be a multiple of 32, K at most 32768)");
    MI355_REQUIRE(K % type_block_elems(type) == 0 && K % 64 == 0, "moe_gate_up_swiglu: K=%lld must be a multiple of the block size and of 64", (long long)K);
    MI355_REQUIRE(n_used * T <= 65535, "moe_gate_up_swiglu: too many expert slots for one launch");
    MI355_REQUIRE(ids != nullptr && gate != nullptr && up != nullptr && ((uintptr_t)act & 15) == 0 && ((uintptr_t)act_out & 15) == 0,
                  "moe_gate_up_swiglu: misaligned or missing operands");
    const row_layout L = make_row_layout(type, K);
    MI355_REQUIRE(layout_aligned(as_gate, L) && layout_aligned(as_up, L), "moe_gate_up_swiglu: expert rows must be 16-byte aligned");
    const int8_t *aq = (const int8_t *)act;
    const act_ds *ads = (const act_ds *)(aq + nb1 * T * K);
    return launch_gate_up_blk_id((hipStream_t)stream, type, as_gate, as_up, aq, ads, ids, ids_stride, K, gate, up, act_out, N, n_expert, n_used, nb1, T);
}

int mi355_block_dots_q8_1(void *stream, int type, const void *W, const void *a, int32_t *out, int64_t N, int64_t K) {
    int rc = check_gemv_args("block_dots", type, W, N, K, N);
    if (rc != MI355_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    const int8_t *aq = (const int8_t *)a;
    const act_ds *ads = (const act_ds *)(aq + K);
    const dim3 grid((unsigned)N);
#define MI355_BLOCK_DOTS_LAUNCH(TY) MI355_LAUNCH(k_block_dots<TY>, grid, dim3(64), 0, s, (const uint8_t *)W, aq, ads, out, N, (int)K);
    MI355_WEIGHT_TYPE_SWITCH(type, MI355_BLOCK_DOTS_LAUNCH)
#undef MI355_BLOCK_DOTS_LAUNCH
    return launch_status("k_block_dots");
}

}  // extern "C"
