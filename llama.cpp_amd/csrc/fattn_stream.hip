// FLASH_ATTN_EXT for one query token over a long KV cache (head size 128, up to four query heads per kv head): the streaming
// form, for f16 caches (k_fattn_dec_stream, described here) and for Q8_0 / Q4_0 caches in the device row layout
// (k_fattn_dec_stream_q, further down).
//
// The kernel is bound by how many bytes of K and V a compute unit keeps in flight, not by arithmetic: a token reads every cell
// once and does 4 flops per byte.  So a wave owns a contiguous range of 64-cell tiles of one kv head and moves them with
// global-to-LDS transfers (no registers in between) into its own two-stage ring: while tile t is worked on, tile t + 1 (32 KiB:
// 64 K rows, 64 V rows) is on its way and tile t + 2 is requested as soon as t's last LDS read has returned.  Two waves share a
// compute unit (2 x 2 x 32 KiB of LDS), 512 waves the chip; no barrier anywhere, every wave writes its own partial result
// (running maximum, sum, un-normalised output) and k_fattn_combine merges them.
//
// Per tile a lane stands for one cell.  Scores: v_mfma_f32_4x4x4f16 works on sixteen independent 4 x 4 blocks, block b = lanes
// 4b .. 4b + 3; lane l supplies row l % 4 of A and column l % 4 of B and receives column l % 4 of D with the rows in its four
// registers.  With A = q (row = query head, the same in every block) and B = K^T (column = cell 4b + l % 4 = l) the four scores
// of cell l land in lane l's registers after 32 steps over the head dimension: no padding columns, no cross-lane sums.  The
// soft-max update is then ordinary per-lane arithmetic on 64 cells at once with one wave-wide maximum per head.  Output:
// the same instruction with A = P (row = head, k = four consecutive cells, read back from a 512-byte transposed copy in LDS)
// and B = V (k = cell, column = element l or 64 + l), whose operand - four cells at one element - is a transposing LDS read
// (ds_read_b64_tr_b16) of the row-major V tile.
//
// LDS layout of a stage: K rows at row * 256 with 16-byte chunk c of row r stored at chunk position c ^ (r & 15), so that the
// 64 lanes reading chunk c of their own rows hit all banks; V rows row-major.  Both are written by transfers that cover four
// whole rows each (fully coalesced in HBM); the permutation happens in the choice of the global address per lane.
#include "common.hpp"
#include "fattn.hpp"

#include <float.h>

namespace mi355 {

constexpr int FS_TILE = 64;                    // cells per tile
constexpr int FS_D = 128;                      // head size
constexpr int FS_ROW = FS_D * 2;               // bytes of a K or V row
constexpr int FS_KT = FS_TILE * FS_ROW;        // bytes of a K (or V) tile
constexpr int FS_STAGE = 2 * FS_KT;
constexpr int FS_WAVES = 2;                    // per group (= per compute unit)
constexpr int FS_MAX_TILES = 64;               // tiles per wave: its mask values are fetched into LDS up front
constexpr int FS_TOTAL_WAVES = 512;

#define FS_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (7 << 4) | (0xF << 8))

// Running soft-max state of a wave: per lane the sums of its own cells' weights; the maxima and the outputs are wave-wide.
struct fs_state {
    float m[4], lsum[4];
    f32x4 o0, o1;   // elements lane and 64 + lane of heads 0..3
};
__device__ __forceinline__ void fs_init(fs_state &S) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
        S.m[r] = -FLT_MAX / 2;
        S.lsum[r] = 0.0f;
    }
    S.o0 = f32x4{0.f, 0.f, 0.f, 0.f};
    S.o1 = f32x4{0.f, 0.f, 0.f, 0.f};
}
// q of head head0 + lane % 4 (zeros past the R heads of the group) as f16 pairs, rounded as the reference rounds q to the K type
// (ggml-cpu.c:11037-11040)
__device__ __forceinline__ void fs_load_q(const fattn_args &a, int64_t head0, int R, int lane, u32 (&qv)[FS_D / 2]) {
    const int hr = lane & 3;
    const float *qp = (const float *)(a.q + (head0 + (hr < R ? hr : 0)) * a.q_nb2);
#pragma unroll
    for (int i = 0; i < FS_D / 4; i++) {
        f32x4 x = *(const f32x4 *)(qp + 4 * i);
        if (hr >= R) x = f32x4{0.f, 0.f, 0.f, 0.f};
        const f16x2 p0 = {(_Float16)x[0], (_Float16)x[1]}, p1 = {(_Float16)x[2], (_Float16)x[3]};
        qv[2 * i] = __builtin_bit_cast(u32, p0);
        qv[2 * i + 1] = __builtin_bit_cast(u32, p1);
    }
}
// ALiBi slopes of the four heads (ggml-cpu.c:10998-11003), wave-uniform
__device__ __forceinline__ void fs_slopes(const fattn_args &a, int64_t head0, float (&slope)[4]) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
        slope[r] = 1.0f;
        if (a.max_bias > 0.0f) {
            const unsigned h = (unsigned)(head0 + r);
            slope[r] = h < a.n_head_log2 ? powf(a.m0, (float)(h + 1)) : powf(a.m1, (float)(2 * (h - a.n_head_log2) + 1));
        }
    }
}
// The soft-max update of the state with one tile's raw scores (q . k of this lane's cell and the four heads), and P^T (head, cell)
// as f16 into the wave's 512 bytes of LDS at p_wr (= base + 2 * lane), where fs_output reads it back as the A operand.  LDS serves a
// wave's operations in order: those reads see these writes, and the next tile's writes come after them.
__device__ __forceinline__ void fs_softmax(const float (&raw)[4], float mv, float scale, float softcap, const float (&slope)[4], unsigned p_wr, fs_state &S) {
    constexpr float NEG = -FLT_MAX / 2;
    const bool valid = mv != -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        float sc = raw[r] * scale;
        if (softcap != 0.0f) sc = softcap * tanhf(sc);
        sc += slope[r] * mv;
        sc = valid ? sc : NEG;
        const float mn = fmaxf(S.m[r], wave_max_dpp(sc));
        const float f = __expf(S.m[r] - mn);
        S.m[r] = mn;
        const float p = valid ? __expf(sc - mn) : 0.0f;
        S.lsum[r] = S.lsum[r] * f + p;
        S.o0[r] *= f;
        S.o1[r] *= f;
        const u32 ph = float_to_half_bits(p);
        asm volatile("ds_write_b16 %0, %1 offset:%2" ::"v"(p_wr), "v"(ph), "n"(r * FS_TILE * 2) : "memory");
    }
}
// Scores of one tile (kc: the 16 chunks of this lane's K row), then fs_softmax.
__device__ __forceinline__ void fs_scores(const u32 (&qv)[FS_D / 2], const u32x4 (&kc)[16], float mv, float scale, float softcap, const float (&slope)[4],
                                          unsigned p_wr, fs_state &S) {
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 16; c++) {
        const u32 a0 = qv[4 * c], a1 = qv[4 * c + 1], a2 = qv[4 * c + 2], a3 = qv[4 * c + 3];
        const u32 b0 = kc[c][0], b1 = kc[c][1], b2 = kc[c][2], b3 = kc[c][3];
        const u32x2 qa = {a0, a1}, qb = {a2, a3}, ka = {b0, b1}, kb2 = {b2, b3};
        s0 = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, qa), __builtin_bit_cast(f16x4, ka), s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, qb), __builtin_bit_cast(f16x4, kb2), s1, 0, 0, 0);
    }
    float raw[4];
#pragma unroll
    for (int r = 0; r < 4; r++) raw[r] = s0[r] + s1[r];
    fs_softmax(raw, mv, scale, softcap, slope, p_wr, S);
}
// This lane's offset inside a row-major V tile for the transposing reads of fs_output: lane l' = lane % 16 of its 16-lane group
// g points at row c0 + l' / 4, elements 16 g + 4 (l' % 4) .. + 3
__device__ __forceinline__ unsigned fs_v_lane(int lane) {
    return (unsigned)((lane & 15) >> 2) * FS_ROW + (unsigned)((lane >> 4) * 16 + (lane & 3) * 4) * 2;
}
// Output of one tile: four cells per step, elements lane and 64 + lane; every operand of the tile is requested before the first
// is used.  v_addr: LDS byte address of the V tile + fs_v_lane; p_rd: the wave's P^T + 128 * (lane % 4).
template <int NJ = 16>   // steps of four cells: 16 = a whole tile, 8 = half of one
__device__ __forceinline__ void fs_output(unsigned v_addr, unsigned p_rd, fs_state &S) {
    u32x2 vlo[NJ], vhi[NJ], pa[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const unsigned addr = v_addr + (unsigned)(j * 4 * FS_ROW);
        asm volatile("ds_read_b64 %0, %1" : "=v"(pa[j]) : "v"(p_rd + (unsigned)(j * 8)));
        asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(vlo[j]) : "v"(addr));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:128" : "=v"(vhi[j]) : "v"(addr));
    }
#pragma unroll
    for (int jb = 0; jb < NJ; jb += 8)   // the wait names its registers so that nothing is used ahead of it; 24 operands per statement
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(vlo[jb]), "+v"(vlo[jb + 1]), "+v"(vlo[jb + 2]), "+v"(vlo[jb + 3]), "+v"(vlo[jb + 4]), "+v"(vlo[jb + 5]), "+v"(vlo[jb + 6]), "+v"(vlo[jb + 7]),
                       "+v"(vhi[jb]), "+v"(vhi[jb + 1]), "+v"(vhi[jb + 2]), "+v"(vhi[jb + 3]), "+v"(vhi[jb + 4]), "+v"(vhi[jb + 5]), "+v"(vhi[jb + 6]), "+v"(vhi[jb + 7]),
                       "+v"(pa[jb]), "+v"(pa[jb + 1]), "+v"(pa[jb + 2]), "+v"(pa[jb + 3]), "+v"(pa[jb + 4]), "+v"(pa[jb + 5]), "+v"(pa[jb + 6]), "+v"(pa[jb + 7]));
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        S.o0 = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, pa[j]), __builtin_bit_cast(f16x4, vlo[j]), S.o0, 0, 0, 0);
        S.o1 = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, pa[j]), __builtin_bit_cast(f16x4, vhi[j]), S.o1, 0, 0, 0);
    }
}

__global__ void __launch_bounds__(FS_WAVES * 64, 1) k_fattn_dec_stream(fattn_args a, int tiles_per_wave, int n_tiles, int R) {
    __shared__ __attribute__((aligned(1024))) uint8_t ring_buf[FS_WAVES * 2 * FS_STAGE];
    __shared__ __attribute__((aligned(16))) unsigned short pbuf[FS_WAVES][4][FS_TILE];
    __shared__ __attribute__((aligned(16))) unsigned short mbuf[FS_WAVES][FS_MAX_TILES * FS_TILE];
    // the ring is written by global-to-LDS transfers only
    asm volatile("" ::"v"((void *)ring_buf) : "memory");
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int split = (int)blockIdx.x * FS_WAVES + wave;
    const int64_t hk = blockIdx.y;
    const int t_begin = split * tiles_per_wave;
    const int t_end = t_begin + tiles_per_wave < n_tiles ? t_begin + tiles_per_wave : n_tiles;
    const int n = t_end > t_begin ? t_end - t_begin : 0;
    const int64_t c_begin = (int64_t)t_begin * FS_TILE;

    float slope[4];
    fs_slopes(a, hk * R, slope);
    uint8_t *ring = ring_buf + wave * (2 * FS_STAGE);
    // transfers of tile t into stage st: instruction i moves rows 4i .. 4i + 3; lane p -> row 4i + p / 16, chunk position p % 16.
    // A whole tile in range: scalar row addresses plus per-lane offsets that are the same for every tile; the last, partial tile
    // of the cache clamps its rows per lane (rows past the end repeat the last cell; their scores are discarded).
    const int rsub = lane >> 4, pos = lane & 15;
    unsigned koff[4], voff;
#pragma unroll
    for (int vv = 0; vv < 4; vv++) koff[vv] = (unsigned)rsub * (unsigned)a.k_nb1 + (unsigned)((pos ^ ((4 * vv + rsub) & 15)) << 4);
    voff = (unsigned)rsub * (unsigned)a.v_nb1 + (unsigned)(pos << 4);
    const uint8_t *k_head = a.k + hk * a.k_nb2, *v_head = a.v + hk * a.v_nb2;
    auto dma = [&](const uint8_t *g, unsigned off, uint8_t *l) {   // g, l: wave-uniform
        asm volatile("" : "+v"(off));   // keeps the sum from being formed per lane ahead of the loop (two registers per source)
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)(g + off), (void __attribute__((address_space(3))) *)l, 16, 0, 0);
    };
    // which = 0: the K half of the stage, 1: the V half (sixteen transfers each)
    auto issue = [&](int t, int st, int which) {
        const int64_t c0 = c_begin + (int64_t)t * FS_TILE;
        uint8_t *hb = ring + st * FS_STAGE + which * FS_KT;
        const uint8_t *head = which ? v_head : k_head;
        const int64_t nb1 = which ? (int64_t)a.v_nb1 : (int64_t)a.k_nb1;
        if (c0 + FS_TILE <= a.Nkv) {
            const uint8_t *g = head + c0 * nb1;
#pragma unroll
            for (int i = 0; i < 16; i++) dma(g + (int64_t)(4 * i) * nb1, which ? voff : koff[i & 3], hb + i * 1024);
        } else {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int row = 4 * i + rsub;
                int64_t cell = c0 + row;
                if (cell >= a.Nkv) cell = a.Nkv - 1;
                const uint8_t *g = head + cell * nb1 + ((which ? pos : (pos ^ (row & 15))) << 4);
                __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)g, (void __attribute__((address_space(3))) *)(hb + i * 1024), 16, 0, 0);
            }
        }
    };

    fs_state S;
    fs_init(S);
    const float scale = a.softcap != 0.0f ? a.scale / a.softcap : a.scale;

    // order of the transfers: K0 V0 K1 V1, then K(t + 2) once the scores of tile t are taken and V(t + 2) once its output is
    if (n > 0) {
        issue(0, 0, 0);
        issue(0, 0, 1);
    }
    if (n > 1) {
        issue(1, 1, 0);
        issue(1, 1, 1);
    }
    // While the first two tiles travel: q and this wave's mask values (all requested before the first is used).
    const int hr = lane & 3;
    u32 qv[FS_D / 2];
    fs_load_q(a, hk * R, R, lane, qv);
    // ---- mask values of the wave's cells into LDS, eight cells per lane and step (cells past the end count as masked)
    unsigned short *mw = mbuf[wave];
    {
        const unsigned short *mrow = (const unsigned short *)a.mask;
        const bool wide = ((uintptr_t)mrow & 15) == 0;
        u32x4 mc[FS_MAX_TILES / 8];
#pragma unroll
        for (int it = 0; it < FS_MAX_TILES / 8; it++) {
            const int j = it * 64 + lane;
            const int64_t c = c_begin + (int64_t)j * 8;
            mc[it] = u32x4{0xFC00FC00u, 0xFC00FC00u, 0xFC00FC00u, 0xFC00FC00u};   // -inf
            if (j * 8 < n * FS_TILE) {
                if (mrow && wide && c + 8 <= a.Nkv) {
                    mc[it] = load16(mrow + c);
                } else {
                    unsigned short e[8];
#pragma unroll
                    for (int i = 0; i < 8; i++) e[i] = c + i < a.Nkv ? (mrow ? mrow[c + i] : (unsigned short)0) : (unsigned short)0xFC00;
#pragma unroll
                    for (int i = 0; i < 4; i++) mc[it][i] = (u32)e[2 * i] | ((u32)e[2 * i + 1] << 16);
                }
            }
        }
#pragma unroll
        for (int it = 0; it < FS_MAX_TILES / 8; it++) {
            const int j = it * 64 + lane;
            if (j * 8 < n * FS_TILE) *(u32x4 *)(mw + j * 8) = mc[it];
        }
    }
    // From here on LDS is read and written through inline assembly with waits placed by hand: for an access it can see, the
    // compiler waits for every global-to-LDS transfer in flight, which would serialise the ring.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    // LDS byte addresses of this lane's operands inside a stage
    const unsigned ring_lds = (unsigned)(uintptr_t)(void __attribute__((address_space(3))) *)ring;
    const unsigned k_lane = (unsigned)lane * FS_ROW + ((unsigned)(lane & 15) << 4);                      // chunk c at k_lane ^ (c << 4)
    const unsigned v_lane = FS_KT + fs_v_lane(lane);
    const unsigned m_lane = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned short *)mw + (unsigned)lane * 2;
    const unsigned p_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned short *)&pbuf[wave][0][0];
    const unsigned p_wr = p_base + (unsigned)lane * 2, p_rd = p_base + (unsigned)hr * (FS_TILE * 2);

    for (int t = 0; t < n; t++) {
        const int st = t & 1;
        // K(t) has landed when at most V(t), K(t + 1), V(t + 1) are still on their way (transfers complete in the order issued)
        if (t + 1 < n) FS_WAIT_VM(48);
        else FS_WAIT_VM(16);
        const unsigned sb = ring_lds + (unsigned)st * FS_STAGE;

        // ---- scores: 16 chunks of this lane's K row, 32 MFMA steps
        u32x4 kc[16];
        u32 mbits;
        asm volatile("ds_read_u16 %0, %1" : "=v"(mbits) : "v"(m_lane + (unsigned)t * (FS_TILE * 2)));
#pragma unroll
        for (int c = 0; c < 16; c++) asm volatile("ds_read_b128 %0, %1" : "=v"(kc[c]) : "v"(sb + (k_lane ^ (unsigned)(c << 4))));
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(mbits), "+v"(kc[0]), "+v"(kc[1]), "+v"(kc[2]), "+v"(kc[3]), "+v"(kc[4]), "+v"(kc[5]), "+v"(kc[6]), "+v"(kc[7]), "+v"(kc[8]), "+v"(kc[9]),
                       "+v"(kc[10]), "+v"(kc[11]), "+v"(kc[12]), "+v"(kc[13]), "+v"(kc[14]), "+v"(kc[15]));
        if (t + 2 < n) issue(t + 2, st, 0);   // the K rows are in registers: their half of the stage is free
        fs_scores(qv, kc, half_bits_to_float((unsigned short)mbits), scale, a.softcap, slope, p_wr, S);
        // V(t) has landed when at most K(t + 1), V(t + 1), K(t + 2) are outstanding
        if (t + 2 < n) FS_WAIT_VM(48);
        else if (t + 1 < n) FS_WAIT_VM(32);
        else FS_WAIT_VM(0);
        fs_output(sb + v_lane, p_rd, S);
        // every LDS read of this stage has returned (the last wait above): the V half may be overwritten
        if (t + 2 < n) issue(t + 2, st, 1);
    }

    // ---- partial result of this split: un-normalised outputs, running maximum, sum
#pragma unroll
    for (int r = 0; r < 4; r++) {
        if (r < R) {
            const float L = wave_sum_dpp(S.lsum[r]);
            float *p = a.ws + (((int64_t)hk * R + r) * a.n_splits + split) * (FS_D + 2);
            p[lane] = S.o0[r];
            p[64 + lane] = S.o1[r];
            if (lane == 0) {
                p[FS_D] = S.m[r];
                p[FS_D + 1] = L;
            }
        }
    }
}

// ---- the same over a Q8_0 / Q4_0 cache in the device row layout --------------------------------------------------------------
// A cell's row in such a cache holds the levels of all its kv heads first and their f16 scales behind them, so the levels of one
// (cell, head) are 128 / 64 contiguous, 16-byte aligned bytes and its four scales 8 bytes: both move by global-to-LDS transfers like
// the f16 rows above (levels 16 bytes per lane, scales 4), half the bytes or less per cell.
// Scores follow the reference's arithmetic for a quantized K (ggml-cpu.c:11037-11046: q is quantized to Q8_0, kq_vec_dot is the
// integer block dot ggml_vec_dot_q8_0_q8_0 / ggml_vec_dot_q4_0_q8_0, ggml-cpu-quants.c): v_mfma_i32_4x4x4_16b_i8 with A = q levels
// (row = head) and B = this lane's cell, one accumulator per 32-element block, then sum_b d_k d_q sumi in f32.
// V (ggml-cpu.c:11078-11090 dequantizes the row and accumulates in f32): the wave turns the tile's levels into d * level as f16 -
// bytes into the low byte of halves whose high byte is 0x64 (1024 + u), minus 1152 or 1032, times the block's scale, all packed
// f16 operations on exact values until the one rounding of the product - and writes them row-major into its own 16 KiB of LDS,
// where fs_output finds what it finds for an f16 cache.
struct fsq_src {
    const uint8_t *lv, *sc;   // levels / scales of (cell 0, kv head 0)
    int64_t head_lv, head_sc; // bytes from one kv head to the next
    int64_t cell_lv, cell_sc; // bytes from one cell to the next
};
template <int T>
struct fsq_geo {
    static constexpr int ROW = T == MI355_Q8_0 ? 128 : 64;   // bytes of levels per (cell, head)
    static constexpr int CH = ROW / 16;                       // 16-byte chunks per row
    static constexpr int RPT = 64 / CH;                       // rows per transfer
    static constexpr int NT = FS_TILE / RPT;                  // level transfers per tile
    static constexpr int CNT = NT + 2;                        // with the two scale transfers
};
constexpr int FSQ_SCALES = FS_TILE * 8;   // bytes of scales per tile and operand

template <int R4>
__device__ __forceinline__ int quad_bcast_i(int v) { return __builtin_amdgcn_update_dpp(0, v, R4 * 0x55, 0xF, 0xF, true); }

// q of head head0 + lane % 4 as Q8_0 (quantize_row_q8_0_ref, ggml-quants.c:194-218): 32 words of levels, the f16-rounded scales of
// the four blocks and the sums of their levels; zeros past the R heads of the group
__device__ __forceinline__ void fsq_load_q(const fattn_args &a, int64_t head0, int R, int lane, u32 (&qw)[32], float (&dq)[4], int (&qs)[4]) {
    const int hr = lane & 3;
    const float *qp = (const float *)(a.q + (head0 + (hr < R ? hr : 0)) * a.q_nb2);
#pragma unroll
    for (int b = 0; b < 4; b++) {
        f32x4 x[8];
        float amax = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            x[i] = *(const f32x4 *)(qp + 32 * b + 4 * i);
            if (hr >= R) x[i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 4; j++) amax = fmaxf(amax, fabsf(x[i][j]));
        }
        const float d = amax / 127.0f;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        int sum = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            u32 w = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int q = (int)roundf(x[i][j] * id);
                sum += q;
                w |= (u32)(q & 0xFF) << (8 * j);
            }
            qw[8 * b + i] = w;
        }
        dq[b] = half_bits_to_float(float_to_half_bits(d));
        qs[b] = sum;
    }
}

// raw scores of this lane's cell against the four heads: kc = the chunks of its K row, ksc = its four scales
template <int TK>
__device__ __forceinline__ void fsq_scores(const u32 (&qw)[32], const float (&dqa)[4][4], const int (&qsa)[4][4], const u32x4 (&kc)[fsq_geo<TK>::CH], const u32x2 &ksc,
                                           float (&raw)[4]) {
    i32x4 ab[4];
#pragma unroll
    for (int b = 0; b < 4; b++) ab[b] = i32x4{0, 0, 0, 0};
    if constexpr (TK == MI355_Q8_0) {
#pragma unroll
        for (int c = 0; c < 8; c++)
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const u32 kw = kc[c][w];
                ab[c >> 1] = __builtin_amdgcn_mfma_i32_4x4x4i8((int)qw[4 * c + w], (int)kw, ab[c >> 1], 0, 0, 0);
            }
    } else {
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const u32 kw = kc[c][w];
                ab[c] = __builtin_amdgcn_mfma_i32_4x4x4i8((int)qw[8 * c + w], (int)(kw & 0x0F0F0F0Fu), ab[c], 0, 0, 0);
                ab[c] = __builtin_amdgcn_mfma_i32_4x4x4i8((int)qw[8 * c + 4 + w], (int)((kw >> 4) & 0x0F0F0F0Fu), ab[c], 0, 0, 0);
            }
    }
    float dk[4];
    dk[0] = half_bits_to_float((unsigned short)(ksc[0] & 0xFFFFu));
    dk[1] = half_bits_to_float((unsigned short)(ksc[0] >> 16));
    dk[2] = half_bits_to_float((unsigned short)(ksc[1] & 0xFFFFu));
    dk[3] = half_bits_to_float((unsigned short)(ksc[1] >> 16));
#pragma unroll
    for (int r = 0; r < 4; r++) {
        float sum = 0.0f;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const int sumi = TK == MI355_Q8_0 ? ab[b][r] : ab[b][r] - 8 * qsa[r][b];
            sum += (float)sumi * (dk[b] * dqa[r][b]);
        }
        raw[r] = sum;
    }
}

// four bytes u -> the f16 pairs (u0 + bias, u1 + bias) * d and (u2 + bias, u3 + bias) * d; 1024 + u is exact in a half whose high
// byte is 0x64, and so is the sum with bias = -(1024 + offset of the level)
__device__ __forceinline__ u32x2 fsq_bytes_to_f16(u32 u, f16x2 bias, f16x2 d2) {
    const u32 a = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u), b = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);
    const f16x2 x = (__builtin_bit_cast(f16x2, a) + bias) * d2, y = (__builtin_bit_cast(f16x2, b) + bias) * d2;
    return u32x2{__builtin_bit_cast(u32, x), __builtin_bit_cast(u32, y)};
}

// V levels of 32 cells of a stage (LDS byte addresses of the first cell's levels / scales) -> d * level as f16, row-major
// [32][128], at LDS byte address v_f16
template <int TV>
__device__ __forceinline__ void fsq_convert_v(unsigned v_lv, unsigned v_sc, unsigned v_f16, int lane) {
    typedef fsq_geo<TV> G;
    constexpr int NJ = 32 * G::CH / 64;   // chunks per lane: 4 (Q8_0, 16 elements each) or 2 (Q4_0, 32 elements each)
    u32x4 lv[NJ];
    u32 sc[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int chunk = j * 64 + lane, row = chunk / G::CH, c = chunk % G::CH;
        const int blk = TV == MI355_Q8_0 ? c >> 1 : c;
        asm volatile("ds_read_b128 %0, %1" : "=v"(lv[j]) : "v"(v_lv + (unsigned)chunk * 16u));
        asm volatile("ds_read_u16 %0, %1" : "=v"(sc[j]) : "v"(v_sc + (unsigned)(row * 8 + blk * 2)));
    }
    if constexpr (NJ == 4)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lv[0]), "+v"(lv[1]), "+v"(lv[2]), "+v"(lv[3]), "+v"(sc[0]), "+v"(sc[1]), "+v"(sc[2]), "+v"(sc[3]));
    else
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lv[0]), "+v"(lv[1]), "+v"(sc[0]), "+v"(sc[1]));
    const f16x2 bias = TV == MI355_Q8_0 ? f16x2{(_Float16)-1152.0f, (_Float16)-1152.0f} : f16x2{(_Float16)-1032.0f, (_Float16)-1032.0f};
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int chunk = j * 64 + lane, row = chunk / G::CH, c = chunk % G::CH;
        const u32 dd = sc[j] | (sc[j] << 16);
        const f16x2 d2 = __builtin_bit_cast(f16x2, dd);
        if constexpr (TV == MI355_Q8_0) {
            // elements 16 c .. 16 c + 7, .. + 15 of the row
            const u32 w0 = lv[j][0], w1 = lv[j][1], w2 = lv[j][2], w3 = lv[j][3];
            const u32x2 e0 = fsq_bytes_to_f16(w0 ^ 0x80808080u, bias, d2), e1 = fsq_bytes_to_f16(w1 ^ 0x80808080u, bias, d2);
            const u32x2 e2 = fsq_bytes_to_f16(w2 ^ 0x80808080u, bias, d2), e3 = fsq_bytes_to_f16(w3 ^ 0x80808080u, bias, d2);
            const u32x4 o0 = {e0[0], e0[1], e1[0], e1[1]}, o1 = {e2[0], e2[1], e3[0], e3[1]};
            const unsigned dst = v_f16 + (unsigned)(row * FS_ROW + c * 32);
            asm volatile("ds_write_b128 %0, %1" ::"v"(dst), "v"(o0) : "memory");
            asm volatile("ds_write_b128 %0, %1 offset:16" ::"v"(dst), "v"(o1) : "memory");
        } else {
            u32x4 o[4];   // elements 32 c + 0..7, 8..15 (low nibbles), 16..23, 24..31 (high nibbles)
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const u32 wa = lv[j][2 * h], wb = lv[j][2 * h + 1];
                const u32x2 la = fsq_bytes_to_f16(wa & 0x0F0F0F0Fu, bias, d2), lb = fsq_bytes_to_f16(wb & 0x0F0F0F0Fu, bias, d2);
                const u32x2 ha = fsq_bytes_to_f16((wa >> 4) & 0x0F0F0F0Fu, bias, d2), hb = fsq_bytes_to_f16((wb >> 4) & 0x0F0F0F0Fu, bias, d2);
                o[h] = u32x4{la[0], la[1], lb[0], lb[1]};
                o[2 + h] = u32x4{ha[0], ha[1], hb[0], hb[1]};
            }
            const unsigned dst = v_f16 + (unsigned)(row * FS_ROW + c * 64);
            asm volatile("ds_write_b128 %0, %1" ::"v"(dst), "v"(o[0]) : "memory");
            asm volatile("ds_write_b128 %0, %1 offset:16" ::"v"(dst), "v"(o[1]) : "memory");
            asm volatile("ds_write_b128 %0, %1 offset:32" ::"v"(dst), "v"(o[2]) : "memory");
            asm volatile("ds_write_b128 %0, %1 offset:48" ::"v"(dst), "v"(o[3]) : "memory");
        }
    }
}

// Waves per group (= per compute unit): as many as LDS holds - each wave keeps two stages, half a tile of f16 V, its P^T and the mask
// values of up to FSQ_MAX_TILES tiles.  A wave on its own is one dependent chain (reads, scores, soft-max, conversion, output);
// more of them per compute unit is what keeps its vector ALUs and its transfers busy.
constexpr int FSQ_MAX_TILES = 32;
constexpr int FSQ_VF = 32 * FS_ROW;   // bytes of half a V tile as f16
template <int TK, int TV>
constexpr int fsq_waves() { return TK == MI355_Q8_0 && TV == MI355_Q8_0 ? 3 : (TK == MI355_Q4_0 && TV == MI355_Q4_0 ? 5 : 4); }
static int fsq_waves_rt(int tk, int tv) { return tk == MI355_Q8_0 && tv == MI355_Q8_0 ? 3 : (tk == MI355_Q4_0 && tv == MI355_Q4_0 ? 5 : 4); }
constexpr int FSQ_TOTAL_GROUPS = 256;

template <int TK, int TV>
__global__ void __launch_bounds__((fsq_waves<TK, TV>() * 64), 1) k_fattn_dec_stream_q(fattn_args a, fsq_src ksrc, fsq_src vsrc, int tiles_per_wave, int n_tiles, int R) {
    typedef fsq_geo<TK> GK;
    typedef fsq_geo<TV> GV;
    constexpr int NWV = fsq_waves<TK, TV>();
    constexpr int K_LV = FS_TILE * GK::ROW, V_LV = FS_TILE * GV::ROW;
    constexpr int OFF_V = K_LV, OFF_KS = K_LV + V_LV, OFF_VS = OFF_KS + FSQ_SCALES;
    constexpr int STAGE = OFF_VS + FSQ_SCALES;
    constexpr int CK = GK::CNT, CV = GV::CNT;   // transfers of the K / V part of a tile
    __shared__ __attribute__((aligned(1024))) uint8_t ring_buf[NWV * 2 * STAGE];
    __shared__ __attribute__((aligned(1024))) uint8_t vf_buf[NWV * FSQ_VF];   // half of the wave's V tile as f16
    __shared__ __attribute__((aligned(16))) unsigned short pbuf[NWV][4][FS_TILE];
    __shared__ __attribute__((aligned(16))) unsigned short mbuf[NWV][FSQ_MAX_TILES * FS_TILE];
    asm volatile("" ::"v"((void *)ring_buf), "v"((void *)vf_buf) : "memory");
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int split = (int)blockIdx.x * (int)(blockDim.x >> 6) + wave;   // the launch may give a group fewer than NWV waves
    const int64_t hk = blockIdx.y;
    const int t_begin = split * tiles_per_wave;
    const int t_end = t_begin + tiles_per_wave < n_tiles ? t_begin + tiles_per_wave : n_tiles;
    const int n = t_end > t_begin ? t_end - t_begin : 0;
    const int64_t c_begin = (int64_t)t_begin * FS_TILE;

    float slope[4];
    fs_slopes(a, hk * R, slope);
    uint8_t *ring = ring_buf + wave * (2 * STAGE);
    const uint8_t *k_lv = ksrc.lv + hk * ksrc.head_lv, *k_sc = ksrc.sc + hk * ksrc.head_sc;
    const uint8_t *v_lv = vsrc.lv + hk * vsrc.head_lv, *v_sc = vsrc.sc + hk * vsrc.head_sc;
    // per-lane offsets of the transfers.  K levels: transfer i moves rows RPT i .. + RPT - 1, lane p -> row RPT i + p / CH, LDS position
    // p % CH, which holds chunk position ^ swz(row) (swz: (row >> 1) & 7 for 128-byte rows, (row >> 2) & 3 for 64-byte rows), so that
    // the 64 lanes reading chunk c of their own rows hit all banks.  V levels: rows as they are.  Scales: two transfers of 32 rows.
    unsigned koff[2], voff, ksoff, vsoff;
    {
        const unsigned p = (unsigned)lane;
        if constexpr (TK == MI355_Q8_0) {
#pragma unroll
            for (int e = 0; e < 2; e++) koff[e] = (p >> 3) * (unsigned)ksrc.cell_lv + (((p & 7) ^ ((4 * e + (p >> 4)) & 7)) << 4);
        } else {
            koff[0] = koff[1] = (p >> 2) * (unsigned)ksrc.cell_lv + (((p & 3) ^ ((p >> 4) & 3)) << 4);
        }
        voff = TV == MI355_Q8_0 ? (p >> 3) * (unsigned)vsrc.cell_lv + ((p & 7) << 4) : (p >> 2) * (unsigned)vsrc.cell_lv + ((p & 3) << 4);
        ksoff = (p >> 1) * (unsigned)ksrc.cell_sc + ((p & 1) << 2);
        vsoff = (p >> 1) * (unsigned)vsrc.cell_sc + ((p & 1) << 2);
    }
    auto dma16 = [&](const uint8_t *g, unsigned off, uint8_t *l) {   // g, l: wave-uniform
        asm volatile("" : "+v"(off));
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)(g + off), (void __attribute__((address_space(3))) *)l, 16, 0, 0);
    };
    auto dma4 = [&](const uint8_t *g, unsigned off, uint8_t *l) {
        asm volatile("" : "+v"(off));
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)(g + off), (void __attribute__((address_space(3))) *)l, 4, 0, 0);
    };
    // which = 0: K levels and scales of tile t into stage st (CK transfers), 1: V (CV transfers)
    auto issue = [&](int t, int st, int which) {
        const int64_t c0 = c_begin + (int64_t)t * FS_TILE;
        uint8_t *sb = ring + st * STAGE;
        const int64_t nb_lv = which ? vsrc.cell_lv : ksrc.cell_lv, nb_sc = which ? vsrc.cell_sc : ksrc.cell_sc;
        const uint8_t *lvp = which ? v_lv : k_lv, *scp = which ? v_sc : k_sc;
        uint8_t *l_lv = sb + (which ? OFF_V : 0), *l_sc = sb + (which ? OFF_VS : OFF_KS);
        const int NT = which ? GV::NT : GK::NT, RPT = which ? GV::RPT : GK::RPT, CH = which ? GV::CH : GK::CH;
        if (c0 + FS_TILE <= a.Nkv) {
            const uint8_t *g = lvp + c0 * nb_lv;
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (i < NT) dma16(g + (int64_t)(RPT * i) * nb_lv, which ? voff : koff[i & 1], l_lv + i * 1024);
            const uint8_t *gs = scp + c0 * nb_sc;
            dma4(gs, which ? vsoff : ksoff, l_sc);
            dma4(gs + 32 * nb_sc, which ? vsoff : ksoff, l_sc + 256);
        } else {   // the cache's last, partial tile: rows past the end repeat the last cell (their scores are discarded)
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (i < NT) {
                    const int row = RPT * i + lane / CH, pos = lane % CH;
                    int64_t cell = c0 + row;
                    if (cell >= a.Nkv) cell = a.Nkv - 1;
                    const int swz = which ? 0 : (TK == MI355_Q8_0 ? (row >> 1) & 7 : (row >> 2) & 3);
                    const uint8_t *g = lvp + cell * nb_lv + ((pos ^ swz) << 4);
                    __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)g, (void __attribute__((address_space(3))) *)(l_lv + i * 1024), 16, 0, 0);
                }
#pragma unroll
            for (int i = 0; i < 2; i++) {
                int64_t cell = c0 + 32 * i + (lane >> 1);
                if (cell >= a.Nkv) cell = a.Nkv - 1;
                const uint8_t *g = scp + cell * nb_sc + ((lane & 1) << 2);
                __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)g, (void __attribute__((address_space(3))) *)(l_sc + i * 256), 4, 0, 0);
            }
        }
    };

    fs_state S;
    fs_init(S);
    const float scale = a.softcap != 0.0f ? a.scale / a.softcap : a.scale;
    if (n > 0) {
        issue(0, 0, 0);
        issue(0, 0, 1);
    }
    if (n > 1) {
        issue(1, 1, 0);
        issue(1, 1, 1);
    }
    // While the first two tiles travel: q as Q8_0 and this wave's mask values.
    const int hr = lane & 3;
    u32 qw[32];
    float dq[4], dqa[4][4];
    int qs[4], qsa[4][4];
    fsq_load_q(a, hk * R, R, lane, qw, dq, qs);
#pragma unroll
    for (int b = 0; b < 4; b++) {   // every lane needs the scales and sums of all four heads: lane r of its quad holds head r's
        const int di = __builtin_bit_cast(int, dq[b]);
        dqa[0][b] = __builtin_bit_cast(float, quad_bcast_i<0>(di));
        dqa[1][b] = __builtin_bit_cast(float, quad_bcast_i<1>(di));
        dqa[2][b] = __builtin_bit_cast(float, quad_bcast_i<2>(di));
        dqa[3][b] = __builtin_bit_cast(float, quad_bcast_i<3>(di));
        qsa[0][b] = quad_bcast_i<0>(qs[b]);
        qsa[1][b] = quad_bcast_i<1>(qs[b]);
        qsa[2][b] = quad_bcast_i<2>(qs[b]);
        qsa[3][b] = quad_bcast_i<3>(qs[b]);
    }
    unsigned short *mw = mbuf[wave];
    {
        const unsigned short *mrow = (const unsigned short *)a.mask;
        const bool wide = ((uintptr_t)mrow & 15) == 0;
        u32x4 mc[FSQ_MAX_TILES / 8];
#pragma unroll
        for (int it = 0; it < FSQ_MAX_TILES / 8; it++) {
            const int j = it * 64 + lane;
            const int64_t c = c_begin + (int64_t)j * 8;
            mc[it] = u32x4{0xFC00FC00u, 0xFC00FC00u, 0xFC00FC00u, 0xFC00FC00u};   // -inf
            if (j * 8 < n * FS_TILE) {
                if (mrow && wide && c + 8 <= a.Nkv) {
                    mc[it] = load16(mrow + c);
                } else {
                    unsigned short e[8];
#pragma unroll
                    for (int i = 0; i < 8; i++) e[i] = c + i < a.Nkv ? (mrow ? mrow[c + i] : (unsigned short)0) : (unsigned short)0xFC00;
#pragma unroll
                    for (int i = 0; i < 4; i++) mc[it][i] = (u32)e[2 * i] | ((u32)e[2 * i + 1] << 16);
                }
            }
        }
#pragma unroll
        for (int it = 0; it < FSQ_MAX_TILES / 8; it++) {
            const int j = it * 64 + lane;
            if (j * 8 < n * FS_TILE) *(u32x4 *)(mw + j * 8) = mc[it];
        }
    }
    // From here on LDS is read and written through inline assembly with waits placed by hand (see k_fattn_dec_stream).
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    const unsigned ring_lds = (unsigned)(uintptr_t)(void __attribute__((address_space(3))) *)ring;
    const unsigned vf_lds = (unsigned)(uintptr_t)(void __attribute__((address_space(3))) *)(vf_buf + wave * FSQ_VF);
    const unsigned k_lane = TK == MI355_Q8_0 ? (unsigned)lane * 128u + ((((unsigned)lane >> 1) & 7u) << 4) : (unsigned)lane * 64u + ((((unsigned)lane >> 2) & 3u) << 4);
    const unsigned m_lane = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned short *)mw + (unsigned)lane * 2;
    const unsigned p_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned short *)&pbuf[wave][0][0];
    const unsigned p_wr = p_base + (unsigned)lane * 2, p_rd = p_base + (unsigned)hr * (FS_TILE * 2);

    for (int t = 0; t < n; t++) {
        const int st = t & 1;
        // K(t) has landed when at most V(t), K(t + 1), V(t + 1) are still on their way (transfers complete in the order issued)
        if (t + 1 < n) FS_WAIT_VM(CV + CK + CV);
        else FS_WAIT_VM(CV);
        const unsigned sb = ring_lds + (unsigned)st * STAGE;
        u32x4 kc[GK::CH];
        u32x2 ksc;
        u32 mbits;
        asm volatile("ds_read_u16 %0, %1" : "=v"(mbits) : "v"(m_lane + (unsigned)t * (FS_TILE * 2)));
        asm volatile("ds_read_b64 %0, %1" : "=v"(ksc) : "v"(sb + (unsigned)OFF_KS + (unsigned)lane * 8u));
#pragma unroll
        for (int c = 0; c < GK::CH; c++) asm volatile("ds_read_b128 %0, %1" : "=v"(kc[c]) : "v"(sb + (k_lane ^ (unsigned)(c << 4))));
        if constexpr (GK::CH == 8)
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(mbits), "+v"(ksc), "+v"(kc[0]), "+v"(kc[1]), "+v"(kc[2]), "+v"(kc[3]), "+v"(kc[4]), "+v"(kc[5]), "+v"(kc[6]), "+v"(kc[7]));
        else
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(mbits), "+v"(ksc), "+v"(kc[0]), "+v"(kc[1]), "+v"(kc[2]), "+v"(kc[3]));
        if (t + 2 < n) issue(t + 2, st, 0);   // the K rows are in registers: their part of the stage is free
        float raw[4];
        fsq_scores<TK>(qw, dqa, qsa, kc, ksc, raw);
        fs_softmax(raw, half_bits_to_float((unsigned short)mbits), scale, a.softcap, slope, p_wr, S);
        // V(t) has landed when at most K(t + 1), V(t + 1), K(t + 2) are outstanding
        if (t + 2 < n) FS_WAIT_VM(CK + CV + CK);
        else if (t + 1 < n) FS_WAIT_VM(CK + CV);
        else FS_WAIT_VM(0);
        // the tile's V in two halves of 32 cells through the wave's 8 KiB of f16 rows
        fsq_convert_v<TV>(sb + (unsigned)OFF_V, sb + (unsigned)OFF_VS, vf_lds, lane);
        fs_output<8>(vf_lds + fs_v_lane(lane), p_rd, S);
        fsq_convert_v<TV>(sb + (unsigned)(OFF_V + 32 * GV::ROW), sb + (unsigned)(OFF_VS + 32 * 8), vf_lds, lane);
        // the levels are in registers or already converted: the V part of the stage may be overwritten
        if (t + 2 < n) issue(t + 2, st, 1);
        fs_output<8>(vf_lds + fs_v_lane(lane), p_rd + 64, S);
    }

#pragma unroll
    for (int r = 0; r < 4; r++) {
        if (r < R) {
            const float L = wave_sum_dpp(S.lsum[r]);
            float *p = a.ws + (((int64_t)hk * R + r) * a.n_splits + split) * (FS_D + 2);
            p[lane] = S.o0[r];
            p[64 + lane] = S.o1[r];
            if (lane == 0) {
                p[FS_D] = S.m[r];
                p[FS_D + 1] = L;
            }
        }
    }
}

// ---- short caches: at most 512 cells, one launch -------------------------------------------------------------------------------
// One group per kv head, one wave per 64-cell tile (up to eight).  Nothing here is bound by bytes: the time is one trip to memory
// plus the arithmetic of one tile, so a wave requests everything at once - its K and V tiles as coalesced 16-byte loads into
// registers (four whole rows per instruction), q, its mask value - and then passes first K, then V through its own 16 KiB of
// LDS to bring them into operand form: K rows with their chunks XOR-ed across the banks, so that each lane reads back the row of
// its cell; V row-major for the transposing reads.  (A lane loading its own K row directly would touch 64 cache lines per
// instruction: measured 2.8 us per wave of the group.)  The waves' states meet in LDS; the group normalises and writes the output
// (and its Q8_1 form where the next product wants it), so no second launch merges anything.
constexpr int FSS_MAX_WAVES = 8;

__global__ void __launch_bounds__(FSS_MAX_WAVES * 64, 1) k_fattn_dec_short(fattn_args a, int R) {
    __shared__ __attribute__((aligned(1024))) uint8_t tbuf[FSS_MAX_WAVES * FS_KT];
    __shared__ __attribute__((aligned(16))) unsigned short pbuf[FSS_MAX_WAVES][4][FS_TILE];
    __shared__ float s_m[FSS_MAX_WAVES][4], s_l[FSS_MAX_WAVES][4];
    __shared__ float s_o[FSS_MAX_WAVES][4][FS_D];
    __shared__ __attribute__((aligned(16))) unsigned short qbuf[FSS_MAX_WAVES][4][FS_D];

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int n_waves = (int)(blockDim.x >> 6);
    const int64_t hk = blockIdx.x;
    const int64_t c0 = (int64_t)wave * FS_TILE;
    const int rsub = lane >> 4, pos = lane & 15;

    // load i: rows 4i .. 4i + 3, lane -> row 4i + lane / 16, chunk lane % 16 (rows past the end repeat the last cell; their weights are zero)
    u32x4 kraw[16], vraw[16];
#pragma unroll
    for (int i = 0; i < 16; i++) {
        int64_t cell = c0 + 4 * i + rsub;
        if (cell >= a.Nkv) cell = a.Nkv - 1;
        kraw[i] = load16(a.k + cell * a.k_nb1 + hk * a.k_nb2 + (pos << 4));
        vraw[i] = load16(a.v + cell * a.v_nb1 + hk * a.v_nb2 + (pos << 4));
    }
    const int64_t cell = c0 + lane;
    unsigned short mbits = 0xFC00;   // -inf
    if (cell < a.Nkv) mbits = a.mask ? ((const unsigned short *)a.mask)[cell] : (unsigned short)0;
    // q of the group's four heads: two coalesced loads per lane (chunk ch of 128: head ch / 32, floats 4 (ch % 32) .. + 3), rounded to
    // f16 into the wave's 1 KiB of LDS; every lane then reads the 128 values of head lane % 4 (128 floats per lane in flight would
    // not fit beside the K and V tiles)
    f32x4 qraw[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int ch = lane + 64 * j, head = ch >> 5;
        qraw[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (head < R) qraw[j] = *(const f32x4 *)(a.q + (hk * R + head) * a.q_nb2 + (size_t)(ch & 31) * 16);
    }
    float slope[4];
    fs_slopes(a, hk * R, slope);
    const float scale = a.softcap != 0.0f ? a.scale / a.softcap : a.scale;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int ch = lane + 64 * j;
        const f16x2 p0 = {(_Float16)qraw[j][0], (_Float16)qraw[j][1]}, p1 = {(_Float16)qraw[j][2], (_Float16)qraw[j][3]};
        const u32x2 packed = {__builtin_bit_cast(u32, p0), __builtin_bit_cast(u32, p1)};
        *(u32x2 *)(&qbuf[wave][0][0] + ch * 4) = packed;
    }
    u32 qv[FS_D / 2];
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const u32x4 t = *(const u32x4 *)(&qbuf[wave][lane & 3][0] + i * 8);
        qv[4 * i] = t[0];
        qv[4 * i + 1] = t[1];
        qv[4 * i + 2] = t[2];
        qv[4 * i + 3] = t[3];
    }

    // K through LDS: chunk c of row r at position c ^ (r & 15); then each lane reads the row of its cell
    uint8_t *tb = tbuf + wave * FS_KT;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int row = 4 * i + rsub;
        *(u32x4 *)(tb + row * FS_ROW + ((pos ^ (row & 15)) << 4)) = kraw[i];
    }
    u32x4 kc[16];
#pragma unroll
    for (int c = 0; c < 16; c++) kc[c] = *(const u32x4 *)(tb + lane * FS_ROW + ((c ^ (lane & 15)) << 4));

    fs_state S;
    fs_init(S);
    const unsigned p_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned short *)&pbuf[wave][0][0];
    fs_scores(qv, kc, half_bits_to_float(mbits), scale, a.softcap, slope, p_base + (unsigned)lane * 2, S);

    // V through the same bytes, row-major (the K rows are in registers)
#pragma unroll
    for (int i = 0; i < 16; i++) *(u32x4 *)(tb + (4 * i + rsub) * FS_ROW + (pos << 4)) = vraw[i];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // fs_output reads LDS through inline assembly: nothing may be moved across
    fs_output((unsigned)(uintptr_t)(void __attribute__((address_space(3))) *)tb + fs_v_lane(lane), p_base + (unsigned)(lane & 3) * (FS_TILE * 2), S);

    // ---- the waves' states meet in LDS
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const float L = wave_sum_dpp(S.lsum[r]);
        if (lane == 0) {
            s_m[wave][r] = S.m[r];
            s_l[wave][r] = L;
        }
        s_o[wave][r][lane] = S.o0[r];
        s_o[wave][r][64 + lane] = S.o1[r];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < R * FS_D; idx += (int)blockDim.x) {   // whole waves: R * 128 and the group size are multiples of 64
        const int r = idx / FS_D, d = idx % FS_D;
        float M = s_m[0][r];
        for (int w = 1; w < n_waves; w++) M = fmaxf(M, s_m[w][r]);
        float L = 0.0f, O = 0.0f;
        for (int w = 0; w < n_waves; w++) {
            const float f = __expf(s_m[w][r] - M);
            L += s_l[w][r] * f;
            O += s_o[w][r][d] * f;
        }
        const int64_t head = hk * R + r;
        const float o = O / L;
        a.dst[head * FS_D + d] = o;
        if (a.act_q) quantize_lane32(o, a.act_q, a.act_s, head * FS_D + d);
    }
}

int launch_fattn_dec_short(hipStream_t s, fattn_args &a, int64_t D) {
    const int64_t R = a.Hq / a.Hkv;
    if (D != FS_D || a.Nq != 1 || R > 4 || a.Hkv > 65535 || a.Nkv > FSS_MAX_WAVES * FS_TILE) return 1;
    if ((a.q_nb2 % 16) != 0 || (a.k_nb1 % 16) != 0 || (a.k_nb2 % 16) != 0 || (a.v_nb1 % 16) != 0 || (a.v_nb2 % 16) != 0) return 1;
    const int n_waves = (int)((a.Nkv + FS_TILE - 1) / FS_TILE);
    MI355_LAUNCH(k_fattn_dec_short, dim3((unsigned)a.Hkv), dim3((unsigned)n_waves * 64), 0, s, a, (int)R);
    return launch_status("k_fattn_dec_short");
}

// One query token, head size 128, R <= 4 query heads per kv head, rows 16-byte aligned.  Sets a.n_splits; the caller merges the
// splits with k_fattn_combine.  Returns 1 when the shape is not served.
int launch_fattn_dec_stream(hipStream_t s, fattn_args &a, int64_t D, size_t ws_bytes) {
    const int64_t R = a.Hq / a.Hkv;
    if (D != FS_D || a.Nq != 1 || R > 4 || a.Hkv > 65535 || a.ws == nullptr) return 1;
    if ((a.q_nb2 % 16) != 0 || (a.k_nb1 % 16) != 0 || (a.k_nb2 % 16) != 0 || (a.v_nb1 % 16) != 0 || (a.v_nb2 % 16) != 0) return 1;
    const int64_t n_tiles = (a.Nkv + FS_TILE - 1) / FS_TILE;
    int64_t waves_per_head = FS_TOTAL_WAVES / a.Hkv;
    if (waves_per_head < FS_WAVES) waves_per_head = FS_WAVES;
    if (waves_per_head > 256) waves_per_head = 256;   // k_fattn_combine takes up to 256 splits
    int64_t tiles_per_wave = (n_tiles + waves_per_head - 1) / waves_per_head;
    if (tiles_per_wave > FS_MAX_TILES) return 1;
    int64_t n_splits = (n_tiles + tiles_per_wave - 1) / tiles_per_wave;
    n_splits = (n_splits + FS_WAVES - 1) / FS_WAVES * FS_WAVES;   // whole groups; a wave without tiles writes an empty partial
    if (ws_bytes < (size_t)a.Hq * (size_t)n_splits * (size_t)(FS_D + 2) * sizeof(float)) return 1;
    a.n_splits = (int)n_splits;
    MI355_LAUNCH(k_fattn_dec_stream, dim3((unsigned)(n_splits / FS_WAVES), (unsigned)a.Hkv), dim3(FS_WAVES * 64), 0, s, a, (int)tiles_per_wave, (int)n_tiles, (int)R);
    return launch_status("k_fattn_dec_stream");
}

// fsq_src of a kv_src in the device row layout; false when the operand does not have the shape the kernel moves (whole heads of four
// blocks inside one row of the owner, levels 16-byte and scales 4-byte aligned)
static bool fsq_describe(int type, const kv_src &q, fsq_src &o) {
    if (q.row_blocks <= 0 || q.base == nullptr) return false;
    const int64_t BB = type == MI355_Q8_0 ? Q8_0_BYTES : Q4_0_BYTES, LB = type == MI355_Q8_0 ? 32 : 16;
    const int64_t row0 = q.first_block / q.row_blocks, b0 = q.first_block % q.row_blocks, RB = q.row_blocks * BB;
    if (q.head_blocks < FS_D / 32) return false;   // (that heads and cells stay inside their rows of the owner was checked with kv_src)
    o.lv = q.base + row0 * RB + b0 * LB;
    o.sc = q.base + row0 * RB + q.row_blocks * LB + b0 * 2;
    o.head_lv = q.head_blocks * LB;
    o.head_sc = q.head_blocks * 2;
    o.cell_lv = q.cell_lv;
    o.cell_sc = q.cell_sc;
    if (((uintptr_t)o.lv & 15) != 0 || (o.head_lv & 15) != 0 || (o.cell_lv & 15) != 0 || ((uintptr_t)o.sc & 3) != 0 || (o.head_sc & 3) != 0 || (o.cell_sc & 3) != 0) return false;
    if (o.cell_lv >= ((int64_t)1 << 26) || o.cell_sc >= ((int64_t)1 << 26)) return false;   // the per-lane offsets are 32-bit
    return true;
}

// One query token over a long Q8_0 / Q4_0 cache in the device row layout (a.type_k, a.type_v, a.kq, a.vq filled in), head size 128,
// R <= 4.  Sets a.n_splits; the caller merges the splits with k_fattn_combine.  Returns 1 when the shape is not served.
int launch_fattn_dec_stream_q(hipStream_t s, fattn_args &a, int64_t D, size_t ws_bytes) {
    const int64_t R = a.Hq / a.Hkv;
    if (D != FS_D || a.Nq != 1 || R > 4 || a.Hkv > 65535 || a.ws == nullptr || (a.q_nb2 % 16) != 0) return 1;
    if ((a.type_k != MI355_Q8_0 && a.type_k != MI355_Q4_0) || (a.type_v != MI355_Q8_0 && a.type_v != MI355_Q4_0)) return 1;
    fsq_src ks, vs;
    if (!fsq_describe(a.type_k, a.kq, ks) || !fsq_describe(a.type_v, a.vq, vs)) return 1;
    const int64_t n_tiles = (a.Nkv + FS_TILE - 1) / FS_TILE;
    // Waves per group: all that LDS holds once every wave has a dozen tiles or more (131072 cells of 8 kv heads: 94.5 -> 82 us for
    // Q8_0, 90 -> 73 us for Q4_0); with fewer tiles, two per group spread over more compute units are quicker (32768 cells: 34 us
    // against 39 us).
    int nwv = fsq_waves_rt(a.type_k, a.type_v);
    if (n_tiles * a.Hkv < (int64_t)FSQ_TOTAL_GROUPS * nwv * 12) nwv = 2;
    int64_t waves_per_head = (int64_t)FSQ_TOTAL_GROUPS * nwv / a.Hkv;
    if (waves_per_head < nwv) waves_per_head = nwv;
    if (waves_per_head > 256) waves_per_head = 256;   // k_fattn_combine takes up to 256 splits
    int64_t tiles_per_wave = (n_tiles + waves_per_head - 1) / waves_per_head;
    if (tiles_per_wave > FSQ_MAX_TILES) return 1;
    int64_t n_splits = (n_tiles + tiles_per_wave - 1) / tiles_per_wave;
    n_splits = (n_splits + nwv - 1) / nwv * nwv;   // whole groups; a wave without tiles writes an empty partial
    if (n_splits > 256) return 1;
    if (ws_bytes < (size_t)a.Hq * (size_t)n_splits * (size_t)(FS_D + 2) * sizeof(float)) return 1;
    a.n_splits = (int)n_splits;
    const dim3 grid((unsigned)(n_splits / nwv), (unsigned)a.Hkv), block((unsigned)nwv * 64);
#define MI355_FSQ_LAUNCH(TK, TV) MI355_LAUNCH((k_fattn_dec_stream_q<TK, TV>), grid, block, 0, s, a, ks, vs, (int)tiles_per_wave, (int)n_tiles, (int)R)
    if (a.type_k == MI355_Q8_0 && a.type_v == MI355_Q8_0) MI355_FSQ_LAUNCH(MI355_Q8_0, MI355_Q8_0);
    else if (a.type_k == MI355_Q8_0) MI355_FSQ_LAUNCH(MI355_Q8_0, MI355_Q4_0);
    else if (a.type_v == MI355_Q8_0) MI355_FSQ_LAUNCH(MI355_Q4_0, MI355_Q8_0);
    else MI355_FSQ_LAUNCH(MI355_Q4_0, MI355_Q4_0);
#undef MI355_FSQ_LAUNCH
    return launch_status("k_fattn_dec_stream_q");
}

}  // namespace mi355
