// FLASH_ATTN_EXT for one query token over a long f16 KV cache (head size 128, up to four query heads per kv head): the
// streaming form.
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
// Scores of one tile (kc: the 16 chunks of this lane's K row), the soft-max update of the state, and P^T (head, cell) as f16 into
// the wave's 512 bytes of LDS at p_wr (= base + 2 * lane), where fs_output reads it back as the A operand.  LDS serves a wave's
// operations in order: those reads see these writes, and the next tile's writes come after them.
__device__ __forceinline__ void fs_scores(const u32 (&qv)[FS_D / 2], const u32x4 (&kc)[16], float mv, float scale, float softcap, const float (&slope)[4],
                                          unsigned p_wr, fs_state &S) {
    constexpr float NEG = -FLT_MAX / 2;
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 16; c++) {
        const u32 a0 = qv[4 * c], a1 = qv[4 * c + 1], a2 = qv[4 * c + 2], a3 = qv[4 * c + 3];
        const u32 b0 = kc[c][0], b1 = kc[c][1], b2 = kc[c][2], b3 = kc[c][3];
        const u32x2 qa = {a0, a1}, qb = {a2, a3}, ka = {b0, b1}, kb2 = {b2, b3};
        s0 = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, qa), __builtin_bit_cast(f16x4, ka), s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, qb), __builtin_bit_cast(f16x4, kb2), s1, 0, 0, 0);
    }
    const bool valid = mv != -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        float sc = (s0[r] + s1[r]) * scale;
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
// This lane's offset inside a row-major V tile for the transposing reads of fs_output: lane l' = lane % 16 of its 16-lane group
// g points at row c0 + l' / 4, elements 16 g + 4 (l' % 4) .. + 3
__device__ __forceinline__ unsigned fs_v_lane(int lane) {
    return (unsigned)((lane & 15) >> 2) * FS_ROW + (unsigned)((lane >> 4) * 16 + (lane & 3) * 4) * 2;
}
// Output of one tile: four cells per step, elements lane and 64 + lane; every operand of the tile is requested before the first
// is used.  v_addr: LDS byte address of the V tile + fs_v_lane; p_rd: the wave's P^T + 128 * (lane % 4).
__device__ __forceinline__ void fs_output(unsigned v_addr, unsigned p_rd, fs_state &S) {
    u32x2 vlo[16], vhi[16], pa[16];
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const unsigned addr = v_addr + (unsigned)(j * 4 * FS_ROW);
        asm volatile("ds_read_b64 %0, %1" : "=v"(pa[j]) : "v"(p_rd + (unsigned)(j * 8)));
        asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(vlo[j]) : "v"(addr));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:128" : "=v"(vhi[j]) : "v"(addr));
    }
#pragma unroll
    for (int jb = 0; jb < 16; jb += 8)   // the wait names its registers so that nothing is used ahead of it; 24 operands per statement
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(vlo[jb]), "+v"(vlo[jb + 1]), "+v"(vlo[jb + 2]), "+v"(vlo[jb + 3]), "+v"(vlo[jb + 4]), "+v"(vlo[jb + 5]), "+v"(vlo[jb + 6]), "+v"(vlo[jb + 7]),
                       "+v"(vhi[jb]), "+v"(vhi[jb + 1]), "+v"(vhi[jb + 2]), "+v"(vhi[jb + 3]), "+v"(vhi[jb + 4]), "+v"(vhi[jb + 5]), "+v"(vhi[jb + 6]), "+v"(vhi[jb + 7]),
                       "+v"(pa[jb]), "+v"(pa[jb + 1]), "+v"(pa[jb + 2]), "+v"(pa[jb + 3]), "+v"(pa[jb + 4]), "+v"(pa[jb + 5]), "+v"(pa[jb + 6]), "+v"(pa[jb + 7]));
#pragma unroll
    for (int j = 0; j < 16; j++) {
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

}  // namespace mi355
