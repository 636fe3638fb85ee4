// MUL_MAT for 33 .. 128 activation rows on Q4_K weights: a weight-streaming kernel on the int8 matrix cores.
//
// Between the few-row kernel (skinny.hip, up to 32 rows, per-32-block f32 scaling: bound by the vector ALU beyond that) and the
// tile kernels (mmq_k.hip / mmq_w.hip, built around a K loop with group barriers and, for the wide tiles, a 2-byte-per-weight
// image) a product with a few dozen activation rows is bound by the weight bytes, which should be read once, packed, and by
// nothing else.  Here
//   * a wave owns 32 weight rows and a part of the launch's K range and never waits for another wave until the end; the rows'
//     nibbles and headers travel from memory straight into the wave's own ring of LDS stages (global-to-LDS transfers, two
//     256-element super-blocks ahead, no registers in between) and are read back in operand order;
//   * the activations are quantized per super-block exactly as ggml-cpu does it (quantize_row_q8_K_ref, ggml-quants.c:2479-2516)
//     and kept as tile images (tiles.hpp), whose 16-byte chunks ARE matrix-core operands: they go from L2 straight into registers;
//   * the 6-bit sub-block scale is folded into the weight operand while it is unpacked: sc = 8 a + b, nibble n -> the two int8
//     planes a n and b n (one 32-bit multiply per four weights and plane), so v_mfma_i32_32x32x32_i8 accumulates a whole
//     super-block in int32 and the vector ALU touches a result once per 256 elements: sum_j sc_j (q4 . q8)_j = 8 HI + LO, the
//     integer ggml_vec_dot_q4_K_q8_K forms (ggml-cpu-quants.c:6817-6848);
//   * the minimum term sum_j m_j bsum_j is one v_mfma_f32_32x32x16_f16 per super-block on exact small integers (m_j and 64 m_j
//     against bsum_j & 63 and bsum_j >> 6);
//   * a wave contracts its weights with one or two activation tiles of 32 rows (an unpacked operand then serves two matrix
//     instructions); a group's four waves are four parts of K, or two parts of K times two pairs of tiles; the parts meet in LDS
//     at the end and are added in a fixed order; products with few 32-row tiles are also cut into slices of K whose partial sums a second
//     launch adds (with the residual);
//   * the operands of the next super-block are requested into the registers of the current one as soon as each has been used.
// A lane ends up with ONE weight row and 16 activation rows, so the weight scales are per-lane scalars.
// Result: the CPU path's integer sums, f32 summation order aside.
#include "qdot.hpp"
#include "tiles.hpp"

namespace mi355 {

namespace {

// A wave's ring of weight stages in LDS, filled by global-to-LDS transfers (no registers in between): per super-block four
// transfers of 8 rows x 128 bytes of nibbles (1 KiB each, placed 16 bytes further apart so that rows 8 apart fall into different
// banks) and one of the 32 rows' 16-byte headers (lanes 32..63 repeat them).  Slot p (16 bytes) of a nibble transfer holds piece
// (p & 7) ^ (p >> 3) of row p >> 3: lanes that read the same piece of 32 different rows then hit different banks.
constexpr int MID_STAGES = 3;
constexpr int MID_SPAN = 1024 + 16;
constexpr int MID_STAGE = 4 * MID_SPAN + 1024;

// chunks (64 columns = two 32-element blocks) of activation operands a wave holds ahead: a whole super-block with one activation
// tile per wave, half of one with two (registers)
template <int NB> constexpr int mid_ring() { return NB == 1 ? 4 : 2; }
template <int NB> struct mid_act {
    u32x4 a[NB][2 * mid_ring<NB>()];   // the lane's operand chunks of the ring's 32-element blocks, per activation tile
    f16x8 bs[NB];     // its rows' {bsum_j & 63} (kh = 0) or {bsum_j >> 6} (kh = 1)
};

// grid.x = 32-row tiles of the weight matrix, grid.y = slices of K (partial sums to `dst` as [slice][B][dst_stride] then).
// A wave contracts its 32 weight rows with NB activation tiles of 32 rows (an unpacked weight operand serves NB matrix
// instructions); the group's four waves are NBW such sets of tiles x 4 / NBW parts of the slice's K range: wave = part * NBW + set.
// Waves of one part copy the same weights, each to its own LDS (no barrier; the second copy comes from cache).
// act: tile images of B rows (mi355_quantize_act_q8k_tiled).
// Up to three matrices that read the same activation go out in one launch, their 32-row tiles numbered one matrix after the other
// (Q, K and V; gate and up: the small ones alone are a handful of groups each, and every launch costs its start-up).
struct mid_mat {
    const uint8_t *W;
    float *dst;
    const float *residual;   // may be null; same shape and stride as dst; may be dst itself
    int64_t N, dst_stride;
    int first_tile;          // index of the matrix's first 32-row tile in the launch (unused entries: INT_MAX)
};
struct mid_launch {
    mid_mat m[3];
};
template <int NB, int NBW>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 8)))
k_mm_mid_q4k(mid_launch P, const uint8_t *__restrict__ act, int K, int B, int steps_per_slice, int steps_per_wave) {
    const int mi = ((int)blockIdx.x >= P.m[1].first_tile ? 1 : 0) + ((int)blockIdx.x >= P.m[2].first_tile ? 1 : 0);   // uniform
    const uint8_t *__restrict__ W = P.m[mi].W;
    float *__restrict__ dst = P.m[mi].dst;
    const float *__restrict__ residual = P.m[mi].residual;
    const int64_t N = P.m[mi].N, dst_stride = P.m[mi].dst_stride;
    const int tile_x = (int)blockIdx.x - P.m[mi].first_tile;
    constexpr int KS = 4 / NBW;
    constexpr int WAVE_BYTES = MID_STAGES * MID_STAGE;
    constexpr int RED_BYTES = 4 * NB * 16 * 64 * 4;
    __shared__ __attribute__((aligned(16))) uint8_t s_mem[4 * WAVE_BYTES > RED_BYTES ? 4 * WAVE_BYTES : RED_BYTES];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int set = wave % NBW, part = wave / NBW;
    const int r = lane & 31, kh = lane >> 5;
    uint8_t *ring = s_mem + wave * WAVE_BYTES;
    const unsigned ring_lds = (unsigned)(uintptr_t)(void __attribute__((address_space(3))) *)ring;

    const int64_t row0 = (int64_t)tile_x * 32;
    const int nsteps = K >> 8;
    const int slice_lo = blockIdx.y * steps_per_slice;
    const int slice_hi = slice_lo + steps_per_slice < nsteps ? slice_lo + steps_per_slice : nsteps;
    const int s_lo = slice_lo + part * steps_per_wave;
    const int s_hi = s_lo + steps_per_wave < slice_hi ? s_lo + steps_per_wave : slice_hi;   // may be <= s_lo: a wave without steps

    // sources of the transfers: 32-bit offsets from W (the launcher keeps matrices below 4 GiB); rows past the end repeat the
    // last row and are not stored
    const int64_t row_bytes = (int64_t)nsteps * Q4_K_BYTES;
    unsigned w_off[4], h_off;
#pragma unroll
    for (int u = 0; u < 4; u++) {
        int64_t row = row0 + 8 * u + (lane >> 3);
        row = row < N ? row : N - 1;
        w_off[u] = (unsigned)(row * row_bytes + 16 + 16 * ((lane & 7) ^ ((lane >> 3) & 7)));
    }
    {
        const int64_t my_row = row0 + r < N ? row0 + r : N - 1;
        h_off = (unsigned)(my_row * row_bytes);
    }
    auto dma = [&](const uint8_t *g, unsigned off, uint8_t *l) {   // g, l: wave-uniform
        asm volatile("" : "+v"(off));   // keeps the sum from being formed per lane ahead of the loop (two registers per source)
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)(g + off), (void __attribute__((address_space(3))) *)l, 16, 0, 0);
    };
    auto issue = [&](int step, int slot) {   // super-block `step` of the wave's rows into stage `slot`
        const uint8_t *g = W + (int64_t)step * Q4_K_BYTES;
        uint8_t *st = ring + slot * MID_STAGE;
#pragma unroll
        for (int u = 0; u < 4; u++) dma(g, w_off[u], st + u * MID_SPAN);
        dma(g, h_off, st + 4 * MID_SPAN);
    };
    // what the lane reads back: its own row's header, and piece 2 g + kh of its row for chunk g
    const unsigned rd_hdr = 4 * MID_SPAN + r * 16;
    unsigned rd_w[4];
#pragma unroll
    for (int g = 0; g < 4; g++) rd_w[g] = (unsigned)((r >> 3) * MID_SPAN + ((r & 7) * 8 + ((2 * g + kh) ^ (r & 7))) * 16);

    // activation operands: lane (r, kh) supplies levels 16 kh .. + 16 of a 32-element block of activation row 32 (NB set + nb) + r
    const int64_t b16 = ((int64_t)B + 15) & ~(int64_t)15;
    const int64_t cb_pad = wt_cb_pad(B);
    const int64_t aux0 = b16 * K;   // the records behind the image
    // 32-bit offsets from `act` (the launcher keeps images below 4 GiB): a uniform base plus one register per address
    u32 a_tile[NB];   // the lane's row inside its 16-row block's first tile
    u32 a_rec[NB];    // its sums in the block's record, super-block 0
    int a_sw[NB];     // chunk swizzle of that row
    u32 d_rec[NB][2];   // scales of the tile's two 16-row blocks, first row of the lane's four; the lane's 16 results
                        // of a tile are activation rows 8 q + 4 kh + i (q, i = 0..3) of the tile
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        int64_t arow = (int64_t)32 * (NB * set + nb) + r;
        arow = arow < b16 ? arow : b16 - 1;   // rows past the image repeat its last row; their results are not stored
        const int r16 = (int)(arow & 15);
        a_tile[nb] = (u32)((arow >> 4) * (int64_t)(K >> 6) * WT_TILE + r16 * 64);
        a_sw[nb] = (r16 >> 2) & 3;
        a_rec[nb] = (u32)(aux0 + (arow >> 4) * WT_A_AUX + 64 + r16 * 32 + kh * 16);
#pragma unroll
        for (int hb = 0; hb < 2; hb++) {
            int64_t rb = (int64_t)2 * (NB * set + nb) + hb;
            rb = rb < cb_pad ? rb : cb_pad - 1;
            d_rec[nb][hb] = (u32)(aux0 + rb * WT_A_AUX + 4 * kh * 4);
        }
    }
    const u32 rec_step = (u32)(cb_pad * WT_A_AUX);

    constexpr int RING = mid_ring<NB>();
    auto fetch_a = [&](int step, int g, mid_act<NB> &A) {   // the two blocks of chunk g (one 64-column tile) into ring slot g % RING
        const int s = step < nsteps ? step : nsteps - 1;
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int h = 0; h < 2; h++)
                A.a[nb][2 * (g % RING) + h] = load16(act + (a_tile[nb] + (u32)(s * 4 + g) * WT_TILE + (u32)(((2 * h + kh) ^ a_sw[nb]) << 4)));
    };
    auto fetch_s = [&](int step, mid_act<NB> &A) {
        const int s = step < nsteps ? step : nsteps - 1;
#pragma unroll
        for (int nb = 0; nb < NB; nb++) A.bs[nb] = *(const f16x8 *)(act + (a_rec[nb] + (u32)s * rec_step));
    };

    f32x16 accf[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int i = 0; i < 16; i++) accf[nb][i] = 0.0f;

    mid_act<NB> A;
    // order of the requests: the weight stages first, then the activation operands of the same super-block, so that the arrival
    // of a super-block's first activation operand (loads complete in order) says that its weight stage has landed
#pragma unroll
    for (int p = 0; p < MID_STAGES - 1; p++)
        if (s_lo + p < s_hi) issue(s_lo + p, p);
    if (s_lo < s_hi) {
#pragma unroll
        for (int g = 0; g < RING; g++) fetch_a(s_lo, g, A);
        fetch_s(s_lo, A);
    }
    int slot = 0;   // stage of the current super-block
    for (int step = s_lo; step < s_hi; step++) {
        {   // the stage read last step takes the super-block MID_STAGES - 1 on
            const int ahead = step + MID_STAGES - 1;
            const int aslot = slot == 0 ? MID_STAGES - 1 : slot - 1;
            if (ahead < s_hi) issue(ahead, aslot);
        }
        // ---- the lane's header and its four operand pieces out of the stage (inline assembly: the compiler would wait for every
        //      transfer in flight before an LDS read it can see).  The first read names an activation operand of this super-block
        //      as an input, which puts the compiler's wait for that operand - and with it the arrival of the stage - in front.
        const unsigned st = ring_lds + (unsigned)slot * MID_STAGE;
        u32x4 hdr, wq[4];
        asm volatile("ds_read_b128 %0, %1" : "=v"(hdr) : "v"(st + rd_hdr), "v"(A.a[0][0]) : "memory");
#pragma unroll
        for (int g = 0; g < 4; g++) asm volatile("ds_read_b128 %0, %1" : "=v"(wq[g]) : "v"(st + rd_w[g]) : "memory");
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(hdr), "+v"(wq[0]), "+v"(wq[1]), "+v"(wq[2]), "+v"(wq[3]) : : "memory");
        slot = slot == MID_STAGES - 1 ? 0 : slot + 1;

        // all eight 6-bit (scale, min) pairs as the bytes of four words (get_scale_min_k4, ggml-quants.c:631-638)
        const float d = half_bits_to_float((unsigned short)(hdr[0] & 0xFFFFu));
        const float dmin = half_bits_to_float((unsigned short)(hdr[0] >> 16));
        const u32 u0 = hdr[1], u1 = hdr[2], u2 = hdr[3];
        const u32 sc_lo = u0 & 0x3F3F3F3Fu, m_lo = u1 & 0x3F3F3F3Fu;
        const u32 sc_hi = (u2 & 0x0F0F0F0Fu) | (((u0 >> 6) & 0x03030303u) << 4);
        const u32 m_hi = ((u2 >> 4) & 0x0F0F0F0Fu) | (((u1 >> 6) & 0x03030303u) << 4);

        // ---- minimum term: B operand = {m_j} (kh = 0) or {64 m_j} (kh = 1) of the lane's row, A operand = the activation row's
        //      {bsum_j & 63} (kh = 0) or {bsum_j >> 6} (kh = 1): sum over the 16 products = sum_j m_j bsum_j, exact in f32
        f16x8 mop;
        {
            const float f = kh ? 64.0f : 1.0f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const u32 M = j < 4 ? m_lo : m_hi;
                mop[j] = (_Float16)(f * (float)((M >> (8 * (j & 3))) & 0xFFu));
            }
        }
        i32x16 hi[NB], lo[NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int i = 0; i < 16; i++) { hi[nb][i] = 0; lo[nb][i] = 0; }
        f32x4 d8[NB][4];   // the scales of the rows this lane finishes: wanted at the end of the step, requested before its last chunk
#pragma unroll
        for (int g = 0; g < 4; g++) {   // chunk g: sub-blocks 2 g (low nibbles) and 2 g + 1 (high nibbles), one 64-column tile
            if (g == 3) {
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
#pragma unroll
                    for (int q = 0; q < 4; q++) d8[nb][q] = *(const f32x4 *)(act + (d_rec[nb][q >> 1] + (u32)step * rec_step + (u32)((8 * (q & 1)) * 4)));
            }
            const u32x4 v = wq[g];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int j = 2 * g + h;
                const u32 S = j < 4 ? sc_lo : sc_hi;
                const u32 sc = (S >> (8 * (j & 3))) & 0xFFu;
                const u32 a = sc >> 3, b = sc & 7u;
                i32x4 wh, wl;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const u32 n = (v[i] >> (4 * h)) & 0x0F0F0F0Fu;
                    wh[i] = (int)(n * a);   // bytes <= 15 * 7: no carries between them
                    wl[i] = (int)(n * b);
                }
#pragma unroll
                for (int nb = 0; nb < NB; nb++) {
                    hi[nb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, A.a[nb][2 * (g % RING) + h]), wh, hi[nb], 0, 0, 0);
                    lo[nb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, A.a[nb][2 * (g % RING) + h]), wl, lo[nb], 0, 0, 0);
                }
            }
            // the chunk's registers take the operands RING chunks on
            if (g + RING < 4) fetch_a(step, g + RING, A);
            else if (step + 1 < s_hi) fetch_a(step + 1, g + RING - 4, A);
        }
        // ---- finish the super-block: accf += d8 (d (8 HI + LO) - dmin MS)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            f32x16 z;
#pragma unroll
            for (int i = 0; i < 16; i++) z[i] = 0.0f;
            const f32x16 ms = __builtin_amdgcn_mfma_f32_32x32x16_f16(A.bs[nb], mop, z, 0, 0, 0);
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float isum = (float)(8 * hi[nb][4 * q + i] + lo[nb][4 * q + i]);
                    const float t = __builtin_fmaf(d, isum, -(dmin * ms[4 * q + i]));
                    accf[nb][4 * q + i] = __builtin_fmaf(d8[nb][q][i], t, accf[nb][4 * q + i]);
                }
        }
        if (step + 1 < s_hi) fetch_s(step + 1, A);
    }

    // the parts of K: fixed order 0, 1, ...
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no transfer is in flight when the ring's memory changes hands
    __syncthreads();
    float *s_red = (float *)s_mem;   // [wave][NB * 16][64]
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int i = 0; i < 16; i++) s_red[((wave * NB + nb) * 16 + i) * 64 + lane] = accf[nb][i];
    __syncthreads();
    // value v = (set, tile of the set, i) is finished by wave v % 4
    for (int v = wave; v < NBW * NB * 16; v += 4) {
        const int tset = v / (NB * 16), tnb = (v / 16) % NB, i = v & 15;
        float sum = s_red[(((0 * NBW + tset) * NB + tnb) * 16 + i) * 64 + lane];
#pragma unroll
        for (int p = 1; p < KS; p++) sum += s_red[(((p * NBW + tset) * NB + tnb) * 16 + i) * 64 + lane];
        const int c = 32 * (NB * tset + tnb) + 8 * (i >> 2) + 4 * kh + (i & 3);
        if (c < B && row0 + r < N) {
            const int64_t o = ((int64_t)blockIdx.y * B + c) * dst_stride + row0 + r;
            dst[o] = residual ? sum + residual[o] : sum;
        }
    }
}

// sum of the K slices: dst[c][n] = sum_s part[s][c][n] (+ residual), slices in ascending order; blockIdx.z = matrix of the launch,
// whose partial sums lie behind those of the matrices before it
struct mid_sum {
    const float *part[3];
    float *dst[3];
    const float *residual[3];
    int64_t N[3], dst_stride[3];
};
__global__ void __launch_bounds__(256) k_mid_slices(mid_sum S, int B, int slices) {
    const int mi = blockIdx.z;
    const int64_t N = S.N[mi];
    const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int c = blockIdx.y;
    if (n >= N) return;
    const float *__restrict__ part = S.part[mi];
    float sum = part[(int64_t)c * N + n];
    for (int s = 1; s < slices; s++) sum += part[((int64_t)s * B + c) * N + n];
    const int64_t o = c * S.dst_stride[mi] + n;
    S.dst[mi][o] = S.residual[mi] ? sum + S.residual[mi][o] : sum;
}

// sets of activation tiles across the waves of a group (a wave takes 1 tile up to 32 rows, 2 beyond)
int mid_sets(int64_t B) { return B <= 64 ? 1 : 2; }

// slices of K: enough groups to cover the chip about twice, as long as a wave keeps two super-blocks
int mid_slices(int64_t N, int64_t K, int64_t B) {   // N: rows of all matrices of the launch (each a multiple of 32, or one matrix)
    const int64_t groups = (N + 31) / 32, nsteps = K >> 8;
    const int ks = 4 / mid_sets(B);
    int s = 1;
    while (s < 8 && groups * s < 448 && nsteps / (s * 2 * ks) >= 2) s *= 2;
    return s;
}

}  // namespace

}  // namespace mi355

using namespace mi355;

extern "C" {

int mi355_mul_mat_mid_supported(int type, const void *W, int64_t K, int64_t B) {
    return type == MI355_Q4_K && B >= 1 && B <= 128 && K > 0 && K % 256 == 0 && K < (int64_t(1) << 30) && ((uintptr_t)W & 15) == 0;
}

size_t mi355_mul_mat_mid_ws_bytes(int64_t N, int64_t K, int64_t B) {
    const int s = mid_slices(N, K, B);
    return s > 1 ? (size_t)s * B * N * sizeof(float) : 0;
}

// norm: the single matrix's rows are normalised next; taken when the product is cut along K, whose sum launch then carries the norm
struct mid_norm {
    const float *w;
    float eps;
    float *y;
    int64_t y_stride;
    void *act_out;
};
static int mul_mat_mid_launch(void *stream, int type, int n_mats, const mi355_gemv_mat *mats, const void *act, int64_t K, int64_t B, void *ws, size_t ws_bytes,
                              const mid_norm *norm, bool *norm_done);

int mi355_mul_mat_mid_multi(void *stream, int type, int n_mats, const mi355_gemv_mat *mats, const void *act, int64_t K, int64_t B, void *ws, size_t ws_bytes) {
    return mul_mat_mid_launch(stream, type, n_mats, mats, act, K, B, ws, ws_bytes, nullptr, nullptr);
}

int mi355_mul_mat_mid_norm(void *stream, int type, const void *W, const void *act, float *dst, const float *residual, int64_t N, int64_t K, int64_t B,
                           int64_t dst_stride, void *ws, size_t ws_bytes, const float *norm_w, float eps, float *y, int64_t y_stride, void *act_out) {
    MI355_REQUIRE(N > 0 && N % QKK == 0, "mul_mat_mid_norm: N=%lld must be a multiple of 256", (long long)N);
    MI355_REQUIRE(norm_w != nullptr && act_out != nullptr && ((uintptr_t)norm_w & 15) == 0 && ((uintptr_t)act_out & 15) == 0 && ((uintptr_t)y & 15) == 0 &&
                  y_stride % 4 == 0, "mul_mat_mid_norm: the norm's operands must be 16-byte aligned");
    mi355_gemv_mat m;
    m.type = type;
    m.W = W;
    m.N = N;
    m.dst = dst;
    m.dst_stride = dst_stride;
    m.residual = residual;
    const mid_norm nm = {norm_w, eps, y, y_stride, act_out};
    bool done = false;
    const int rc = mul_mat_mid_launch(stream, type, 1, &m, act, K, B, ws, ws_bytes, &nm, &done);
    if (rc != MI355_OK || done) return rc;
    return mi355_rms_norm_mul_quant_q8k_tiled(stream, dst, dst_stride, norm_w, y, y_stride, act_out, N, B, eps);   // an uncut product: the norm is its own launch
}

static int mul_mat_mid_launch(void *stream, int type, int n_mats, const mi355_gemv_mat *mats, const void *act, int64_t K, int64_t B, void *ws, size_t ws_bytes,
                              const mid_norm *norm, bool *norm_done) {
    MI355_REQUIRE(n_mats >= 1 && n_mats <= 3 && mats != nullptr, "mul_mat_mid: 1 to 3 matrices per launch, got %d", n_mats);
    MI355_REQUIRE(((uintptr_t)act & 15) == 0, "mul_mat_mid: activation image is not 16-byte aligned");
    MI355_REQUIRE(mi355_act_q8k_tiled_bytes(K, B) < ((size_t)1 << 32), "mul_mat_mid: activation image of 4 GiB or more");
    int64_t n_sum = 0, tiles = 0;
    mid_launch L;
    for (int i = 0; i < 3; i++) {
        const mi355_gemv_mat &m = mats[i < n_mats ? i : 0];
        if (i < n_mats) {
            MI355_REQUIRE(m.type == type && mi355_mul_mat_mid_supported(type, m.W, K, B), "mul_mat_mid: type %d, K=%lld, B=%lld or the weight alignment is not supported",
                          m.type, (long long)K, (long long)B);
            MI355_REQUIRE(m.N > 0 && m.dst_stride >= m.N && m.N < (int64_t(1) << 31), "mul_mat_mid: bad shape N=%lld dst_stride=%lld", (long long)m.N, (long long)m.dst_stride);
            MI355_REQUIRE(m.N * (K / 256 * Q4_K_BYTES) < (int64_t(1) << 32), "mul_mat_mid: matrix of 4 GiB or more");
        }
        L.m[i].W = (const uint8_t *)m.W;
        L.m[i].dst = m.dst;
        L.m[i].residual = m.residual;
        L.m[i].N = m.N;
        L.m[i].dst_stride = m.dst_stride;
        L.m[i].first_tile = i < n_mats ? (int)tiles : 0x7fffffff;
        if (i < n_mats) {
            tiles += (m.N + 31) / 32;
            n_sum += m.N;
        }
    }
    MI355_REQUIRE(tiles < (1 << 30), "mul_mat_mid: too many tiles");
    int slices = mid_slices(tiles * 32, K, B);
    if (slices > 1 && (ws == nullptr || ws_bytes < (size_t)slices * B * n_sum * sizeof(float))) slices = 1;   // no room for partial sums: one slice
    hipStream_t s = (hipStream_t)stream;
    const int nsteps = (int)(K >> 8);
    const int steps_per_slice = (nsteps + slices - 1) / slices;
    const int nbw = mid_sets(B);
    const int steps_per_wave = (steps_per_slice + 4 / nbw - 1) / (4 / nbw);
    const dim3 grid((unsigned)tiles, (unsigned)slices);
    mid_sum S;
    int64_t n_max = 0;
    if (slices > 1) {   // partial sums: per matrix [slice][B][N], one matrix after the other
        float *part = (float *)ws;
        for (int i = 0; i < 3; i++) {
            const int k = i < n_mats ? i : 0;
            S.part[i] = part;
            S.dst[i] = mats[k].dst;
            S.residual[i] = mats[k].residual;
            S.N[i] = mats[k].N;
            S.dst_stride[i] = mats[k].dst_stride;
            if (i < n_mats) {
                L.m[i].dst = part;
                L.m[i].residual = nullptr;
                L.m[i].dst_stride = mats[i].N;
                part += (int64_t)slices * B * mats[i].N;
                n_max = mats[i].N > n_max ? mats[i].N : n_max;
            }
        }
    }
#define MI355_MID_ARGS grid, dim3(256), 0, s, L, (const uint8_t *)act, (int)K, (int)B, steps_per_slice, steps_per_wave
    if (B <= 32) MI355_LAUNCH((k_mm_mid_q4k<1, 1>), MI355_MID_ARGS);
    else if (B <= 64) MI355_LAUNCH((k_mm_mid_q4k<2, 1>), MI355_MID_ARGS);
    else MI355_LAUNCH((k_mm_mid_q4k<2, 2>), MI355_MID_ARGS);
#undef MI355_MID_ARGS
    if (slices > 1 && norm && n_mats == 1 && mats[0].N <= 4096 && mats[0].N % 4 == 0 && mats[0].dst_stride % 4 == 0 && ((uintptr_t)mats[0].dst & 15) == 0 &&
        (mats[0].residual == nullptr || ((uintptr_t)mats[0].residual & 15) == 0) && ((uintptr_t)ws & 15) == 0) {
        launch_split_sum_norm(s, (const float *)ws, mats[0].dst, mats[0].residual, mats[0].N, B, mats[0].dst_stride, slices, norm->w, norm->eps, norm->y,
                              norm->y_stride, norm->act_out);
        *norm_done = true;
    } else if (slices > 1) {
        MI355_LAUNCH(k_mid_slices, dim3((unsigned)((n_max + 255) / 256), (unsigned)B, (unsigned)n_mats), dim3(256), 0, s, S, (int)B, slices);
    }
    return launch_status("k_mm_mid");
}

size_t mi355_mul_mat_mid_multi_ws_bytes(int n_mats, const int64_t *Ns, int64_t K, int64_t B) {
    if (n_mats < 1 || n_mats > 3 || Ns == nullptr) return 0;
    int64_t n_sum = 0, tiles = 0;
    for (int i = 0; i < n_mats; i++) {
        n_sum += Ns[i];
        tiles += (Ns[i] + 31) / 32;
    }
    const int s = mid_slices(tiles * 32, K, B);
    return s > 1 ? (size_t)s * B * n_sum * sizeof(float) : 0;
}

int mi355_mul_mat_mid(void *stream, int type, const void *W, const void *act, float *dst, const float *residual, int64_t N, int64_t K, int64_t B,
                      int64_t dst_stride, void *ws, size_t ws_bytes) {
    mi355_gemv_mat m;
    m.type = type;
    m.W = W;
    m.N = N;
    m.dst = dst;
    m.dst_stride = dst_stride;
    m.residual = residual;
    return mi355_mul_mat_mid_multi(stream, type, 1, &m, act, K, B, ws, ws_bytes);
}

}  // extern "C"
