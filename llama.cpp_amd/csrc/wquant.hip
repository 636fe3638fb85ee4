// Weight quantizers on the device: f32 rows -> blocks in the reference's own byte layout, bit for bit what the reference's
// quantize_row_*_ref functions write (ggml/src/ggml-quants.c: q4_0 :31-66, q8_0 :194-217, q4_K :1208-1278, q5_K :1395-1480,
// q6_K :1620-1688, q4_1 / q5_0 / q5_1 :68-192, iq4_nl / iq4_xs :4573-4745, with make_qkx2_quants :550-629, make_qx_quants :379-446 and nearest_int :372-377) - the functions llama-quantize
// runs without an importance matrix (ggml_quantize_chunk, ggml/src/ggml.c:6410).  Used to build model files and resident models
// from f32 tensors without a host pass.
//
// The searches are sequential per group of 32 (16 for Q6_K) elements and are kept that way: one thread per group with the
// group in registers, every sum in the reference's order, no contraction of multiplies and adds (the reference is compiled as
// ISO C, where the compiler may not contract either), correctly rounded division and square root.  The threads of a 256-element
// super-block (8, or 16 for Q6_K) are neighbouring lanes and meet through cross-lane moves and LDS for the super-block's scales
// and the packing of the levels.
#include "common.hpp"

namespace mi355 {

namespace {

#define MI355_EXACT _Pragma("clang fp contract(off)")

__device__ __forceinline__ int nearest_int(float fval) {   // round to nearest even by the magic-number addition
    MI355_EXACT
    const float val = fval + 12582912.f;
    return (__builtin_bit_cast(int, val) & 0x007fffff) - 0x00400000;
}
__device__ __forceinline__ int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// make_qkx2_quants(32, NMAX, x, weights, L, &the_min, Laux, rmin, rdelta, nstep, false)
template <int NMAX>
__device__ __forceinline__ float qkx2_quants(const float (&x)[32], const float (&w)[32], int (&L)[32], float &the_min, float rmin, float rdelta, int nstep) {
    MI355_EXACT
    float mn = x[0], mx = x[0];
    float sum_w = w[0];
    float sum_x = sum_w * x[0];
#pragma unroll
    for (int i = 1; i < 32; i++) {
        if (x[i] < mn) mn = x[i];
        if (x[i] > mx) mx = x[i];
        sum_w += w[i];
        sum_x += w[i] * x[i];
    }
    if (mn > 0) mn = 0;
    if (mx == mn) {
#pragma unroll
        for (int i = 0; i < 32; i++) L[i] = 0;
        the_min = -mn;
        return 0.f;
    }
    float iscale = (float)NMAX / (mx - mn);
    float scale = 1 / iscale;
    float best_mad = 0;
#pragma unroll
    for (int i = 0; i < 32; i++) {
        const int l = nearest_int(iscale * (x[i] - mn));
        L[i] = clampi(l, 0, NMAX);
        float diff = scale * (float)L[i] + mn - x[i];
        diff = diff * diff;
        best_mad += w[i] * diff;
    }
    for (int is = 0; is <= nstep; is++) {
        iscale = (rmin + rdelta * (float)is + (float)NMAX) / (mx - mn);
        float sum_l = 0, sum_l2 = 0, sum_xl = 0;
        int Laux[32];
#pragma unroll
        for (int i = 0; i < 32; i++) {
            int l = nearest_int(iscale * (x[i] - mn));
            l = clampi(l, 0, NMAX);
            Laux[i] = l;
            const float fl = (float)l;
            sum_l += w[i] * fl;
            sum_l2 += w[i] * fl * fl;
            sum_xl += w[i] * fl * x[i];
        }
        const float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0) {
                this_min = 0;
                this_scale = sum_xl / sum_l2;
            }
            float mad = 0;
#pragma unroll
            for (int i = 0; i < 32; i++) {
                float diff = this_scale * (float)Laux[i] + this_min - x[i];
                diff = diff * diff;
                mad += w[i] * diff;
            }
            if (mad < best_mad) {
#pragma unroll
                for (int i = 0; i < 32; i++) L[i] = Laux[i];
                best_mad = mad;
                scale = this_scale;
                mn = this_min;
            }
        }
    }
    the_min = -mn;
    return scale;
}

// quantize_row_q4_K_ref (FIVE = false) and quantize_row_q5_K_ref (FIVE = true): thread = one 32-element sub-block, eight
// neighbouring lanes = one super-block
template <bool FIVE>
__global__ void __launch_bounds__(256) k_quantize_q45_K(const float *__restrict__ x, uint8_t *__restrict__ y, int64_t n_sub) {
    MI355_EXACT
    constexpr int NMAX = FIVE ? 31 : 15;
    constexpr int BLOCK = FIVE ? Q5_K_BYTES : Q4_K_BYTES;
    const int64_t sub = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool live = sub < n_sub;              // whole super-blocks are live or not (n_sub is a multiple of 8)
    const int64_t s = live ? sub : n_sub - 1;
    const int j = (int)(s & 7);
    float xv[32], w[32];
    {
        const f32x4 *p = (const f32x4 *)(x + s * 32);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const f32x4 v = p[i];
            xv[4 * i] = v[0]; xv[4 * i + 1] = v[1]; xv[4 * i + 2] = v[2]; xv[4 * i + 3] = v[3];
        }
    }
    float sum_x2 = 0;
#pragma unroll
    for (int l = 0; l < 32; l++) sum_x2 += xv[l] * xv[l];
    const float av_x = sqrtf(sum_x2 / 32);
#pragma unroll
    for (int l = 0; l < 32; l++) w[l] = av_x + fabsf(xv[l]);
    int L[32];
    float mn;
    const float scale = FIVE ? qkx2_quants<NMAX>(xv, w, L, mn, -0.5f, 0.1f, 15) : qkx2_quants<NMAX>(xv, w, L, mn, -1.f, 0.1f, 20);
    // the super-block's largest scale and minimum
    float max_scale = scale > 0 ? scale : 0, max_min = mn > 0 ? mn : 0;
#pragma unroll
    for (int off = 1; off < 8; off <<= 1) {
        max_scale = fmaxf(max_scale, __shfl_xor(max_scale, off, 64));
        max_min = fmaxf(max_min, __shfl_xor(max_min, off, 64));
    }
    const float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
    const float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
    int ls = nearest_int(inv_scale * scale) & 0xFF, lm = nearest_int(inv_min * mn) & 0xFF;   // stored through uint8_t
    ls = ls < 63 ? ls : 63;
    lm = lm < 63 ? lm : 63;
    const unsigned short dh = float_to_half_bits(max_scale / 63.f), dmh = float_to_half_bits(max_min / 63.f);
    // final levels with the stored scales
    const float d = half_bits_to_float(dh) * (float)ls;
    if (d != 0.0f) {
        const float dm = half_bits_to_float(dmh) * (float)lm;
#pragma unroll
        for (int i = 0; i < 32; i++) L[i] = clampi(nearest_int((xv[i] + dm) / d), 0, NMAX);
    }
    // ---- packing: the 12 scale bytes by the super-block's first lane, the nibbles by the even lanes (with the odd neighbour's),
    //      Q5_K's fifth bits by every lane for four of the 32 bytes
    const int lane = threadIdx.x & 63, base = lane & ~7;
    int all_ls[8], all_lm[8];
#pragma unroll
    for (int k = 0; k < 8; k++) {
        all_ls[k] = __shfl(ls, base + k, 64);
        all_lm[k] = __shfl(lm, base + k, 64);
    }
    u32 low[8];   // the sub-block's low nibbles, four per word
    u32 hb = 0;   // bit l: level l of this sub-block is above 15
#pragma unroll
    for (int i = 0; i < 8; i++) {
        low[i] = 0;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const int l = L[4 * i + b];
            low[i] |= (u32)(l & 15) << (8 * b);
            hb |= (u32)(l > 15) << (4 * i + b);
        }
    }
    u32 other[8];
#pragma unroll
    for (int i = 0; i < 8; i++) other[i] = __shfl_down(low[i], 1, 64);
    u32 hbs[8];
#pragma unroll
    for (int k = 0; k < 8; k++) hbs[k] = __shfl(hb, base + k, 64);
    if (!live) return;
    uint8_t *blk = y + (s >> 3) * BLOCK;
    if (j == 0) {
        uint8_t sc[12];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            sc[k] = (uint8_t)(all_ls[k] | ((all_ls[k + 4] >> 4) << 6));
            sc[k + 4] = (uint8_t)(all_lm[k] | ((all_lm[k + 4] >> 4) << 6));
            sc[k + 8] = (uint8_t)((all_ls[k + 4] & 0xF) | ((all_lm[k + 4] & 0xF) << 4));
        }
        u32 *o = (u32 *)blk;
        o[0] = (u32)dh | ((u32)dmh << 16);
#pragma unroll
        for (int k = 0; k < 3; k++) o[1 + k] = (u32)sc[4 * k] | ((u32)sc[4 * k + 1] << 8) | ((u32)sc[4 * k + 2] << 16) | ((u32)sc[4 * k + 3] << 24);
    }
    if constexpr (FIVE) {
        // qh[l] bit k = fifth bit of level l of sub-block k; this lane writes bytes 4 j .. 4 j + 3
        u32 word = 0;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            u32 byte = 0;
#pragma unroll
            for (int k = 0; k < 8; k++) byte |= ((hbs[k] >> (4 * j + b)) & 1u) << k;
            word |= byte << (8 * b);
        }
        *(u32 *)(blk + 16 + 4 * j) = word;
    }
    if ((j & 1) == 0) {
        u32 *q = (u32 *)(blk + (FIVE ? 48 : 16) + 32 * (j >> 1));
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = low[i] | (other[i] << 4);
    }
}

// quantize_row_q6_K_ref: thread = one 16-element group (make_qx_quants(16, 32, x, L, 1, NULL)), sixteen neighbouring lanes = one super-block
__global__ void __launch_bounds__(256) k_quantize_q6_K(const float *__restrict__ x, uint8_t *__restrict__ y, int64_t n_grp) {
    MI355_EXACT
    __shared__ uint8_t s_L[16][256];
    const int64_t grp = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool live = grp < n_grp;
    const int64_t g = live ? grp : n_grp - 1;
    const int ib = (int)(g & 15), sbl = threadIdx.x >> 4;
    float xv[16];
    {
        const f32x4 *p = (const f32x4 *)(x + g * 16);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const f32x4 v = p[i];
            xv[4 * i] = v[0]; xv[4 * i + 1] = v[1]; xv[4 * i + 2] = v[2]; xv[4 * i + 3] = v[3];
        }
    }
    constexpr int nmax = 32;
    int L[16];
    float scale;
    {
        float mx = 0, amax = 0;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float ax = fabsf(xv[i]);
            if (ax > amax) { amax = ax; mx = xv[i]; }
        }
        if (amax < 1e-15f) {
#pragma unroll
            for (int i = 0; i < 16; i++) L[i] = 0;
            scale = 0.f;
        } else {
            float iscale = -(float)nmax / mx;
            float sumlx = 0, suml2 = 0;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                int l = nearest_int(iscale * xv[i]);
                l = clampi(l, -nmax, nmax - 1);
                L[i] = l + nmax;
                const float wt = xv[i] * xv[i];
                sumlx += wt * xv[i] * (float)l;
                suml2 += wt * (float)l * (float)l;
            }
            scale = suml2 != 0.0f ? sumlx / suml2 : 0.0f;
            float best = scale * sumlx;
            for (int is = -9; is <= 9; is++) {
                if (is == 0) continue;
                iscale = -((float)nmax + 0.1f * (float)is) / mx;
                sumlx = suml2 = 0;
                int La[16];
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    int l = nearest_int(iscale * xv[i]);
                    l = clampi(l, -nmax, nmax - 1);
                    La[i] = l;
                    const float wt = xv[i] * xv[i];
                    sumlx += wt * xv[i] * (float)l;
                    suml2 += wt * (float)l * (float)l;
                }
                if (suml2 > 0 && sumlx * sumlx > best * suml2) {
#pragma unroll
                    for (int i = 0; i < 16; i++) L[i] = nmax + La[i];
                    scale = sumlx / suml2;
                    best = scale * sumlx;
                }
            }
        }
    }
    // the first group with the largest |scale| gives the super-block's scale
    const int lane = threadIdx.x & 63, base = lane & ~15;
    float max_abs = 0, max_scale = 0;
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const float sk = __shfl(scale, base + k, 64);
        const float ak = fabsf(sk);
        if (ak > max_abs) { max_abs = ak; max_scale = sk; }
    }
    const bool zero = max_abs < 1e-15f;
    unsigned short dh = 0;
    int sc8 = 0;
    if (!zero) {
        const float iscale = -128.f / max_scale;
        dh = float_to_half_bits(1 / iscale);
        const int q = nearest_int(iscale * scale);
        sc8 = q < 127 ? q : 127;
        sc8 = (int)(signed char)sc8;   // stored through int8_t
        const float d = half_bits_to_float(dh) * (float)sc8;
        if (d != 0.0f) {
#pragma unroll
            for (int i = 0; i < 16; i++) L[i] = clampi(nearest_int(xv[i] / d), -32, 31) + 32;
        }
    }
#pragma unroll
    for (int i = 0; i < 16; i++) s_L[sbl][16 * ib + i] = (uint8_t)(zero ? 0 : L[i]);
    __syncthreads();
    if (!live) return;
    uint8_t *blk = y + (g >> 4) * Q6_K_BYTES;
    const uint8_t *Ls = s_L[sbl];
    // ql bytes 8 ib .. + 7, qh bytes 4 ib .. + 3, scale ib; d by the first lane
#pragma unroll
    for (int t = 0; t < 8; t++) {
        const int b = 8 * ib + t, h = b >> 6, bb = b & 63, l = bb & 31, q = bb >> 5;   // q = 0: quarters 0 and 2, q = 1: quarters 1 and 3
        const uint8_t lo = Ls[128 * h + 32 * q + l] & 0xF, hi = Ls[128 * h + 32 * q + l + 64] & 0xF;
        blk[b] = zero ? 0 : (uint8_t)(lo | (hi << 4));
    }
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const int c = 4 * ib + t, h = c >> 5, l = c & 31;
        const uint8_t v = (uint8_t)((Ls[128 * h + l] >> 4) | ((Ls[128 * h + l + 32] >> 4) << 2) | ((Ls[128 * h + l + 64] >> 4) << 4) | ((Ls[128 * h + l + 96] >> 4) << 6));
        blk[128 + c] = zero ? 0 : v;
    }
    blk[192 + ib] = (uint8_t)(zero ? 0 : sc8);
    if (ib == 0) *(unsigned short *)(blk + 208) = dh;
}

// quantize_row_q4_0_ref / quantize_row_q8_0_ref: thread = one 32-element block
template <int TYPE>
__global__ void __launch_bounds__(256) k_quantize_q4_0_q8_0(const float *__restrict__ x, uint8_t *__restrict__ y, int64_t n_blk) {
    MI355_EXACT
    const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= n_blk) return;
    float xv[32];
    const f32x4 *p = (const f32x4 *)(x + b * 32);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const f32x4 v = p[i];
        xv[4 * i] = v[0]; xv[4 * i + 1] = v[1]; xv[4 * i + 2] = v[2]; xv[4 * i + 3] = v[3];
    }
    if constexpr (TYPE == MI355_Q4_0) {
        float amax = 0.0f, mx = 0.0f;
#pragma unroll
        for (int jj = 0; jj < 32; jj++) {
            if (amax < fabsf(xv[jj])) { amax = fabsf(xv[jj]); mx = xv[jj]; }
        }
        // d = max / -8 is exact as an eighth with the sign flipped.  Its half is formed from the eighth and the sign bit flipped in
        // the half's bits: a zero block keeps the reference's -0.0 this way (the compiler folds a conversion of a product into a
        // fused multiply-add with a +0.0 addend, which turns -0.0 into +0.0).
        const float e = mx * 0.125f;
        const float d = -e;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        unsigned short *o = (unsigned short *)(y + b * Q4_0_BYTES);
        o[0] = (unsigned short)(float_to_half_bits(e) ^ 0x8000u);
#pragma unroll
        for (int jj = 0; jj < 16; jj += 2) {
            u32 w2 = 0;
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const float x0 = xv[jj + t] * id, x1 = xv[16 + jj + t] * id;
                int q0 = (int)(signed char)(int)(x0 + 8.5f), q1 = (int)(signed char)(int)(x1 + 8.5f);
                q0 = q0 < 15 ? q0 : 15;
                q1 = q1 < 15 ? q1 : 15;
                w2 |= (u32)((q0 & 0xF) | ((q1 & 0xF) << 4)) << (8 * t);
            }
            o[1 + (jj >> 1)] = (unsigned short)w2;
        }
    } else {
        float amax = 0.0f;
#pragma unroll
        for (int jj = 0; jj < 32; jj++) amax = fmaxf(amax, fabsf(xv[jj]));
        const float d = amax / 127;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        unsigned short *o = (unsigned short *)(y + b * Q8_0_BYTES);
        o[0] = float_to_half_bits(d);
#pragma unroll
        for (int jj = 0; jj < 32; jj += 2) {
            const int q0 = (int)roundf(xv[jj] * id), q1 = (int)roundf(xv[jj + 1] * id);
            o[1 + (jj >> 1)] = (unsigned short)((q0 & 0xFF) | ((q1 & 0xFF) << 8));
        }
    }
}

// quantize_row_q4_1_ref / q5_0_ref / q5_1_ref (ggml/src/ggml-quants.c:68-103, 105-147, 149-192): thread = one 32-element block.
// Blocks are written in 16-bit pieces (Q5_0's 22-byte blocks are only 2-byte aligned).
template <int TYPE>
__global__ void __launch_bounds__(256) k_quantize_q4_1_q5(const float *__restrict__ x, uint8_t *__restrict__ y, int64_t n_blk) {
    MI355_EXACT
    constexpr bool MIN = TYPE != MI355_Q5_0, FIVE = TYPE != MI355_Q4_1;
    const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= n_blk) return;
    float xv[32];
    const f32x4 *p = (const f32x4 *)(x + b * 32);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const f32x4 v = p[i];
        xv[4 * i] = v[0]; xv[4 * i + 1] = v[1]; xv[4 * i + 2] = v[2]; xv[4 * i + 3] = v[3];
    }
    unsigned short *o = (unsigned short *)(y + b * (TYPE == MI355_Q4_1 ? Q4_1_BYTES : TYPE == MI355_Q5_0 ? Q5_0_BYTES : Q5_1_BYTES));
    float id, vmin = 0.0f;
    int at = 1;   // next 16-bit piece of the block
    if constexpr (MIN) {
        vmin = 3.402823466e+38f;
        float vmax = -3.402823466e+38f;
#pragma unroll
        for (int j = 0; j < 32; j++) {
            if (xv[j] < vmin) vmin = xv[j];
            if (xv[j] > vmax) vmax = xv[j];
        }
        const float d = (vmax - vmin) / (FIVE ? 31 : 15);
        id = d != 0.0f ? 1.0f / d : 0.0f;
        o[0] = float_to_half_bits(d);
        o[1] = float_to_half_bits(vmin);
        at = 2;
    } else {
        float amax = 0.0f, mx = 0.0f;
#pragma unroll
        for (int j = 0; j < 32; j++) {
            if (amax < fabsf(xv[j])) { amax = fabsf(xv[j]); mx = xv[j]; }
        }
        // d = max / -16: exact as a sixteenth with the sign flipped in the half's bits (a zero block keeps the reference's -0.0)
        const float e = mx * 0.0625f;
        const float d = -e;
        id = d != 0.0f ? 1.0f / d : 0.0f;
        o[0] = (unsigned short)(float_to_half_bits(e) ^ 0x8000u);
    }
    int lv[32];
#pragma unroll
    for (int j = 0; j < 32; j++) {
        if constexpr (TYPE == MI355_Q4_1) {
            const int q = (int)(signed char)(int)((xv[j] - vmin) * id + 0.5f);
            lv[j] = q < 15 ? q : 15;
        } else if constexpr (TYPE == MI355_Q5_0) {
            const int q = (int)(signed char)(int)(xv[j] * id + 16.5f);
            lv[j] = q < 31 ? q : 31;
        } else {
            lv[j] = (int)(unsigned char)(int)((xv[j] - vmin) * id + 0.5f);   // no clamp in the reference: bits above the fifth are dropped
        }
    }
    if constexpr (FIVE) {
        u32 h = 0;
#pragma unroll
        for (int j = 0; j < 32; j++) h |= (u32)((lv[j] >> 4) & 1) << j;
        o[at] = (unsigned short)(h & 0xFFFFu);
        o[at + 1] = (unsigned short)(h >> 16);
        at += 2;
    }
#pragma unroll
    for (int j = 0; j < 16; j += 2) {
        const u32 b0 = (u32)((lv[j] & 0xF) | ((lv[16 + j] & 0xF) << 4)), b1 = (u32)((lv[j + 1] & 0xF) | ((lv[17 + j] & 0xF) << 4));
        o[at + (j >> 1)] = (unsigned short)(b0 | (b1 << 8));
    }
}

// quantize_iq4_nl / quantize_iq4_xs without importance weights (ggml/src/ggml-quants.c:4684-4745) = quantize_row_iq4_nl_impl
// (:4573-4682) with ntry = 7: thread = one 32-element block; the eight threads of an IQ4_XS super-block are neighbouring lanes.
__device__ __forceinline__ int iq4nl_best_index(float x) {   // best_index_int8 (:4562-4571) on kvalues_iq4nl
    MI355_EXACT
    constexpr int8_t val[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
    if (x <= (float)val[0]) return 0;
    if (x >= (float)val[15]) return 15;
    int ml = 0, mu = 15;
    while (mu - ml > 1) {
        const int mav = (ml + mu) / 2;
        if (x < (float)val[mav]) mu = mav; else ml = mav;
    }
    return x - (float)val[mu - 1] < (float)val[mu] - x ? mu - 1 : mu;
}
__device__ __forceinline__ float iq4nl_value(int l) {
    constexpr int8_t val[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
    return (float)val[l];
}
template <bool XS>
__global__ void __launch_bounds__(256) k_quantize_iq4(const float *__restrict__ x, uint8_t *__restrict__ y, int64_t n_blk) {
    MI355_EXACT
    const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= n_blk) return;   // n_blk is a multiple of 8 for IQ4_XS: the lanes of a super-block leave together
    float xv[32];
    const f32x4 *p = (const f32x4 *)(x + b * 32);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const f32x4 v = p[i];
        xv[4 * i] = v[0]; xv[4 * i + 1] = v[1]; xv[4 * i + 2] = v[2]; xv[4 * i + 3] = v[3];
    }
    // the block's scale: first guess max / 127 with the sign that maps max onto -127, then 15 candidates, scored by the least-squares fit
    float amax = 0.0f, mx = 0.0f;
    for (int j = 0; j < 32; j++) {
        const float ax = fabsf(xv[j]);
        if (ax > amax) { amax = ax; mx = xv[j]; }
    }
    float scale = 0.0f;
    if (!(amax < 1e-15f)) {
        float d = -mx / -127.0f;
        float id = 1 / d;
        float sumqx = 0, sumq2 = 0;
        for (int j = 0; j < 32; j++) {
            const float q = iq4nl_value(iq4nl_best_index(id * xv[j]));
            const float w = xv[j] * xv[j];
            sumqx += w * q * xv[j];
            sumq2 += w * q * q;
        }
        d = sumqx / sumq2;
        float best = d * sumqx;
        for (int itry = -7; itry <= 7; itry++) {
            id = (float)(itry - 127) / mx;
            sumqx = sumq2 = 0;
            for (int j = 0; j < 32; j++) {
                const float q = iq4nl_value(iq4nl_best_index(id * xv[j]));
                const float w = xv[j] * xv[j];
                sumqx += w * q * xv[j];
                sumq2 += w * q * q;
            }
            if (sumq2 > 0 && sumqx * sumqx > best * sumq2) { d = sumqx / sumq2; best = d * sumqx; }
        }
        scale = d;
    }
    float id_levels;   // what the levels are chosen with
    u32 *qs;           // the block's 16 bytes of level pairs (4-byte aligned in both layouts... IQ4_NL: 2-byte, written as halves below)
    if constexpr (XS) {
        const int lane = threadIdx.x & 63, base = lane & ~7, ib = lane & 7;
        float max_scale = 0, amax_scale = 0;
        for (int i = 0; i < 8; i++) {
            const float si = __shfl(scale, base + i, 64);
            const float a = fabsf(si);
            if (a > amax_scale) { amax_scale = a; max_scale = si; }
        }
        const float d = -max_scale / 32;
        const float id = d != 0.0f ? 1 / d : 0.f;
        int l = clampi(nearest_int(id * scale), -32, 31);
        const float dl = d * (float)l;
        id_levels = dl != 0.0f ? 1 / dl : 0.f;
        l += 32;
        u32 sl = 0, sh = 0;
        for (int i = 0; i < 8; i++) {
            const int li = __shfl(l, base + i, 64);
            sl |= (u32)(li & 0xF) << (4 * i);
            sh |= (u32)(li >> 4) << (2 * i);
        }
        uint8_t *blk = y + (b >> 3) * IQ4_XS_BYTES;
        if (ib == 0) {
            ((u32 *)blk)[0] = (u32)float_to_half_bits(d) | (sh << 16);
            ((u32 *)blk)[1] = sl;
        }
        qs = (u32 *)(blk + 8 + 16 * ib);
    } else {
        id_levels = scale != 0.0f ? 1 / scale : 0.f;
        qs = nullptr;
    }
    u32 packed[4] = {0, 0, 0, 0};
    for (int j = 0; j < 16; j++) {
        const u32 lo = (u32)iq4nl_best_index(id_levels * xv[j]), hi = (u32)iq4nl_best_index(id_levels * xv[16 + j]);
        packed[j >> 2] |= (lo | (hi << 4)) << (8 * (j & 3));
    }
    if constexpr (XS) {
#pragma unroll
        for (int i = 0; i < 4; i++) qs[i] = packed[i];
    } else {
        unsigned short *o = (unsigned short *)(y + b * IQ4_NL_BYTES);   // 18-byte blocks: 2-byte aligned
        o[0] = float_to_half_bits(scale);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            o[1 + 2 * i] = (unsigned short)(packed[i] & 0xFFFFu);
            o[2 + 2 * i] = (unsigned short)(packed[i] >> 16);
        }
    }
}

}  // namespace

}  // namespace mi355

using namespace mi355;

extern "C" {

int mi355_quantize_weights_supported(int type) {
    return is_weight_type(type);   // every weight type the kernels read
}

int mi355_quantize_weights(void *stream, int type, const float *x, void *y, int64_t k, int64_t nrows) {
    MI355_REQUIRE(mi355_quantize_weights_supported(type), "quantize_weights: no device quantizer for type %d", type);
    MI355_REQUIRE(k > 0 && nrows > 0 && k % type_block_elems(type) == 0, "quantize_weights: k=%lld is not a multiple of the block size (nrows=%lld)", (long long)k,
                  (long long)nrows);
    MI355_REQUIRE(x != nullptr && y != nullptr && ((uintptr_t)x & 15) == 0 && ((uintptr_t)y & 3) == 0, "quantize_weights: x must be 16-byte, y 4-byte aligned");
    const int64_t n = k * nrows;   // rows are contiguous on both sides: the blocks of all rows form one sequence
    hipStream_t s = (hipStream_t)stream;
    if (type == MI355_Q4_K || type == MI355_Q5_K) {
        const int64_t n_sub = n / 32;
        MI355_REQUIRE((n_sub + 255) / 256 < 0x7fffffff, "quantize_weights: tensor too large for one launch");
        if (type == MI355_Q4_K) MI355_LAUNCH(k_quantize_q45_K<false>, dim3((unsigned)((n_sub + 255) / 256)), dim3(256), 0, s, x, (uint8_t *)y, n_sub);
        else MI355_LAUNCH(k_quantize_q45_K<true>, dim3((unsigned)((n_sub + 255) / 256)), dim3(256), 0, s, x, (uint8_t *)y, n_sub);
    } else if (type == MI355_Q6_K) {
        const int64_t n_grp = n / 16;
        MI355_REQUIRE((n_grp + 255) / 256 < 0x7fffffff, "quantize_weights: tensor too large for one launch");
        MI355_LAUNCH(k_quantize_q6_K, dim3((unsigned)((n_grp + 255) / 256)), dim3(256), 0, s, x, (uint8_t *)y, n_grp);
    } else {
        const int64_t n_blk = n / 32;
        MI355_REQUIRE((n_blk + 255) / 256 < 0x7fffffff, "quantize_weights: tensor too large for one launch");
        if (type == MI355_Q4_0) MI355_LAUNCH(k_quantize_q4_0_q8_0<MI355_Q4_0>, dim3((unsigned)((n_blk + 255) / 256)), dim3(256), 0, s, x, (uint8_t *)y, n_blk);
        else if (type == MI355_Q4_1) MI355_LAUNCH(k_quantize_q4_1_q5<MI355_Q4_1>, dim3((unsigned)((n_blk + 255) / 256)), dim3(256), 0, s, x, (uint8_t *)y, n_blk);
        else if (type == MI355_Q5_0) MI355_LAUNCH(k_quantize_q4_1_q5<MI355_Q5_0>, dim3((unsigned)((n_blk + 255) / 256)), dim3(256), 0, s, x, (uint8_t *)y, n_blk);
        else if (type == MI355_Q5_1) MI355_LAUNCH(k_quantize_q4_1_q5<MI355_Q5_1>, dim3((unsigned)((n_blk + 255) / 256)), dim3(256), 0, s, x, (uint8_t *)y, n_blk);
        else if (type == MI355_IQ4_NL) MI355_LAUNCH(k_quantize_iq4<false>, dim3((unsigned)((n_blk + 255) / 256)), dim3(256), 0, s, x, (uint8_t *)y, n_blk);
        else if (type == MI355_IQ4_XS) MI355_LAUNCH(k_quantize_iq4<true>, dim3((unsigned)((n_blk + 255) / 256)), dim3(256), 0, s, x, (uint8_t *)y, n_blk);
        else MI355_LAUNCH(k_quantize_q4_0_q8_0<MI355_Q8_0>, dim3((unsigned)((n_blk + 255) / 256)), dim3(256), 0, s, x, (uint8_t *)y, n_blk);
    }
    return launch_status("k_quantize_weights");
}

}  // extern "C"
