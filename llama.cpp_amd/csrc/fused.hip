// Fused forms of the glue sequences llama.cpp's graph emits between the matrix products.
// A decoded token is ~800 graph nodes whose useful work is a few microseconds each; what they
// cost is launches and HBM round trips of 16 KB vectors.  Each kernel here does the work of two
// to four consecutive nodes and, where the consumer is a quantized MUL_MAT, also emits the
// Q8_1 activation (same arithmetic as k_quantize_q8_1, i.e. quantize_row_q8_1_ref), so the
// separate quantization launch disappears:
//   RMS_NORM -> MUL(weight) [-> Q8_1 | Q8_K]     k_rms_norm_mul_quant
//   UNARY(SILU) -> MUL(up)  [-> Q8_1 | Q8_K]     k_swiglu_quant
// (Q8_K: the per-super-block form the K-quant tile GEMM reads, same arithmetic as k_quantize_q8k; a wave's 64 lanes hold
// exactly one 256-element super-block)
//   ROPE(q), ROPE(k), CPY(k -> cache), CPY(v -> cache)   k_rope_kv_store
#include "common.hpp"
#include "kv_blocks.hpp"
#include "moe.hpp"
#include "norm_quant.hpp"
#include "q8k.hpp"
#include "tiles.hpp"

namespace mi355 {

// one 256-thread group per row
template <int NV, int FMT>
__global__ void __launch_bounds__(256) k_rms_norm_mul_quant(const float *__restrict__ x, int64_t x_stride, const float *__restrict__ w,
                                                            float *__restrict__ y, int64_t y_stride, void *__restrict__ act, int64_t k,
                                                            int64_t nrows, float eps) {
    __shared__ float sh[4];
    const int64_t row = blockIdx.x;
    rms_norm_quant_row<NV, FMT, false>(x + row * x_stride, w, y ? y + row * y_stride : nullptr, act, row, k, nrows, eps, sh);
}

// The FFN norm of a mixture-of-experts layer for a few tokens, continued with the router (llm_build_moe_ffn, src/llama.cpp:438-468):
// logits[e] = W[e] . y for the row y the group has just normalised, then soft-max and the descending order.  A thread's pieces of y
// are the pieces k_mul_mat_f (glue.hip) gives thread t of its 256-thread group - elements 4 t + 1024 i - and the sums are formed in
// its order (the pieces in order, the wave, then the waves in order), so the logits hold the bits of that launch; the router's rows
// are requested before the norm's own loads are waited for.  NE8: experts in rounds of eight.
template <int NV>
__global__ void __launch_bounds__(256) k_rms_norm_mul_quant_router(const float *__restrict__ x, int64_t x_stride, const float *__restrict__ w,
                                                                   float *__restrict__ y, int64_t y_stride, void *__restrict__ act, int64_t k, int64_t nrows,
                                                                   float eps, const float *__restrict__ W, int64_t w_stride, float *__restrict__ logits,
                                                                   float *__restrict__ probs, int32_t *__restrict__ order, int n_expert) {
    __shared__ float sh[4];
    __shared__ float s_part[8][4];
    __shared__ float s_logit[64];
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // the first eight experts' rows: on their way before the norm waits for anything
    f32x4 wpre[NV][8];
#pragma unroll
    for (int it = 0; it < NV; it++) {
        const int64_t k0 = ((int64_t)it * 256 + tid) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            wpre[it][i] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (k0 < k && i < n_expert) wpre[it][i] = *(const f32x4 *)(W + (int64_t)i * w_stride + k0);
        }
    }
    f32x4 yv[NV];
    rms_norm_quant_row<NV, 0, false>(x + row * x_stride, w, y ? y + row * y_stride : nullptr, act, row, k, nrows, eps, sh, yv);
    for (int e0 = 0; e0 < n_expert; e0 += 8) {
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = 0.0f;
#pragma unroll
        for (int it = 0; it < NV; it++) {
            const int64_t k0 = ((int64_t)it * 256 + tid) * 4;
            if (k0 < k) {
                const f32x4 x0 = yv[it];
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    if (e0 + i < n_expert) {
                        const f32x4 w0 = e0 == 0 ? wpre[it][i] : *(const f32x4 *)(W + (int64_t)(e0 + i) * w_stride + k0);
                        acc[i] += w0[0] * x0[0] + w0[1] * x0[1] + w0[2] * x0[2] + w0[3] * x0[3];
                    }
                }
            }
        }
        __syncthreads();   // s_part of the previous round has been read
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float v = wave_sum(acc[i]);
            if (lane == 0) s_part[i][wave] = v;
        }
        __syncthreads();
        if (tid < 8 && e0 + tid < n_expert) {
            float t = 0.0f;
            for (int q = 0; q < 4; q++) t += s_part[tid][q];
            s_logit[e0 + tid] = t;
            logits[row * n_expert + e0 + tid] = t;
        }
    }
    __syncthreads();
    if (wave != 0) return;
    float p;
    const int rank = moe_route_lane(lane < n_expert ? s_logit[lane] : -INFINITY, lane, n_expert, p);
    if (lane < n_expert) {
        probs[row * n_expert + lane] = p;
        order[row * n_expert + rank] = lane;
    }
}

// h = silu(gate) * up, optional f32 output, optional Q8_1 output; one lane per 4 elements
template <int FMT>
__global__ void __launch_bounds__(256) k_swiglu_quant(const float *__restrict__ gate, const float *__restrict__ up, int64_t in_stride,
                                                      float *__restrict__ y, int64_t y_stride, void *__restrict__ act, int64_t k,
                                                      int64_t nrows) {
    const int64_t row = blockIdx.y;
    const int64_t e0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    const bool live = e0 < k;
    f32x4 o = {0.f, 0.f, 0.f, 0.f};
    if (live) {
        const f32x4 g = *(const f32x4 *)(gate + row * in_stride + e0);
        const f32x4 u = *(const f32x4 *)(up + row * in_stride + e0);
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = silu_fast(g[i]) * u[i];
        if (y) *(f32x4 *)(y + row * y_stride + e0) = o;
    }
    if (act) {
        int8_t *qplane = (int8_t *)act;
        if constexpr (FMT == 2) {
            if (live) q8k_quantize_wave_tiled(o, threadIdx.x & 63, (uint8_t *)act, k, nrows, row, e0 >> 8);   // whole wave: k is a multiple of 256
        } else if constexpr (FMT == 1) {
            if (live) {   // whole wave: k is a multiple of 256
                const int64_t nsb = k >> 8, sb = e0 >> 8;
                float *d8 = (float *)(qplane + q8k_d_offset(k, nrows));
                _Float16 *bs = (_Float16 *)(qplane + q8k_bs_offset(k, nrows));
                q8k_quantize_wave(o, threadIdx.x & 63, qplane + row * k + sb * QKK, d8 + row * nsb + sb, bs + (row * nsb + sb) * 16);
            }
        } else {
            quantize_block_lane(o, live, qplane, (act_ds *)(qplane + nrows * k), row, k, e0);
        }
    }
}

struct rope_kv_args {
    const float *q;         // [T][H][D] f32
    float *q_out;           // rotated q (may be q itself)
    const float *k;         // [T][HK][D] f32
    const float *v;         // [T][HK][D] f32
    uint8_t *kcache, *vcache;   // f16; element (cell, head, d) at cell*nb1 + head*nb2 + 2*d
                                // Q8_0 / Q4_0 (type_k / type_v): data of the tensor that owns the memory; nb1 = index of cell 0's first
                                // block within it, nb2 = its blocks per row in the device row layout (0: plain ggml blocks)
    int type_k, type_v;
    const int32_t *pos;     // [T] rope positions
    const int32_t *cells;   // [T] cache cell of each token
    const float *ff;        // rope frequency factors [n_dims/2] or null
    int64_t k_nb1, k_nb2, v_nb1, v_nb2;
    int T, H, HK, D, n_dims, mode;
    float theta_scale, freq_scale, ext_factor, attn_factor, corr0, corr1;
};

// rope_yarn as in k_rope (glue.hip) / ggml-cpu.c:9268-9306: the rotation of pair `pair` at position `pos`
__device__ __forceinline__ void rope_cos_sin(const rope_kv_args &a, int pos, int pair, float &c, float &s) {
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

// {cos, sin} of every (token, pair), for a launch that rotates the rows it has just formed (the Q/K/V launch of the wide-tile GEMM):
// the values k_rope_kv_store works out per pair, written once per batch and read by every layer's launch
__global__ void __launch_bounds__(64) k_rope_table(rope_kv_args a, float2 *__restrict__ cs) {
    const int t = blockIdx.x;
    const int pos = a.pos[t];
    for (int pair = threadIdx.x; 2 * pair < a.D; pair += 64) {
        float c = 1.0f, sn = 0.0f;
        if (2 * pair < a.n_dims) rope_cos_sin(a, pos, pair, c, sn);
        cs[(int64_t)t * (a.D / 2) + pair] = make_float2(c, sn);
    }
}

// One 256-thread group per token.  The rotation of a pair depends on the token's position and the pair only, so a wave works it
// out once per pair (lane = pair) and applies it to every head it is given: the four waves share the H query heads, HK key heads
// and HK value heads (plain f16 copies) between them, wave w taking slots w, w + 4, ...  Same roundings as k_rope: no contraction.
// QC: K and / or V go to a Q8_0 / Q4_0 cache (adjacent-pair mode, D a multiple of 32): a lane holds two adjacent elements, 16 lanes
// one block, quantized as quantize_row_q8_0_ref / quantize_row_q4_0_ref do.
template <bool QC>
__global__ void __launch_bounds__(256) k_rope_kv_store(rope_kv_args a) {
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int D = a.D, n_slots = a.H + 2 * a.HK;
    const bool neox = (a.mode & 2) != 0;
    const int pos = a.pos[t];
    const int64_t cell = a.cells[t];
    for (int pair = lane; 2 * pair < D; pair += 64) {
        const int i0 = 2 * pair;
        const bool rot = i0 < a.n_dims;
        const int ia = (rot && neox) ? pair : i0, ib = (rot && neox) ? pair + a.n_dims / 2 : i0 + 1;
        float c = 1.0f, sn = 0.0f;
        if (rot) rope_cos_sin(a, pos, pair, c, sn);
        // four of the wave's slots at a time: all loads first, so that their round trips overlap
        for (int h0 = wave; h0 < n_slots; h0 += 16) {
            float x0[4], x1[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int h = h0 + 4 * u;
                x0[u] = x1[u] = 0.0f;
                if (h >= n_slots) continue;
                const float *p = h < a.H ? a.q + ((int64_t)t * a.H + h) * D
                                 : h < a.H + a.HK ? a.k + ((int64_t)t * a.HK + (h - a.H)) * D : a.v + ((int64_t)t * a.HK + (h - a.H - a.HK)) * D;
                const bool is_v = h >= a.H + a.HK;
                x0[u] = p[is_v ? i0 : ia];
                x1[u] = p[is_v ? i0 + 1 : ib];
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int h = h0 + 4 * u;
                if (h >= n_slots) continue;
                float y0 = x0[u], y1 = x1[u];
                if (h < a.H + a.HK && rot) {
                    y0 = sub_rn(mul_rn(x0[u], c), mul_rn(x1[u], sn));
                    y1 = add_rn(mul_rn(x0[u], sn), mul_rn(x1[u], c));
                }
                if (h < a.H) {
                    float *o = a.q_out + ((int64_t)t * a.H + h) * D;
                    o[ia] = y0;
                    o[ib] = y1;
                } else if (QC && (h < a.H + a.HK ? a.type_k : a.type_v) != MI355_F16) {   // uniform over the wave
                    const bool is_k = h < a.H + a.HK;
                    const int type = is_k ? a.type_k : a.type_v;
                    const int head = is_k ? h - a.H : h - a.H - a.HK;
                    const kv_place pl = {0, is_k ? a.k_nb2 : a.v_nb2};
                    const int64_t g = (is_k ? a.k_nb1 : a.v_nb1) + (cell * a.HK + head) * (D >> 5) + (i0 >> 5);
                    uint8_t *base = is_k ? a.kcache : a.vcache;
                    int64_t lv, sc;
                    if (type == MI355_Q8_0) {
                        kv_block_offsets<MI355_Q8_0>(pl, g, lv, sc);
                        kv_store_q8_0_pair16(y0, y1, pair & 15, base, lv, sc);
                    } else {
                        kv_block_offsets<MI355_Q4_0>(pl, g, lv, sc);
                        kv_store_q4_0_pair16(y0, y1, pair & 15, base, lv, sc);
                    }
                } else if (h < a.H + a.HK) {
                    _Float16 *kc = (_Float16 *)(a.kcache + cell * a.k_nb1 + (int64_t)(h - a.H) * a.k_nb2);
                    kc[ia] = (_Float16)y0;
                    kc[ib] = (_Float16)y1;
                } else {
                    _Float16 *vc = (_Float16 *)(a.vcache + cell * a.v_nb1 + (int64_t)(h - a.H - a.HK) * a.v_nb2);
                    vc[i0] = (_Float16)y0;
                    vc[i0 + 1] = (_Float16)y1;
                }
            }
        }
    }
}

}  // namespace mi355

using namespace mi355;

extern "C" {

static int rms_norm_mul_quant(void *stream, const float *x, int64_t x_stride, const float *w, float *y, int64_t y_stride, void *act, int64_t k,
                              int64_t nrows, float eps, int fmt) {
    const bool q8k = fmt != 0;
    MI355_REQUIRE(k > 0 && k % 32 == 0 && k <= 16384, "rms_norm_mul_quant: k=%lld must be a multiple of 32 and at most 16384", (long long)k);
    MI355_REQUIRE(!q8k || k % QKK == 0, "rms_norm_mul_quant: k=%lld is not a multiple of 256", (long long)k);
    MI355_REQUIRE(nrows >= 0 && nrows < 0x7fffffff, "rms_norm_mul_quant: bad row count");
    MI355_REQUIRE(((uintptr_t)x & 15) == 0 && x_stride % 4 == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)y & 15) == 0 && y_stride % 4 == 0 &&
                  ((uintptr_t)act & 15) == 0, "rms_norm_mul_quant: operands must be 16-byte aligned");
    MI355_REQUIRE(y != nullptr || act != nullptr, "rms_norm_mul_quant: no output requested");
    if (nrows == 0) return MI355_OK;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)nrows), block(256);
#define MI355_LAUNCH_NORM(NV)                                                                                                        \
    do {                                                                                                                              \
        if (fmt == 2) MI355_LAUNCH((k_rms_norm_mul_quant<NV, 2>), grid, block, 0, s, x, x_stride, w, y, y_stride, act, k, nrows, eps);  \
        else if (fmt == 1) MI355_LAUNCH((k_rms_norm_mul_quant<NV, 1>), grid, block, 0, s, x, x_stride, w, y, y_stride, act, k, nrows, eps);  \
        else MI355_LAUNCH((k_rms_norm_mul_quant<NV, 0>), grid, block, 0, s, x, x_stride, w, y, y_stride, act, k, nrows, eps);     \
    } while (0)
    if (k <= 4096) MI355_LAUNCH_NORM(4);
    else if (k <= 8192) MI355_LAUNCH_NORM(8);
    else MI355_LAUNCH_NORM(16);
#undef MI355_LAUNCH_NORM
    return launch_status("k_rms_norm_mul_quant");
}

int mi355_rms_norm_mul_quant_router(void *stream, const float *x, int64_t x_stride, const float *w, float *y, int64_t y_stride, void *act, int64_t k,
                                    int64_t nrows, float eps, const float *W, int64_t w_stride, float *logits, float *probs, int32_t *order,
                                    int64_t n_expert) {
    MI355_REQUIRE(k > 0 && k % 32 == 0 && k <= 4096, "rms_norm_mul_quant_router: k=%lld must be a multiple of 32 and at most 4096", (long long)k);
    MI355_REQUIRE(nrows >= 0 && nrows <= 64, "rms_norm_mul_quant_router: a few rows (%lld given)", (long long)nrows);
    MI355_REQUIRE(n_expert >= 1 && n_expert <= 64 && w_stride >= k && w_stride % 4 == 0, "rms_norm_mul_quant_router: 1..64 experts, router rows of at least k");
    MI355_REQUIRE(((uintptr_t)x & 15) == 0 && x_stride % 4 == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)y & 15) == 0 && y_stride % 4 == 0 &&
                  ((uintptr_t)act & 15) == 0 && ((uintptr_t)W & 15) == 0, "rms_norm_mul_quant_router: operands must be 16-byte aligned");
    MI355_REQUIRE(W && logits && probs && order, "rms_norm_mul_quant_router: null operand");
    if (nrows == 0) return MI355_OK;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)nrows), block(256);
    if (k <= 1024) MI355_LAUNCH((k_rms_norm_mul_quant_router<1>), grid, block, 0, s, x, x_stride, w, y, y_stride, act, k, nrows, eps, W, w_stride, logits, probs, order, (int)n_expert);
    else if (k <= 2048) MI355_LAUNCH((k_rms_norm_mul_quant_router<2>), grid, block, 0, s, x, x_stride, w, y, y_stride, act, k, nrows, eps, W, w_stride, logits, probs, order, (int)n_expert);
    else MI355_LAUNCH((k_rms_norm_mul_quant_router<4>), grid, block, 0, s, x, x_stride, w, y, y_stride, act, k, nrows, eps, W, w_stride, logits, probs, order, (int)n_expert);
    return launch_status("k_rms_norm_mul_quant_router");
}

int mi355_rms_norm_mul_quant(void *stream, const float *x, int64_t x_stride, const float *w, float *y, int64_t y_stride, void *act,
                             int64_t k, int64_t nrows, float eps) {
    return rms_norm_mul_quant(stream, x, x_stride, w, y, y_stride, act, k, nrows, eps, 0);
}

int mi355_rms_norm_mul_quant_q8k(void *stream, const float *x, int64_t x_stride, const float *w, float *y, int64_t y_stride, void *act,
                                 int64_t k, int64_t nrows, float eps) {
    return rms_norm_mul_quant(stream, x, x_stride, w, y, y_stride, act, k, nrows, eps, 1);
}

int mi355_rms_norm_mul_quant_q8k_tiled(void *stream, const float *x, int64_t x_stride, const float *w, float *y, int64_t y_stride, void *act,
                                       int64_t k, int64_t nrows, float eps) {
    return rms_norm_mul_quant(stream, x, x_stride, w, y, y_stride, act, k, nrows, eps, 2);
}

static int swiglu_quant(void *stream, const float *gate, const float *up, int64_t in_stride, float *y, int64_t y_stride, void *act, int64_t k,
                        int64_t nrows, int fmt) {
    const bool q8k = fmt != 0;
    MI355_REQUIRE(k > 0 && k % 32 == 0, "swiglu_quant: k=%lld must be a multiple of 32", (long long)k);
    MI355_REQUIRE(!q8k || k % QKK == 0, "swiglu_quant: k=%lld is not a multiple of 256", (long long)k);
    MI355_REQUIRE(nrows >= 0 && nrows <= 65535, "swiglu_quant: bad row count");
    MI355_REQUIRE(((uintptr_t)gate & 15) == 0 && ((uintptr_t)up & 15) == 0 && in_stride % 4 == 0 && ((uintptr_t)y & 15) == 0 && y_stride % 4 == 0 &&
                  ((uintptr_t)act & 15) == 0, "swiglu_quant: operands must be 16-byte aligned");
    MI355_REQUIRE(y != nullptr || act != nullptr, "swiglu_quant: no output requested");
    if (nrows == 0) return MI355_OK;
    const dim3 grid((unsigned)((k + 1023) / 1024), (unsigned)nrows), block(256);
    if (fmt == 2) MI355_LAUNCH(k_swiglu_quant<2>, grid, block, 0, (hipStream_t)stream, gate, up, in_stride, y, y_stride, act, k, nrows);
    else if (fmt == 1) MI355_LAUNCH(k_swiglu_quant<1>, grid, block, 0, (hipStream_t)stream, gate, up, in_stride, y, y_stride, act, k, nrows);
    else MI355_LAUNCH(k_swiglu_quant<0>, grid, block, 0, (hipStream_t)stream, gate, up, in_stride, y, y_stride, act, k, nrows);
    return launch_status("k_swiglu_quant");
}

int mi355_swiglu_quant(void *stream, const float *gate, const float *up, int64_t in_stride, float *y, int64_t y_stride, void *act,
                       int64_t k, int64_t nrows) {
    return swiglu_quant(stream, gate, up, in_stride, y, y_stride, act, k, nrows, 0);
}

int mi355_swiglu_quant_q8k(void *stream, const float *gate, const float *up, int64_t in_stride, float *y, int64_t y_stride, void *act,
                           int64_t k, int64_t nrows) {
    return swiglu_quant(stream, gate, up, in_stride, y, y_stride, act, k, nrows, 1);
}

int mi355_swiglu_quant_q8k_tiled(void *stream, const float *gate, const float *up, int64_t in_stride, float *y, int64_t y_stride, void *act,
                                 int64_t k, int64_t nrows) {
    return swiglu_quant(stream, gate, up, in_stride, y, y_stride, act, k, nrows, 2);
}

static void rope_freq_args(rope_kv_args &a, int n_dims, int n_ctx_orig, float freq_base, float freq_scale, float ext_factor, float attn_factor,
                           float beta_fast, float beta_slow) {
    a.theta_scale = powf(freq_base, -2.0f / n_dims);
    a.freq_scale = freq_scale; a.ext_factor = ext_factor; a.attn_factor = attn_factor;
    const float pi = 3.14159265358979323846f;   // ggml_rope_yarn_corr_dims, ggml/src/ggml.c:3695-3707
    const float c0 = floorf(n_dims * logf(n_ctx_orig / (beta_fast * 2 * pi)) / (2 * logf(freq_base)));
    const float c1 = ceilf(n_dims * logf(n_ctx_orig / (beta_slow * 2 * pi)) / (2 * logf(freq_base)));
    a.corr0 = c0 > 0 ? c0 : 0;
    a.corr1 = c1 < n_dims - 1 ? c1 : (float)(n_dims - 1);
}

int mi355_rope_table(void *stream, const int32_t *pos, const float *freq_factors, float *table, int64_t T, int64_t D, int n_dims, int n_ctx_orig,
                     float freq_base, float freq_scale, float ext_factor, float attn_factor, float beta_fast, float beta_slow) {
    MI355_REQUIRE(T > 0 && T <= 65535 && D > 0 && D % 2 == 0 && D <= 2048, "rope_table: bad shape");
    MI355_REQUIRE(n_dims > 0 && n_dims % 2 == 0 && n_dims <= D, "rope_table: bad n_dims");
    MI355_REQUIRE(pos != nullptr && table != nullptr && ((uintptr_t)table & 7) == 0, "rope_table: null or misaligned operand");
    rope_kv_args a = {};
    a.pos = pos; a.ff = freq_factors;
    a.T = (int)T; a.D = (int)D; a.n_dims = n_dims;
    rope_freq_args(a, n_dims, n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow);
    MI355_LAUNCH(k_rope_table, dim3((unsigned)T), dim3(64), 0, (hipStream_t)stream, a, (float2 *)table);
    return launch_status("k_rope_table");
}

static int rope_kv_store_impl(void *stream, float *q, const float *k, const float *v, int type_k, void *kcache, int64_t k_a, int64_t k_b, int type_v,
                              void *vcache, int64_t v_a, int64_t v_b, const int32_t *pos, const int32_t *cells, const float *freq_factors, int64_t T,
                              int64_t H, int64_t HK, int64_t D, int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale,
                              float ext_factor, float attn_factor, float beta_fast, float beta_slow) {
    MI355_REQUIRE(T > 0 && T <= 65535 && H > 0 && HK > 0 && D > 0 && D % 2 == 0 && D <= 2048, "rope_kv_store: bad shape");
    MI355_REQUIRE(mode == 0 || mode == 2, "rope_kv_store: mode %d not supported (0 = adjacent pairs, 2 = NeoX)", mode);
    MI355_REQUIRE(n_dims > 0 && n_dims % 2 == 0 && n_dims <= D, "rope_kv_store: bad n_dims");
    const bool qc = type_k != MI355_F16 || type_v != MI355_F16;
    for (int t : {type_k, type_v}) MI355_REQUIRE(t == MI355_F16 || t == MI355_Q8_0 || t == MI355_Q4_0, "rope_kv_store: cache type %d (f16, Q8_0, Q4_0 are served)", t);
    MI355_REQUIRE(!qc || (mode == 0 && D % 32 == 0 && k_a >= 0 && k_b >= 0 && v_a >= 0 && v_b >= 0 && (((uintptr_t)kcache | (uintptr_t)vcache) & 1) == 0),
                  "rope_kv_store: a quantized cache takes the adjacent-pair mode and head sizes that are multiples of 32");
    rope_kv_args a;
    a.q = q; a.q_out = q; a.k = k; a.v = v; a.kcache = (uint8_t *)kcache; a.vcache = (uint8_t *)vcache;
    a.type_k = type_k; a.type_v = type_v;
    a.pos = pos; a.cells = cells; a.ff = freq_factors;
    a.k_nb1 = k_a; a.k_nb2 = k_b; a.v_nb1 = v_a; a.v_nb2 = v_b;
    a.T = (int)T; a.H = (int)H; a.HK = (int)HK; a.D = (int)D; a.n_dims = n_dims; a.mode = mode;
    rope_freq_args(a, n_dims, n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow);
    if (qc) MI355_LAUNCH(k_rope_kv_store<true>, dim3((unsigned)T), dim3(256), 0, (hipStream_t)stream, a);
    else MI355_LAUNCH(k_rope_kv_store<false>, dim3((unsigned)T), dim3(256), 0, (hipStream_t)stream, a);
    return launch_status("k_rope_kv_store");
}

int mi355_rope_kv_store(void *stream, float *q, const float *k, const float *v, void *kcache, void *vcache, const int32_t *pos,
                        const int32_t *cells, const float *freq_factors, int64_t T, int64_t H, int64_t HK, int64_t D, size_t k_nb1,
                        size_t k_nb2, size_t v_nb1, size_t v_nb2, int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale,
                        float ext_factor, float attn_factor, float beta_fast, float beta_slow) {
    return rope_kv_store_impl(stream, q, k, v, MI355_F16, kcache, (int64_t)k_nb1, (int64_t)k_nb2, MI355_F16, vcache, (int64_t)v_nb1, (int64_t)v_nb2, pos, cells,
                              freq_factors, T, H, HK, D, n_dims, mode, n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow);
}

int mi355_rope_kv_store_typed(void *stream, float *q, const float *k, const float *v, int type_k, void *kcache, int64_t k_a, int64_t k_b, int type_v,
                              void *vcache, int64_t v_a, int64_t v_b, const int32_t *pos, const int32_t *cells, const float *freq_factors, int64_t T,
                              int64_t H, int64_t HK, int64_t D, int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale,
                              float ext_factor, float attn_factor, float beta_fast, float beta_slow) {
    return rope_kv_store_impl(stream, q, k, v, type_k, kcache, k_a, k_b, type_v, vcache, v_a, v_b, pos, cells, freq_factors, T, H, HK, D, n_dims, mode,
                              n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow);
}

}  // extern "C"
