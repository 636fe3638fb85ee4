// The small operators that keep a llama graph resident on the device between the matrix
// kernels: RMS_NORM, ADD/SUB/MUL/DIV with broadcast, unary activations, SCALE, CPY/CONT/DUP,
// GET_ROWS, SOFT_MAX, ROPE, SUM_ROWS, ARGSORT and the dense (f32/f16 weight) MUL_MAT used by
// MoE routers.  All honour ggml's byte strides (nb[]); none assumes contiguity unless it
// checks for it.  These are HBM-trivial next to the weight stream, so they are kept simple:
// one thread per element or one wave/group per row, 16-byte accesses where rows allow.
#include "common.hpp"
#include "qdot.hpp"

#include <float.h>

namespace mi355 {

struct tens {
    uint8_t *data;
    int64_t ne[4];
    int64_t nb[4];
};

static tens to_tens(const mi355_tensor *t) {
    tens r;
    r.data = (uint8_t *)t->data;
    for (int i = 0; i < 4; i++) {
        r.ne[i] = t->ne[i];
        r.nb[i] = (int64_t)t->nb[i];
    }
    return r;
}
static int64_t nelements(const mi355_tensor *t) { return t->ne[0] * t->ne[1] * t->ne[2] * t->ne[3]; }
static int64_t nrows(const mi355_tensor *t) { return t->ne[1] * t->ne[2] * t->ne[3]; }
static bool same_shape(const mi355_tensor *a, const mi355_tensor *b) {
    return a->ne[0] == b->ne[0] && a->ne[1] == b->ne[1] && a->ne[2] == b->ne[2] && a->ne[3] == b->ne[3];
}
static size_t elem_size(int type) { return type == MI355_F16 ? 2 : 4; }
static bool rows_dense(const mi355_tensor *t) { return t->nb[0] == elem_size(t->type); }

__device__ __forceinline__ float block_sum(float v, float *sh) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if (nw == 1) return v;
    __syncthreads();
    if (lane == 0) sh[wave] = v;
    __syncthreads();
    float t = 0.0f;
    for (int i = 0; i < nw; i++) t += sh[i];
    return t;
}
__device__ __forceinline__ float block_max(float v, float *sh) {
    v = wave_max(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if (nw == 1) return v;
    __syncthreads();
    if (lane == 0) sh[wave] = v;
    __syncthreads();
    float t = sh[0];
    for (int i = 1; i < nw; i++) t = fmaxf(t, sh[i]);
    return t;
}

__device__ __forceinline__ const uint8_t *row_ptr(const tens &t, int64_t row) {
    const int64_t i1 = row % t.ne[1], i2 = (row / t.ne[1]) % t.ne[2], i3 = row / (t.ne[1] * t.ne[2]);
    return t.data + i1 * t.nb[1] + i2 * t.nb[2] + i3 * t.nb[3];
}

// ---------------------------------------------------------------- RMS_NORM
// ggml_compute_forward_rms_norm_f32, ggml-cpu.c:7015-7061: y = x / sqrt(mean(x^2) + eps)
__global__ void k_rms_norm(tens src, tens dst, float eps) {
    __shared__ float sh[16];
    const int64_t row = blockIdx.x;
    const float *x = (const float *)row_ptr(src, row);
    float *y = (float *)row_ptr(dst, row);
    const int64_t n = src.ne[0];
    float ss = 0.0f;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) ss += x[i] * x[i];
    ss = block_sum(ss, sh);
    const float scale = 1.0f / sqrtf(ss / (float)n + eps);
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) y[i] = x[i] * scale;
}

// ---------------------------------------------------------------- binary ops with broadcast
// ggml_compute_forward_{add,sub,mul,div}_f32, ggml-cpu.c:4067-4140, 5142-5305
template <int OP>
__device__ __forceinline__ float bin_apply(float a, float b) {
    if constexpr (OP == 0) return a + b;
    else if constexpr (OP == 1) return a - b;
    else if constexpr (OP == 2) return a * b;
    else return a / b;
}
template <int OP>
__global__ void k_bin_bcast(tens a, tens b, tens d, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t i0 = i % d.ne[0], i1 = (i / d.ne[0]) % d.ne[1], i2 = (i / (d.ne[0] * d.ne[1])) % d.ne[2],
                  i3 = i / (d.ne[0] * d.ne[1] * d.ne[2]);
    const float va = *(const float *)(a.data + i0 * a.nb[0] + i1 * a.nb[1] + i2 * a.nb[2] + i3 * a.nb[3]);
    const float vb = *(const float *)(b.data + (i0 % b.ne[0]) * b.nb[0] + (i1 % b.ne[1]) * b.nb[1] +
                                      (i2 % b.ne[2]) * b.nb[2] + (i3 % b.ne[3]) * b.nb[3]);
    *(float *)(d.data + i0 * d.nb[0] + i1 * d.nb[1] + i2 * d.nb[2] + i3 * d.nb[3]) = bin_apply<OP>(va, vb);
}

// ---------------------------------------------------------------- unary + scale
// op ids: ggml_unary_op, ggml/include/ggml.h:530-547; math as in ggml-cpu.c:1790-1870
__device__ __forceinline__ float unary_apply(int op, float x, float p) {
    switch (op) {
        case 0: return fabsf(x);                                  // ABS
        case 1: return x > 0.0f ? 1.0f : (x < 0.0f ? -1.0f : 0.0f);   // SGN
        case 2: return -x;                                        // NEG
        case 3: return x > 0.0f ? 1.0f : 0.0f;                    // STEP
        case 4: return tanhf(x);                                  // TANH
        case 5: return x > 0.0f ? x : expm1f(x);                  // ELU
        case 6: return x > 0.0f ? x : 0.0f;                       // RELU
        case 7: return 1.0f / (1.0f + expf(-x));                  // SIGMOID
        case 8: return 0.5f * x * (1.0f + tanhf(0.79788456080286535587989211986876f * x * (1.0f + 0.044715f * x * x)));   // GELU
        case 9: return x * (1.0f / (1.0f + expf(-1.702f * x)));   // GELU_QUICK
        case 10: return x / (1.0f + expf(-x));                    // SILU
        case 11: return x * fminf(1.0f, fmaxf(0.0f, (x + 3.0f) / 6.0f));   // HARDSWISH
        case 12: return fminf(1.0f, fmaxf(0.0f, (x + 3.0f) / 6.0f));       // HARDSIGMOID
        case 13: return expf(x);                                  // EXP
        case 100: return x * p;                                   // SCALE
        default: return x;
    }
}
__global__ void k_unary(int op, tens a, tens d, int64_t n, float p) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t i0 = i % d.ne[0], i1 = (i / d.ne[0]) % d.ne[1], i2 = (i / (d.ne[0] * d.ne[1])) % d.ne[2],
                  i3 = i / (d.ne[0] * d.ne[1] * d.ne[2]);
    const float v = *(const float *)(a.data + i0 * a.nb[0] + i1 * a.nb[1] + i2 * a.nb[2] + i3 * a.nb[3]);
    *(float *)(d.data + i0 * d.nb[0] + i1 * d.nb[1] + i2 * d.nb[2] + i3 * d.nb[3]) = unary_apply(op, v, p);
}

// ---------------------------------------------------------------- CPY / CONT / DUP
// ggml_compute_forward_dup, ggml-cpu.c:3519-3830: element i of src (in src's logical order)
// goes to element i of dst (in dst's logical order); shapes may differ.
template <typename TS, typename TD>
__global__ void k_cpy(tens a, tens d, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t a0 = i % a.ne[0], a1 = (i / a.ne[0]) % a.ne[1], a2 = (i / (a.ne[0] * a.ne[1])) % a.ne[2],
                  a3 = i / (a.ne[0] * a.ne[1] * a.ne[2]);
    const int64_t d0 = i % d.ne[0], d1 = (i / d.ne[0]) % d.ne[1], d2 = (i / (d.ne[0] * d.ne[1])) % d.ne[2],
                  d3 = i / (d.ne[0] * d.ne[1] * d.ne[2]);
    const TS v = *(const TS *)(a.data + a0 * a.nb[0] + a1 * a.nb[1] + a2 * a.nb[2] + a3 * a.nb[3]);
    *(TD *)(d.data + d0 * d.nb[0] + d1 * d.nb[1] + d2 * d.nb[2] + d3 * d.nb[3]) = (TD)v;
}

// ---------------------------------------------------------------- GET_ROWS
// ggml_compute_forward_get_rows_{f32,f16}, ggml-cpu.c:8464-8590
template <typename TS>
__global__ void k_get_rows(tens src, tens ids, tens dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t i0 = i % dst.ne[0], i1 = (i / dst.ne[0]) % dst.ne[1], i2 = (i / (dst.ne[0] * dst.ne[1])) % dst.ne[2],
                  i3 = i / (dst.ne[0] * dst.ne[1] * dst.ne[2]);
    const int32_t r = *(const int32_t *)(ids.data + i1 * ids.nb[0] + i2 * ids.nb[1] + i3 * ids.nb[2]);
    const TS v = *(const TS *)(src.data + i0 * src.nb[0] + (int64_t)r * src.nb[1] + i2 * src.nb[2] + i3 * src.nb[3]);
    *(float *)(dst.data + i0 * dst.nb[0] + i1 * dst.nb[1] + i2 * dst.nb[2] + i3 * dst.nb[3]) = (float)v;
}

// Rows of a quantized matrix (device row layout) as f32: dequantize_row_q4_0 / _q8_0 / _q4_K / _q6_K (ggml/src/ggml-quants.c:255-273,
// 349-363, 1280-1302, 1690-1719) of the selected rows, ggml_compute_forward_get_rows_q (ggml-cpu.c:8464-8506).  One thread per element.
template <int TYPE>
__global__ void k_get_rows_q(tens src, tens ids, tens dst, int64_t n, row_layout L) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t i0 = i % dst.ne[0], i1 = (i / dst.ne[0]) % dst.ne[1], i2 = (i / (dst.ne[0] * dst.ne[1])) % dst.ne[2],
                  i3 = i / (dst.ne[0] * dst.ne[1] * dst.ne[2]);
    const int32_t r = *(const int32_t *)(ids.data + i1 * ids.nb[0] + i2 * ids.nb[1] + i3 * ids.nb[2]);
    const uint8_t *row = src.data + (int64_t)r * src.nb[1] + i2 * src.nb[2] + i3 * src.nb[3];
    *(float *)(dst.data + i0 * dst.nb[0] + i1 * dst.nb[1] + i2 * dst.nb[2] + i3 * dst.nb[3]) = weight_value<TYPE>(row, L, i0);
}

// ---------------------------------------------------------------- scatter rows (KV-cache store)
// dst[:, rows[i1], i2] = convert(src[:, i1, i2]).  The KV-cache write of llm_build_kv_store
// (src/llama.cpp:157-199) is a CPY into a view of the cache at row kv_head; here the target row
// comes from device memory so a captured launch sequence stays valid as the cache fills.
template <typename TD>
__global__ void k_set_rows(tens src, const int32_t *__restrict__ rows, tens dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t i0 = i % src.ne[0], i1 = (i / src.ne[0]) % src.ne[1], i2 = i / (src.ne[0] * src.ne[1]);
    const float v = *(const float *)(src.data + i0 * src.nb[0] + i1 * src.nb[1] + i2 * src.nb[2]);
    *(TD *)(dst.data + i0 * dst.nb[0] + (int64_t)rows[i1] * dst.nb[1] + i2 * dst.nb[2]) = (TD)v;
}

// ---------------------------------------------------------------- SOFT_MAX
// ggml_compute_forward_soft_max_f32, ggml-cpu.c:8959-9055.  mask row = row % ne1, contiguous.
template <typename TM>
__global__ void k_soft_max(tens src, const TM *__restrict__ mask, tens dst, float scale, float max_bias, float m0,
                           float m1, unsigned n_head_log2) {
    __shared__ float sh[16];
    const int64_t row = blockIdx.x;
    const float *x = (const float *)row_ptr(src, row);
    float *y = (float *)row_ptr(dst, row);
    const int64_t n = src.ne[0];
    const TM *mrow = mask ? mask + (row % src.ne[1]) * n : nullptr;
    float slope = 1.0f;
    if (max_bias > 0.0f) {
        const unsigned h = (unsigned)((row / src.ne[1]) % src.ne[2]);
        slope = h < n_head_log2 ? powf(m0, (float)(h + 1)) : powf(m1, (float)(2 * (h - n_head_log2) + 1));
    }
    float mx = -INFINITY;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = x[i] * scale + (mrow ? slope * (float)mrow[i] : 0.0f);
        mx = fmaxf(mx, v);
    }
    mx = block_max(mx, sh);
    float sum = 0.0f;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = x[i] * scale + (mrow ? slope * (float)mrow[i] : 0.0f);
        const float e = expf(v - mx);
        y[i] = e;
        sum += e;
    }
    sum = block_sum(sum, sh);
    const float inv = 1.0f / sum;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) y[i] *= inv;
}

// ---------------------------------------------------------------- ROPE
// ggml_compute_forward_rope_f32 + rope_yarn, ggml-cpu.c:9268-9306, 9366-9549.
// theta = pos * theta_scale^(i0/2) in closed form (the host walks it multiplicatively).
struct rope_params {
    int n_dims, mode;
    float theta_scale, freq_scale, ext_factor, attn_factor, corr0, corr1;
};
// T: float, or _Float16 (the rotation of an f16 K cache in place when the context is shifted, llama_kv_cache K-shift graph:
// values are widened, rotated in f32 and rounded back, ggml_compute_forward_rope_f16, ggml-cpu.c:9530-9700)
template <typename T>
__global__ void k_rope(tens src, const int32_t *__restrict__ pos, const float *__restrict__ ff, tens dst, rope_params p) {
    const int64_t row = blockIdx.x;   // over ne1*ne2*ne3
    const int64_t i2 = (row / src.ne[1]) % src.ne[2];
    const T *x = (const T *)row_ptr(src, row);
    T *y = (T *)row_ptr(dst, row);
    const int64_t ne0 = src.ne[0];
    const bool neox = (p.mode & 2) != 0;
    for (int64_t pair = threadIdx.x; pair < ne0 / 2; pair += blockDim.x) {
        const int64_t i0 = 2 * pair;
        if (i0 >= p.n_dims) {   // pass-through tail
            y[i0] = x[i0];
            y[i0 + 1] = x[i0 + 1];
            continue;
        }
        const float theta_extrap = (float)pos[i2] * powf(p.theta_scale, (float)pair) / (ff ? ff[pair] : 1.0f);
        const float theta_interp = p.freq_scale * theta_extrap;
        float theta = theta_interp, mscale = p.attn_factor;
        if (p.ext_factor != 0.0f) {
            const float yv = ((float)pair - p.corr0) / fmaxf(0.001f, p.corr1 - p.corr0);
            const float ramp = (1.0f - fminf(1.0f, fmaxf(0.0f, yv))) * p.ext_factor;
            theta = theta_interp * (1.0f - ramp) + theta_extrap * ramp;
            mscale *= 1.0f + 0.1f * logf(1.0f / p.freq_scale);
        }
        const float c = cosf(theta) * mscale, s = sinf(theta) * mscale;
        const int64_t ia = neox ? pair : i0, ib = neox ? pair + p.n_dims / 2 : i0 + 1;
        const float x0 = (float)x[ia], x1 = (float)x[ib];
        // separately rounded products: the fused rope + KV-store kernel rotates with the same four roundings
        y[ia] = (T)sub_rn(mul_rn(x0, c), mul_rn(x1, s));
        y[ib] = (T)add_rn(mul_rn(x0, s), mul_rn(x1, c));
    }
}

// ---------------------------------------------------------------- SUM_ROWS
__global__ void k_sum_rows(tens src, tens dst) {
    __shared__ float sh[16];
    const int64_t row = blockIdx.x;
    const float *x = (const float *)row_ptr(src, row);
    float s = 0.0f;
    for (int64_t i = threadIdx.x; i < src.ne[0]; i += blockDim.x) s += x[i];
    s = block_sum(s, sh);
    if (threadIdx.x == 0) *(float *)row_ptr(dst, row) = s;
}

// ---------------------------------------------------------------- ARGSORT
// ggml_compute_forward_argsort_f32, ggml-cpu.c:10857: bitonic network over the row padded to a
// power of two in LDS; padding sorts last.
__global__ void k_argsort(tens src, tens dst, int order, int npad) {
    extern __shared__ int sidx[];
    const int64_t row = blockIdx.x;
    const float *x = (const float *)row_ptr(src, row);
    int32_t *out = (int32_t *)row_ptr(dst, row);
    const int n = (int)src.ne[0];
    for (int i = threadIdx.x; i < npad; i += blockDim.x) sidx[i] = i;
    __syncthreads();
    for (int k = 2; k <= npad; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = threadIdx.x; i < npad; i += blockDim.x) {
                const int ixj = i ^ j;
                if (ixj > i) {
                    const int ia = sidx[i], ib = sidx[ixj];
                    const bool up = (i & k) == 0;
                    // "a should come after b" in the requested order; padding (>= n) always goes last
                    bool a_after_b;
                    if (ia >= n) a_after_b = ib < n;
                    else if (ib >= n) a_after_b = false;
                    else a_after_b = order == 0 ? x[ia] > x[ib] : x[ia] < x[ib];
                    bool b_after_a;
                    if (ib >= n) b_after_a = ia < n;
                    else if (ia >= n) b_after_a = false;
                    else b_after_a = order == 0 ? x[ib] > x[ia] : x[ib] < x[ia];
                    if (up ? a_after_b : b_after_a) {
                        sidx[i] = ib;
                        sidx[ixj] = ia;
                    }
                }
            }
            __syncthreads();
        }
    }
    for (int i = threadIdx.x; i < n; i += blockDim.x) out[i] = sidx[i];
}

// ---------------------------------------------------------------- dense MUL_MAT (f32 / f16 weights)
// dst[i3][i2][b][n] = sum_k W[i3/r3][i2/r2][n][k] * x[i3][i2][b][k]; one 256-thread group per output element.
// VEC: both rows are dense, 16-byte aligned and K is a multiple of 4 (f32) / 8 (f16), so a lane loads 16 bytes at a time.
template <typename TW, bool VEC>
__global__ void __launch_bounds__(256) k_mul_mat_f(tens w, tens x, tens d) {
    __shared__ float sh[16];
    const int64_t n = blockIdx.x, b = blockIdx.y;
    const int64_t i23 = blockIdx.z, i2 = i23 % d.ne[2], i3 = i23 / d.ne[2];
    const int64_t r2 = x.ne[2] / w.ne[2], r3 = x.ne[3] / w.ne[3];
    const uint8_t *wp = w.data + n * w.nb[1] + (i2 / r2) * w.nb[2] + (i3 / r3) * w.nb[3];
    const uint8_t *xp = x.data + b * x.nb[1] + i2 * x.nb[2] + i3 * x.nb[3];
    const int64_t K = w.ne[0];
    float acc = 0.0f;
    if constexpr (VEC) {
        constexpr int PER = 16 / sizeof(TW);   // weight elements per 16-byte load
#pragma unroll 4
        for (int64_t k = (int64_t)threadIdx.x * PER; k < K; k += 256 * PER) {
            const f32x4 x0 = *(const f32x4 *)(xp + k * 4);
            if constexpr (sizeof(TW) == 4) {
                const f32x4 w0 = *(const f32x4 *)(wp + k * 4);
                acc += w0[0] * x0[0] + w0[1] * x0[1] + w0[2] * x0[2] + w0[3] * x0[3];
            } else {
                const f32x4 x1 = *(const f32x4 *)(xp + k * 4 + 16);
                const f16x8 w0 = *(const f16x8 *)(wp + k * 2);
                acc += (float)w0[0] * x0[0] + (float)w0[1] * x0[1] + (float)w0[2] * x0[2] + (float)w0[3] * x0[3] +
                       (float)w0[4] * x1[0] + (float)w0[5] * x1[1] + (float)w0[6] * x1[2] + (float)w0[7] * x1[3];
            }
        }
    } else {
#pragma unroll 4
        for (int64_t k = threadIdx.x; k < K; k += 256) acc += (float)*(const TW *)(wp + k * w.nb[0]) * *(const float *)(xp + k * x.nb[0]);
    }
    acc = block_sum(acc, sh);
    if (threadIdx.x == 0) *(float *)(d.data + n * d.nb[0] + b * d.nb[1] + i2 * d.nb[2] + i3 * d.nb[3]) = acc;
}

static unsigned grid1d(int64_t n, int bs) { return (unsigned)((n + bs - 1) / bs); }
static int row_threads(int64_t n) { return n >= 1024 ? 256 : (n >= 256 ? 128 : 64); }

}  // namespace mi355

using namespace mi355;

extern "C" {

int mi355_rms_norm(void *stream, const mi355_tensor *src, const mi355_tensor *dst, float eps) {
    MI355_REQUIRE(src->type == MI355_F32 && dst->type == MI355_F32, "rms_norm: f32 only");
    MI355_REQUIRE(same_shape(src, dst) && rows_dense(src) && rows_dense(dst), "rms_norm: shapes differ or rows are strided");
    const int64_t nr = nrows(src);
    if (nr == 0 || src->ne[0] == 0) return MI355_OK;
    MI355_REQUIRE(nr < 0x7fffffff, "rms_norm: too many rows");
    // Rows of a contiguous tensor go through the kernel that the fused norm+weight+quantization launch uses, so that a
    // graph run node for node and the same graph run fused sum the squares in the same order and agree bit for bit.
    const int64_t n = src->ne[0];
    auto packed = [n](const mi355_tensor *t) {
        return t->nb[1] == n * 4 && t->nb[2] == t->nb[1] * t->ne[1] && t->nb[3] == t->nb[2] * t->ne[2] && ((uintptr_t)t->data & 15) == 0;
    };
    if (n % 32 == 0 && n <= 16384 && packed(src) && packed(dst))
        return mi355_rms_norm_mul_quant(stream, (const float *)src->data, n, nullptr, (float *)dst->data, n, nullptr, n, nr, eps);
    MI355_LAUNCH(k_rms_norm, dim3((unsigned)nr), dim3(row_threads(src->ne[0])), 0, (hipStream_t)stream, to_tens(src), to_tens(dst), eps);
    return launch_status("k_rms_norm");
}

int mi355_bin_bcast(void *stream, int op, const mi355_tensor *src0, const mi355_tensor *src1, const mi355_tensor *dst) {
    MI355_REQUIRE(src0->type == MI355_F32 && src1->type == MI355_F32 && dst->type == MI355_F32, "bin_bcast: f32 only");
    MI355_REQUIRE(op >= 0 && op <= 3, "bin_bcast: unknown op %d", op);
    MI355_REQUIRE(same_shape(src0, dst), "bin_bcast: src0 and dst shapes differ");
    for (int i = 0; i < 4; i++) MI355_REQUIRE(src1->ne[i] > 0 && dst->ne[i] % src1->ne[i] == 0, "bin_bcast: src1 does not broadcast over dst");
    const int64_t n = nelements(dst);
    if (n == 0) return MI355_OK;
    const dim3 grid(grid1d(n, 256)), block(256);
    hipStream_t s = (hipStream_t)stream;
    const tens a = to_tens(src0), b = to_tens(src1), d = to_tens(dst);
    switch (op) {
        case 0: MI355_LAUNCH(k_bin_bcast<0>, grid, block, 0, s, a, b, d, n); break;
        case 1: MI355_LAUNCH(k_bin_bcast<1>, grid, block, 0, s, a, b, d, n); break;
        case 2: MI355_LAUNCH(k_bin_bcast<2>, grid, block, 0, s, a, b, d, n); break;
        default: MI355_LAUNCH(k_bin_bcast<3>, grid, block, 0, s, a, b, d, n); break;
    }
    return launch_status("k_bin_bcast");
}

static int unary_launch(void *stream, int op, const mi355_tensor *src, const mi355_tensor *dst, float p) {
    MI355_REQUIRE(src->type == MI355_F32 && dst->type == MI355_F32, "unary: f32 only");
    MI355_REQUIRE(same_shape(src, dst), "unary: shapes differ");
    const int64_t n = nelements(dst);
    if (n == 0) return MI355_OK;
    MI355_LAUNCH(k_unary, dim3(grid1d(n, 256)), dim3(256), 0, (hipStream_t)stream, op, to_tens(src), to_tens(dst), n, p);
    return launch_status("k_unary");
}

int mi355_unary(void *stream, int op, const mi355_tensor *src, const mi355_tensor *dst) {
    MI355_REQUIRE(op >= 0 && op <= 13, "unary: unsupported op %d", op);
    return unary_launch(stream, op, src, dst, 0.0f);
}

int mi355_scale(void *stream, const mi355_tensor *src, const mi355_tensor *dst, float s) {
    return unary_launch(stream, 100, src, dst, s);
}

int mi355_cpy(void *stream, const mi355_tensor *src, const mi355_tensor *dst) {
    const int64_t n = nelements(src);
    MI355_REQUIRE(n == nelements(dst), "cpy: element counts differ");
    if (n == 0) return MI355_OK;
    const dim3 grid(grid1d(n, 256)), block(256);
    hipStream_t s = (hipStream_t)stream;
    const tens a = to_tens(src), d = to_tens(dst);
    const int st = src->type, dt = dst->type;
    if (st == MI355_F32 && dt == MI355_F32) MI355_LAUNCH((k_cpy<float, float>), grid, block, 0, s, a, d, n);
    else if (st == MI355_F32 && dt == MI355_F16) MI355_LAUNCH((k_cpy<float, _Float16>), grid, block, 0, s, a, d, n);
    else if (st == MI355_F16 && dt == MI355_F16) MI355_LAUNCH((k_cpy<_Float16, _Float16>), grid, block, 0, s, a, d, n);
    else if (st == MI355_F16 && dt == MI355_F32) MI355_LAUNCH((k_cpy<_Float16, float>), grid, block, 0, s, a, d, n);
    else if (st == MI355_I32 && dt == MI355_I32) MI355_LAUNCH((k_cpy<int32_t, int32_t>), grid, block, 0, s, a, d, n);
    else {
        set_error("cpy: type pair %d -> %d not supported", st, dt);
        return MI355_ERR_ARG;
    }
    return launch_status("k_cpy");
}

int mi355_get_rows(void *stream, const mi355_tensor *src, const mi355_tensor *ids, const mi355_tensor *dst) {
    MI355_REQUIRE((src->type == MI355_F32 || src->type == MI355_F16 || is_weight_type(src->type)) && ids->type == MI355_I32 && dst->type == MI355_F32,
                  "get_rows: src f32/f16/quantized, ids i32, dst f32 only");
    MI355_REQUIRE(dst->ne[0] == src->ne[0] && dst->ne[1] == ids->ne[0] && dst->ne[2] == ids->ne[1] && dst->ne[3] == ids->ne[2],
                  "get_rows: dst shape does not match ids");
    const int64_t n = nelements(dst);
    if (n == 0) return MI355_OK;
    const dim3 grid(grid1d(n, 256)), block(256);
    if (is_weight_type(src->type)) {
        const int64_t K = src->ne[0];
        MI355_REQUIRE(K % type_block_elems(src->type) == 0, "get_rows: row length %lld is not a multiple of the block size", (long long)K);
        const row_layout L = make_row_layout(src->type, K);
        MI355_REQUIRE((int64_t)src->nb[1] == L.row_bytes, "get_rows: quantized rows must be whole and contiguous");
        hipStream_t s = (hipStream_t)stream;
#define MI355_GET_ROWS_LAUNCH(TY) MI355_LAUNCH(k_get_rows_q<TY>, grid, block, 0, s, to_tens(src), to_tens(ids), to_tens(dst), n, L);
        MI355_WEIGHT_TYPE_SWITCH(src->type, MI355_GET_ROWS_LAUNCH)
#undef MI355_GET_ROWS_LAUNCH
        return launch_status("k_get_rows_q");
    }
    if (src->type == MI355_F32) MI355_LAUNCH(k_get_rows<float>, grid, block, 0, (hipStream_t)stream, to_tens(src), to_tens(ids), to_tens(dst), n);
    else MI355_LAUNCH(k_get_rows<_Float16>, grid, block, 0, (hipStream_t)stream, to_tens(src), to_tens(ids), to_tens(dst), n);
    return launch_status("k_get_rows");
}

int mi355_set_rows(void *stream, const mi355_tensor *src, const int32_t *rows, const mi355_tensor *dst) {
    MI355_REQUIRE(src->type == MI355_F32 && (dst->type == MI355_F32 || dst->type == MI355_F16), "set_rows: f32 -> f32/f16 only");
    MI355_REQUIRE(src->ne[0] == dst->ne[0] && src->ne[2] == dst->ne[2] && src->ne[3] == 1 && dst->ne[3] == 1, "set_rows: shapes do not match");
    const int64_t n = nelements(src);
    if (n == 0) return MI355_OK;
    const dim3 grid(grid1d(n, 256)), block(256);
    if (dst->type == MI355_F16) MI355_LAUNCH(k_set_rows<_Float16>, grid, block, 0, (hipStream_t)stream, to_tens(src), rows, to_tens(dst), n);
    else MI355_LAUNCH(k_set_rows<float>, grid, block, 0, (hipStream_t)stream, to_tens(src), rows, to_tens(dst), n);
    return launch_status("k_set_rows");
}

int mi355_soft_max(void *stream, const mi355_tensor *src, const mi355_tensor *mask, const mi355_tensor *dst, float scale,
                   float max_bias) {
    MI355_REQUIRE(src->type == MI355_F32 && dst->type == MI355_F32, "soft_max: f32 only");
    MI355_REQUIRE(same_shape(src, dst) && rows_dense(src) && rows_dense(dst), "soft_max: shapes differ or rows are strided");
    if (mask) {
        MI355_REQUIRE(mask->type == MI355_F32 || mask->type == MI355_F16, "soft_max: mask must be f32 or f16");
        MI355_REQUIRE(mask->ne[0] == src->ne[0] && mask->ne[1] >= src->ne[1] && mask->nb[0] == elem_size(mask->type) &&
                      mask->nb[1] == mask->ne[0] * elem_size(mask->type), "soft_max: mask must be contiguous rows of ne0");
    }
    const int64_t nr = nrows(src);
    if (nr == 0 || src->ne[0] == 0) return MI355_OK;
    MI355_REQUIRE(nr < 0x7fffffff, "soft_max: too many rows");
    unsigned n2 = 1;
    while (n2 * 2 <= (unsigned)src->ne[2]) n2 *= 2;
    const float m0 = powf(2.0f, -(max_bias) / n2), m1 = powf(2.0f, -(max_bias / 2.0f) / n2);
    const dim3 grid((unsigned)nr), block(row_threads(src->ne[0]));
    hipStream_t s = (hipStream_t)stream;
    if (mask && mask->type == MI355_F16)
        MI355_LAUNCH(k_soft_max<_Float16>, grid, block, 0, s, to_tens(src), (const _Float16 *)mask->data, to_tens(dst), scale, max_bias, m0, m1, n2);
    else
        MI355_LAUNCH(k_soft_max<float>, grid, block, 0, s, to_tens(src), (const float *)(mask ? mask->data : nullptr), to_tens(dst), scale, max_bias, m0, m1, n2);
    return launch_status("k_soft_max");
}

int mi355_rope(void *stream, const mi355_tensor *src, const int32_t *pos, const float *freq_factors,
               const mi355_tensor *dst, int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale,
               float ext_factor, float attn_factor, float beta_fast, float beta_slow) {
    MI355_REQUIRE((src->type == MI355_F32 || src->type == MI355_F16) && dst->type == src->type, "rope: f32 -> f32 or f16 -> f16 only");
    MI355_REQUIRE(same_shape(src, dst) && rows_dense(src) && rows_dense(dst), "rope: shapes differ or rows are strided");
    MI355_REQUIRE(mode == 0 || mode == 2, "rope: mode %d not supported (0 = adjacent pairs, 2 = NeoX)", mode);
    MI355_REQUIRE(n_dims > 0 && n_dims % 2 == 0 && n_dims <= src->ne[0] && src->ne[0] % 2 == 0, "rope: bad n_dims");
    const int64_t nr = nrows(src);
    if (nr == 0) return MI355_OK;
    MI355_REQUIRE(nr < 0x7fffffff, "rope: too many rows");
    rope_params p;
    p.n_dims = n_dims;
    p.mode = mode;
    p.theta_scale = powf(freq_base, -2.0f / n_dims);
    p.freq_scale = freq_scale;
    p.ext_factor = ext_factor;
    p.attn_factor = attn_factor;
    // ggml_rope_yarn_corr_dims, ggml/src/ggml.c:3695-3707
    const float pi = 3.14159265358979323846f;
    const float c0 = floorf(n_dims * logf(n_ctx_orig / (beta_fast * 2 * pi)) / (2 * logf(freq_base)));
    const float c1 = ceilf(n_dims * logf(n_ctx_orig / (beta_slow * 2 * pi)) / (2 * logf(freq_base)));
    p.corr0 = c0 > 0 ? c0 : 0;
    p.corr1 = c1 < n_dims - 1 ? c1 : (float)(n_dims - 1);
    if (src->type == MI355_F32) MI355_LAUNCH(k_rope<float>, dim3((unsigned)nr), dim3(64), 0, (hipStream_t)stream, to_tens(src), pos, freq_factors, to_tens(dst), p);
    else MI355_LAUNCH(k_rope<_Float16>, dim3((unsigned)nr), dim3(64), 0, (hipStream_t)stream, to_tens(src), pos, freq_factors, to_tens(dst), p);
    return launch_status("k_rope");
}

int mi355_sum_rows(void *stream, const mi355_tensor *src, const mi355_tensor *dst) {
    MI355_REQUIRE(src->type == MI355_F32 && dst->type == MI355_F32, "sum_rows: f32 only");
    MI355_REQUIRE(dst->ne[0] == 1 && dst->ne[1] == src->ne[1] && dst->ne[2] == src->ne[2] && dst->ne[3] == src->ne[3] && rows_dense(src),
                  "sum_rows: bad dst shape or strided rows");
    const int64_t nr = nrows(src);
    if (nr == 0) return MI355_OK;
    MI355_REQUIRE(nr < 0x7fffffff, "sum_rows: too many rows");
    MI355_LAUNCH(k_sum_rows, dim3((unsigned)nr), dim3(row_threads(src->ne[0])), 0, (hipStream_t)stream, to_tens(src), to_tens(dst));
    return launch_status("k_sum_rows");
}

int mi355_argsort(void *stream, const mi355_tensor *src, const mi355_tensor *dst, int order) {
    MI355_REQUIRE(src->type == MI355_F32 && dst->type == MI355_I32, "argsort: f32 -> i32 only");
    MI355_REQUIRE(same_shape(src, dst) && rows_dense(src) && rows_dense(dst), "argsort: shapes differ or rows are strided");
    MI355_REQUIRE(src->ne[0] >= 1 && src->ne[0] <= 1024, "argsort: row length %lld out of range (1..1024)", (long long)src->ne[0]);
    MI355_REQUIRE(order == 0 || order == 1, "argsort: order must be 0 or 1");
    const int64_t nr = nrows(src);
    if (nr == 0) return MI355_OK;
    MI355_REQUIRE(nr < 0x7fffffff, "argsort: too many rows");
    int npad = 1;
    while (npad < src->ne[0]) npad *= 2;
    const int threads = npad < 64 ? 64 : (npad > 256 ? 256 : npad);
    MI355_LAUNCH(k_argsort, dim3((unsigned)nr), dim3(threads), npad * sizeof(int), (hipStream_t)stream, to_tens(src), to_tens(dst), order, npad);
    return launch_status("k_argsort");
}

int mi355_mul_mat_f(void *stream, const mi355_tensor *src0, const mi355_tensor *src1, const mi355_tensor *dst) {
    MI355_REQUIRE((src0->type == MI355_F32 || src0->type == MI355_F16) && src1->type == MI355_F32 && dst->type == MI355_F32,
                  "mul_mat_f: src0 f32/f16, src1 f32, dst f32 only");
    MI355_REQUIRE(src0->ne[0] == src1->ne[0] && dst->ne[0] == src0->ne[1] && dst->ne[1] == src1->ne[1] && dst->ne[2] == src1->ne[2] && dst->ne[3] == src1->ne[3],
                  "mul_mat_f: shapes do not match");
    MI355_REQUIRE(src0->ne[2] > 0 && src0->ne[3] > 0 && src1->ne[2] % src0->ne[2] == 0 && src1->ne[3] % src0->ne[3] == 0, "mul_mat_f: src0 does not broadcast over src1");
    if (nelements(dst) == 0) return MI355_OK;
    MI355_REQUIRE(dst->ne[1] <= 65535 && dst->ne[2] * dst->ne[3] <= 65535, "mul_mat_f: batch too large for one launch");
    const dim3 grid((unsigned)dst->ne[0], (unsigned)dst->ne[1], (unsigned)(dst->ne[2] * dst->ne[3]));
    const int64_t wsz = src0->type == MI355_F32 ? 4 : 2;
    auto rows16 = [](const mi355_tensor *t, int64_t esz) {
        return t->nb[0] == (size_t)esz && ((uintptr_t)t->data & 15) == 0 && t->nb[1] % 16 == 0 && t->nb[2] % 16 == 0 && t->nb[3] % 16 == 0;
    };
    const bool vec = src0->ne[0] % (16 / wsz) == 0 && rows16(src0, wsz) && rows16(src1, 4);
    const dim3 block(256);
    hipStream_t s = (hipStream_t)stream;
    if (src0->type == MI355_F32) {
        if (vec) MI355_LAUNCH((k_mul_mat_f<float, true>), grid, block, 0, s, to_tens(src0), to_tens(src1), to_tens(dst));
        else MI355_LAUNCH((k_mul_mat_f<float, false>), grid, block, 0, s, to_tens(src0), to_tens(src1), to_tens(dst));
    } else {
        if (vec) MI355_LAUNCH((k_mul_mat_f<_Float16, true>), grid, block, 0, s, to_tens(src0), to_tens(src1), to_tens(dst));
        else MI355_LAUNCH((k_mul_mat_f<_Float16, false>), grid, block, 0, s, to_tens(src0), to_tens(src1), to_tens(dst));
    }
    return launch_status("k_mul_mat_f");
}

}  // extern "C"
