// On-device activation quantization to Q8_1 and the weight-row layout permutation.
#include "common.hpp"
#include "qdot.hpp"

#include <atomic>
#include <stdarg.h>
#include <string.h>

namespace mi355 {

static thread_local char g_err[512] = "";
static std::atomic<uint64_t> g_launches{0};

void count_launch() { g_launches.fetch_add(1, std::memory_order_relaxed); }
uint64_t launches_so_far() { return g_launches.load(std::memory_order_relaxed); }

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

// ---------------------------------------------------------------------------------------
// quantize_row_q8_1_ref, ggml/src/ggml-quants.c:220-253, bit for bit:
//   d = amax / 127 ; id = d ? 1/d : 0 ; q = roundf(x * id) ; y.d = fp16(d) ; y.s = fp16(sum(q) * d)
// Eight lanes share one 32-element block (one float4 each); a 256-thread group covers
// 1024 consecutive elements of one row.  Division and roundf are the IEEE-correct ones
// (no fast-math), so the levels agree with the host for every input.
//
// STD = true : writes block_q8_1 (36 B: fp16 d, fp16 s, 32 x int8)
// STD = false: writes the split layout of mi355_quantize_act (int8 plane + {float d; int sum})
// ---------------------------------------------------------------------------------------
template <bool STD>
__global__ void __launch_bounds__(256) k_quantize_q8_1(const float *__restrict__ x, void *__restrict__ y, int64_t k,
                                                       int64_t nrows, int64_t x_stride) {
    const int64_t row = blockIdx.y;
    const int64_t e0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;   // first of this lane's 4 elements
    const bool live = e0 < k;                                           // k % 32 == 0 so a block is all-live or all-dead
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (live) v = *(const f32x4 *)(x + row * x_stride + e0);

    const float amax = lanes_max<8>(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));

    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    int q[4];
    int sum = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        q[i] = (int)roundf(v[i] * id);
        sum += q[i];
    }
    sum = lanes_sum_i<8>(sum);

    if (!live) return;
    const u32 packed = (u32)(q[0] & 0xFF) | ((u32)(q[1] & 0xFF) << 8) | ((u32)(q[2] & 0xFF) << 16) | ((u32)(q[3] & 0xFF) << 24);
    const int64_t blk = e0 >> 5;
    const int sub = (int)((e0 >> 2) & 7);
    const int64_t nblk = k >> 5;
    if constexpr (STD) {
        uint8_t *b = (uint8_t *)y + (row * nblk + blk) * Q8_1_BYTES;
        *(u32 *)(b + 4 + 4 * sub) = packed;   // 36-byte blocks keep 4-byte alignment
        if (sub == 0) {
            const u32 ds = (u32)float_to_half_bits(d) | ((u32)float_to_half_bits((float)sum * d) << 16);
            *(u32 *)b = ds;
        }
    } else {
        int8_t *qplane = (int8_t *)y;
        act_ds *ds = (act_ds *)(qplane + nrows * k);
        *(u32 *)(qplane + row * k + e0) = packed;
        if (sub == 0) {
            act_ds o;
            o.d = half_bits_to_float(float_to_half_bits(d));
            o.sum = sum;
            ds[row * nblk + blk] = o;
        }
    }
}

// ---------------------------------------------------------------------------------------
// Weight-row layout permutation (byte granular, so any [offset, offset+size) range works).
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ int64_t dev_offset_in_row(int type, int64_t nb, int64_t w) {
    switch (type) {
        case MI355_Q4_0: case MI355_IQ4_NL: {
            const int64_t b = w / Q4_0_BYTES, o = w % Q4_0_BYTES;
            return o < 2 ? nb * 16 + b * 2 + o : b * 16 + (o - 2);
        }
        case MI355_Q4_1: {   // d, m, 16 nibble bytes
            const int64_t b = w / Q4_1_BYTES, o = w % Q4_1_BYTES;
            return o < 4 ? nb * 16 + b * 4 + o : b * 16 + (o - 4);
        }
        case MI355_Q5_0: {   // d, 4 bytes of fifth bits, 16 nibble bytes
            const int64_t b = w / Q5_0_BYTES, o = w % Q5_0_BYTES;
            if (o < 2) return nb * 20 + b * 2 + o;
            return o < 6 ? nb * 16 + b * 4 + (o - 2) : b * 16 + (o - 6);
        }
        case MI355_Q5_1: {   // d, m, 4 bytes of fifth bits, 16 nibble bytes
            const int64_t b = w / Q5_1_BYTES, o = w % Q5_1_BYTES;
            if (o < 4) return nb * 20 + b * 4 + o;
            return o < 8 ? nb * 16 + b * 4 + (o - 4) : b * 16 + (o - 8);
        }
        case MI355_IQ4_XS: {   // d, scales_h, scales_l[4], 128 nibble bytes
            const int64_t b = w / IQ4_XS_BYTES, o = w % IQ4_XS_BYTES;
            return o < 8 ? nb * 128 + b * 8 + o : b * 128 + (o - 8);
        }
        case MI355_Q8_0: {
            const int64_t b = w / Q8_0_BYTES, o = w % Q8_0_BYTES;
            return o < 2 ? nb * 32 + b * 2 + o : b * 32 + (o - 2);
        }
        case MI355_Q6_K: {
            const int64_t b = w / Q6_K_BYTES, o = w % Q6_K_BYTES;
            if (o < 128) return b * 128 + o;
            if (o < 192) return nb * 128 + b * 64 + (o - 128);
            if (o < 208) return nb * 192 + b * 16 + (o - 192);
            return nb * 208 + b * 2 + (o - 208);
        }
        default: return w;
    }
}

template <bool SCATTER>
__global__ void __launch_bounds__(256) k_weights_permute(int type, const uint8_t *__restrict__ src,
                                                         uint8_t *__restrict__ dst, int64_t nb, int64_t row_bytes,
                                                         size_t offset, size_t size) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= size) return;
    const size_t pos = offset + i;
    const int64_t row = (int64_t)(pos / (size_t)row_bytes);
    const int64_t w = (int64_t)(pos % (size_t)row_bytes);
    const size_t dpos = (size_t)row * (size_t)row_bytes + (size_t)dev_offset_in_row(type, nb, w);
    if constexpr (SCATTER) dst[dpos] = src[i];
    else dst[i] = src[dpos];
}

static int weights_permute(bool scatter, void *stream, int type, const void *src, void *dst, int64_t k, int64_t nrows,
                           size_t offset, size_t size) {
    MI355_REQUIRE(is_weight_type(type), "weights layout: unsupported type %d", type);
    MI355_REQUIRE(k > 0 && k % type_block_elems(type) == 0, "weights layout: k=%lld not a multiple of the block size", (long long)k);
    const int64_t nb = k / type_block_elems(type);
    const int64_t row_bytes = nb * type_block_bytes(type);
    MI355_REQUIRE(offset + size <= (size_t)row_bytes * (size_t)nrows, "weights layout: range exceeds tensor");
    if (size == 0) return MI355_OK;
    hipStream_t s = (hipStream_t)stream;
    if (type == MI355_Q4_K || type == MI355_Q5_K) {   // identity layout
        const void *from = scatter ? src : (const void *)((const uint8_t *)src + offset);
        void *to = scatter ? (void *)((uint8_t *)dst + offset) : dst;
        MI355_CHECK_HIP(hipMemcpyAsync(to, from, size, hipMemcpyDeviceToDevice, s));
        return MI355_OK;
    }
    const size_t nblocks = (size + 255) / 256;
    MI355_REQUIRE(nblocks < 0x7fffffffull, "weights layout: range too large for one launch");
    if (scatter)
        MI355_LAUNCH(k_weights_permute<true>, dim3((unsigned)nblocks), dim3(256), 0, s, type, (const uint8_t *)src,
                           (uint8_t *)dst, nb, row_bytes, offset, size);
    else
        MI355_LAUNCH(k_weights_permute<false>, dim3((unsigned)nblocks), dim3(256), 0, s, type, (const uint8_t *)src,
                           (uint8_t *)dst, nb, row_bytes, offset, size);
    return launch_status("k_weights_permute");
}

}  // namespace mi355

using namespace mi355;

extern "C" {

int mi355_abi_version(void) { return 1; }

const char *mi355_last_error(void) { return g_err; }
uint64_t mi355_launch_count(void) { return launches_so_far(); }

int mi355_device_supported(int device) {
    hipDeviceProp_t prop;
    MI355_CHECK_HIP(hipGetDeviceProperties(&prop, device));
    return strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 0;
}

int mi355_weights_scatter(void *stream, int type, const void *raw, void *dev, int64_t k, int64_t nrows, size_t offset,
                          size_t size) {
    return weights_permute(true, stream, type, raw, dev, k, nrows, offset, size);
}

int mi355_weights_gather(void *stream, int type, const void *dev, void *raw, int64_t k, int64_t nrows, size_t offset,
                         size_t size) {
    return weights_permute(false, stream, type, dev, raw, k, nrows, offset, size);
}

size_t mi355_act_bytes(int64_t k, int64_t nrows) {
    if (k <= 0 || nrows <= 0) return 0;
    return (size_t)nrows * (size_t)k + (size_t)nrows * (size_t)(k / QK) * sizeof(act_ds);
}

static int quantize_launch(bool std_layout, void *stream, const float *x, void *y, int64_t k, int64_t nrows,
                           int64_t x_stride) {
    MI355_REQUIRE(k > 0 && k % QK == 0, "quantize_q8_1: k=%lld is not a multiple of 32", (long long)k);
    MI355_REQUIRE(nrows >= 0 && nrows <= 65535, "quantize_q8_1: nrows=%lld out of range", (long long)nrows);
    MI355_REQUIRE(x_stride >= k && x_stride % 4 == 0 && ((uintptr_t)x & 15) == 0, "quantize_q8_1: x must be 16-byte aligned with a row stride that is a multiple of 4 floats");
    if (nrows == 0) return MI355_OK;
    const dim3 grid((unsigned)((k + 1023) / 1024), (unsigned)nrows);
    if (std_layout)
        MI355_LAUNCH(k_quantize_q8_1<true>, grid, dim3(256), 0, (hipStream_t)stream, x, y, k, nrows, x_stride);
    else
        MI355_LAUNCH(k_quantize_q8_1<false>, grid, dim3(256), 0, (hipStream_t)stream, x, y, k, nrows, x_stride);
    return launch_status("k_quantize_q8_1");
}

int mi355_quantize_q8_1(void *stream, const float *x, void *y, int64_t k, int64_t nrows, int64_t x_stride) {
    return quantize_launch(true, stream, x, y, k, nrows, x_stride);
}

int mi355_quantize_act(void *stream, const float *x, void *act, int64_t k, int64_t nrows, int64_t x_stride) {
    MI355_REQUIRE(((uintptr_t)act & 15) == 0, "quantize_act: workspace must be 16-byte aligned");
    return quantize_launch(false, stream, x, act, k, nrows, x_stride);
}

}  // extern "C"
