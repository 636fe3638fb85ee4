// MUL_MAT host entry: quantize activations on the device, then dispatch to the GEMV (few activation rows), the
// weight-streaming matrix-core kernel (up to 32 rows) or the int8-MFMA tile kernels.  Also the byte-load fallback for
// weight rows that are not 16-byte aligned.
#include "common.hpp"
#include "qdot.hpp"

#include <atomic>

namespace mi355 {

// one wave per (row, activation row); any K that is a multiple of the block size
template <int TYPE>
__global__ void __launch_bounds__(64) k_gemv_unaligned(const uint8_t *__restrict__ W, const int8_t *__restrict__ aq,
                                                       const act_ds *__restrict__ ads, float *__restrict__ dst,
                                                       const float *__restrict__ residual, int64_t N, int64_t K,
                                                       int64_t dst_stride, row_layout L) {
    const int64_t row = blockIdx.x, col = blockIdx.y;
    const uint8_t *wrow = W + row * L.row_bytes;
    const int8_t *q = aq + col * K;
    const act_ds *ds = ads + col * (K >> 5);
    float acc = 0.0f;
    for (int64_t e = threadIdx.x; e < K; e += 64) acc += weight_value<TYPE>(wrow, L, e) * (ds[e >> 5].d * (float)q[e]);
    acc = wave_sum(acc);
    if (threadIdx.x == 0) {
        const int64_t o = col * dst_stride + row;
        dst[o] = residual ? acc + residual[o] : acc;
    }
}

// act: split layout holding B quantized rows of K
int gemv_unaligned(hipStream_t s, int type, const void *W, const void *act, float *dst, const float *residual, int64_t N,
                   int64_t K, int64_t B, int64_t dst_stride) {
    const row_layout L = make_row_layout(type, K);
    const int8_t *aq = (const int8_t *)act;
    const act_ds *ads = (const act_ds *)(aq + B * K);
    MI355_REQUIRE(B <= 65535, "mul_mat: batch %lld too large for the unaligned path", (long long)B);
    const dim3 grid((unsigned)N, (unsigned)B);
#define MI355_UNALIGNED_LAUNCH(TY) MI355_LAUNCH(k_gemv_unaligned<TY>, grid, dim3(64), 0, s, (const uint8_t *)W, aq, ads, dst, residual, N, K, dst_stride, L);
    MI355_WEIGHT_TYPE_SWITCH(type, MI355_UNALIGNED_LAUNCH)
#undef MI355_UNALIGNED_LAUNCH
    return launch_status("k_gemv_unaligned");
}

// Scratch of the allocation-free entry point: one array per GPU that loads this library, kept until the process ends.
// Host code never uses the array's name as an address (it is only a host-side handle): the device address is looked up
// once per device with hipGetSymbolAddress and kept in g_scratch_ptr.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)16 << 20;
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[STATIC_SCRATCH_BYTES];
constexpr int MAX_DEVICES = 64;
static std::atomic<void *> g_scratch_ptr[MAX_DEVICES];

// device address of this GPU's scratch array (the current device's); nullptr + error text on failure
static void *static_scratch() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
        set_error("mul_mat_static: no current device");
        return nullptr;
    }
    void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p) return p;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
        set_error("mul_mat_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
        return nullptr;
    }
    g_scratch_ptr[dev].store(p, std::memory_order_release);   // every thread finds the same address for one device
    return p;
}

}  // namespace mi355

using namespace mi355;

extern "C" {

// the per-super-block activation format of the K-quant tile kernel is smaller than the Q8_1 one
size_t mi355_mul_mat_ws_bytes(int64_t K, int64_t B) {
    size_t n = mi355_act_bytes(K, B);
    if (B > 32 && B <= 128 && K % 256 == 0) {   // the weight-streaming kernel for 33..128 rows takes tile images of the activations
        const size_t t = mi355_act_q8k_tiled_bytes(K, B);
        n = t > n ? t : n;
    }
    return (n + 255) & ~(size_t)255;
}

// 4 or 5 (Q6_K) to 32 activation rows: the weight-streaming matrix-core kernel (skinny.hip) where it supports the product.
static bool use_skinny(int type, const void *W, int64_t K, int64_t B) {
    return B >= (type == MI355_Q6_K ? 5 : 4) && B <= 32 && mi355_mul_mat_skinny_supported(type, W, K, B);
}

// 33 to 128 activation rows on Q4_K: the weight-streaming matrix-core kernel with the sub-block scales folded into the operand (mid.hip)
static bool use_mid(int type, const void *W, int64_t K, int64_t B) { return B > 32 && B <= 128 && mi355_mul_mat_mid_supported(type, W, K, B); }

// the super-block tile kernel on packed rows and per-256 activation scales: Q4_K, Q6_K, Q5_K (its per-32-block kernel is 1.5x slower
// at 512 rows, equal at 64), IQ4_XS from 256 rows on (below, the per-32-block kernel is ahead: 34 against 50 us at 64 rows of 14336 x 4096)
static bool use_q8k_tiles(int type, const void *W, int64_t K, int64_t B) {
    const bool typed = type == MI355_Q4_K || type == MI355_Q6_K || type == MI355_Q5_K || (type == MI355_IQ4_XS && B >= 256);
    return B > 8 && !use_skinny(type, W, K, B) && !use_mid(type, W, K, B) && typed && layout_aligned(W, make_row_layout(type, K));
}

int mi355_mul_mat(void *stream, int type, const void *W, const float *x, float *dst, int64_t N, int64_t K, int64_t B,
                  int64_t x_stride, int64_t dst_stride, void *ws, size_t ws_bytes) {
    MI355_REQUIRE(is_weight_type(type), "mul_mat: unsupported weight type %d", type);
    MI355_REQUIRE(N > 0 && K > 0 && B > 0, "mul_mat: bad shape N=%lld K=%lld B=%lld", (long long)N, (long long)K, (long long)B);
    MI355_REQUIRE(K % type_block_elems(type) == 0, "mul_mat: K=%lld is not a multiple of the block size", (long long)K);
    MI355_REQUIRE(dst_stride >= N, "mul_mat: dst_stride < N");
    if (ws_bytes < mi355_mul_mat_ws_bytes(K, B) || ws == nullptr) {
        set_error("mul_mat: workspace of %zu bytes, need %zu", ws_bytes, mi355_mul_mat_ws_bytes(K, B));
        return MI355_ERR_WORKSPACE;
    }
    if (use_mid(type, W, K, B)) {
        int rc = mi355_quantize_act_q8k_tiled(stream, x, ws, K, B, x_stride);
        if (rc != MI355_OK) return rc;
        const size_t used = mi355_mul_mat_ws_bytes(K, B);
        return mi355_mul_mat_mid(stream, type, W, ws, dst, nullptr, N, K, B, dst_stride, (char *)ws + used, ws_bytes - used);
    }
    if (use_q8k_tiles(type, W, K, B)) {
        int rc = mi355_quantize_act_q8k(stream, x, ws, K, B, x_stride);
        if (rc != MI355_OK) return rc;
        // what the workspace holds beyond the quantized activation serves the split along K of products with few tiles
        const size_t used = mi355_mul_mat_ws_bytes(K, B);
        return mi355_mul_mat_q8k_ws(stream, type, W, ws, dst, nullptr, N, K, B, dst_stride, (char *)ws + used, ws_bytes - used);
    }
    int rc = mi355_quantize_act(stream, x, ws, K, B, x_stride);
    if (rc != MI355_OK) return rc;
    const size_t used = mi355_mul_mat_ws_bytes(K, B);
    if (use_skinny(type, W, K, B)) return mi355_mul_mat_skinny(stream, type, W, ws, dst, nullptr, N, K, B, dst_stride, (char *)ws + used, ws_bytes - used);
    if (B <= 8) return mi355_mul_mat_vec_q(stream, type, W, ws, dst, N, K, B, dst_stride);
    return mi355_mul_mat_q_ws(stream, type, W, ws, dst, N, K, B, dst_stride, (char *)ws + used, ws_bytes - used);
}

size_t mi355_mul_mat_static_max_ws(void) { return STATIC_SCRATCH_BYTES; }

int mi355_mul_mat_static_init(void) { return static_scratch() ? MI355_OK : MI355_ERR_HIP; }

int mi355_mul_mat_static(void *stream, int type, const void *W, const float *x, float *dst, int64_t N, int64_t K, int64_t B,
                         int64_t x_stride, int64_t dst_stride) {
    MI355_REQUIRE(K > 0 && B > 0, "mul_mat_static: bad shape K=%lld B=%lld", (long long)K, (long long)B);
    const size_t need = mi355_mul_mat_ws_bytes(K, B);
    if (need > STATIC_SCRATCH_BYTES) {
        set_error("mul_mat_static: K=%lld x B=%lld needs %zu bytes of scratch, the static array holds %zu; use mi355_mul_mat with a workspace",
                  (long long)K, (long long)B, need, STATIC_SCRATCH_BYTES);
        return MI355_ERR_WORKSPACE;
    }
    void *ws = static_scratch();
    if (!ws) return MI355_ERR_HIP;
    // Nothing in the workspace has to start at zero: the quantized activation and the K-slice partial sums are written in
    // full by this call before anything reads them.
    return mi355_mul_mat(stream, type, W, x, dst, N, K, B, x_stride, dst_stride, ws, STATIC_SCRATCH_BYTES);
}

}  // extern "C"
