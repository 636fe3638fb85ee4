// Shared device/host helpers for the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <stdint.h>
#include <stdio.h>

#include "../../include/mi355_kernels.h"

namespace mi355 {

typedef unsigned int u32;
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int WAVE = 64;

// ---- block geometry (ggml/src/ggml-common.h:161-221, 279-290, 296-308, 314-320, 399-412)
constexpr int QK = 32;     // elements per Q4_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL / Q8_0 / Q8_1 block
constexpr int QKK = 256;   // elements per K-quant super-block
constexpr int Q4_0_BYTES = 18, Q8_0_BYTES = 34, Q8_1_BYTES = 36, Q4_K_BYTES = 144, Q5_K_BYTES = 176, Q6_K_BYTES = 210;
constexpr int Q4_1_BYTES = 20, Q5_0_BYTES = 22, Q5_1_BYTES = 24, IQ4_NL_BYTES = 18, IQ4_XS_BYTES = 136;

__host__ __device__ inline int type_block_elems(int t) {
    switch (t) {
        case MI355_Q4_0: case MI355_Q8_0: case MI355_Q8_1: return QK;
        case MI355_Q4_1: case MI355_Q5_0: case MI355_Q5_1: case MI355_IQ4_NL: return QK;
        case MI355_Q4_K: case MI355_Q5_K: case MI355_Q6_K: case MI355_IQ4_XS: return QKK;
        case MI355_F32: case MI355_F16: case MI355_I32: return 1;
        default: return 0;
    }
}
__host__ __device__ inline int type_block_bytes(int t) {
    switch (t) {
        case MI355_Q4_0: return Q4_0_BYTES;
        case MI355_Q4_1: return Q4_1_BYTES;
        case MI355_Q5_0: return Q5_0_BYTES;
        case MI355_Q5_1: return Q5_1_BYTES;
        case MI355_IQ4_NL: return IQ4_NL_BYTES;
        case MI355_IQ4_XS: return IQ4_XS_BYTES;
        case MI355_Q8_0: return Q8_0_BYTES;
        case MI355_Q8_1: return Q8_1_BYTES;
        case MI355_Q4_K: return Q4_K_BYTES;
        case MI355_Q5_K: return Q5_K_BYTES;
        case MI355_Q6_K: return Q6_K_BYTES;
        case MI355_F32: case MI355_I32: return 4;
        case MI355_F16: return 2;
        default: return 0;
    }
}
__host__ __device__ inline bool is_weight_type(int t) {
    return t == MI355_Q4_0 || t == MI355_Q8_0 || t == MI355_Q4_K || t == MI355_Q5_K || t == MI355_Q6_K || t == MI355_Q4_1 || t == MI355_Q5_0 ||
           t == MI355_Q5_1 || t == MI355_IQ4_NL || t == MI355_IQ4_XS;
}
// Expands X(TYPE) for the weight type t (checked with is_weight_type before).
#define MI355_WEIGHT_TYPE_SWITCH(t, X)            \
    switch (t) {                                  \
        case MI355_Q4_0: X(MI355_Q4_0) break;     \
        case MI355_Q4_1: X(MI355_Q4_1) break;     \
        case MI355_Q5_0: X(MI355_Q5_0) break;     \
        case MI355_Q5_1: X(MI355_Q5_1) break;     \
        case MI355_IQ4_NL: X(MI355_IQ4_NL) break; \
        case MI355_Q8_0: X(MI355_Q8_0) break;     \
        case MI355_Q4_K: X(MI355_Q4_K) break;     \
        case MI355_Q5_K: X(MI355_Q5_K) break;     \
        case MI355_IQ4_XS: X(MI355_IQ4_XS) break; \
        default: X(MI355_Q6_K) break;             \
    }

// ---- activation workspace: int8 q[nrows][k] then {float d; int sum;} ds[nrows][k/32]
struct act_ds {
    float d;    // fp16-rounded block scale, widened
    int sum;    // integer sum of the 32 levels
};

// ---- small device helpers
__device__ __forceinline__ float half_bits_to_float(unsigned short h) {
    union { unsigned short u; _Float16 f; } c;
    c.u = h;
    return (float)c.f;
}
__device__ __forceinline__ unsigned short float_to_half_bits(float f) {
    union { unsigned short u; _Float16 h; } c;
    c.h = (_Float16)f;   // v_cvt_f16_f32: round to nearest even
    return c.u;
}
__device__ __forceinline__ int dot4(int a, int b, int c) { return __builtin_amdgcn_sdot4(a, b, c, false); }

// streaming (read-once) 16-byte load: keeps weights from evicting activations out of L2
__device__ __forceinline__ u32x4 load_stream16(const void *p) {
    return __builtin_nontemporal_load((const u32x4 *)p);
}
__device__ __forceinline__ u32x4 load16(const void *p) { return *(const u32x4 *)p; }

// Single roundings that stay single: the compiler may not merge these into fused multiply-adds, whatever surrounds the call.
// (The CUDA-style __fmul_rn / __fadd_rn of the HIP headers are plain operators and do get merged.)  For results that several
// kernels must reproduce bit for bit.
__device__ __forceinline__ float mul_rn(float a, float b) {
#pragma clang fp contract(off)
    return a * b;
}
__device__ __forceinline__ float add_rn(float a, float b) {
#pragma clang fp contract(off)
    return a + b;
}
__device__ __forceinline__ float sub_rn(float a, float b) {
#pragma clang fp contract(off)
    return a - b;
}

// Sum over the 64 lanes with DPP row operations (no LDS round trips: a __shfl_xor butterfly is six ds_bpermute of about a hundred
// cycles each), broadcast from lane 63 through a scalar register.  Every lane gets the same value.
template <int CTRL, int ROWMASK>
__device__ __forceinline__ float dpp_add(float v) {
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROWMASK, 0xF, true));
}
__device__ __forceinline__ float wave_sum_dpp(float v) {
    v = dpp_add<0xB1, 0xF>(v);    // quad_perm [1,0,3,2]
    v = dpp_add<0x4E, 0xF>(v);    // quad_perm [2,3,0,1]
    v = dpp_add<0x141, 0xF>(v);   // row_half_mirror
    v = dpp_add<0x140, 0xF>(v);   // row_mirror: every lane of a 16-lane row holds the row sum
    v = dpp_add<0x142, 0xA>(v);   // row_bcast15 into rows 1 and 3
    v = dpp_add<0x143, 0xC>(v);   // row_bcast31 into rows 2 and 3: lane 63 holds the total
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_sum(float v) { return wave_sum_dpp(v); }
// Maximum over the 64 lanes the same way (rows that a step does not write keep their value)
template <int CTRL, int ROWMASK>
__device__ __forceinline__ float dpp_max(float v) {
    const int b = __builtin_bit_cast(int, v);
    return fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(b, b, CTRL, ROWMASK, 0xF, false)));
}
// Maximum / integer sum over aligned groups of W lanes (4, 8, 16 or 32), every lane of the group getting the result, with DPP row
// operations: a few cycles per step where a cross-lane move through the LDS crossbar (ds_bpermute, what __shfl_xor compiles to)
// is a round trip of a hundred or so.  Both operations are exact whatever the order, so the result is that of a butterfly of
// __shfl_xor steps.  W == 32 ends with one swizzle (lane ^ 16).
template <int CTRL>
__device__ __forceinline__ int dpp_get(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true); }
template <int W>
__device__ __forceinline__ float lanes_max(float v) {
    static_assert(W == 4 || W == 8 || W == 16 || W == 32, "aligned groups of 4, 8, 16 or 32 lanes");
    v = fmaxf(v, __builtin_bit_cast(float, dpp_get<0xB1>(__builtin_bit_cast(int, v))));    // quad_perm [1,0,3,2]
    v = fmaxf(v, __builtin_bit_cast(float, dpp_get<0x4E>(__builtin_bit_cast(int, v))));    // quad_perm [2,3,0,1]
    if constexpr (W >= 8) v = fmaxf(v, __builtin_bit_cast(float, dpp_get<0x141>(__builtin_bit_cast(int, v))));    // row_half_mirror
    if constexpr (W >= 16) v = fmaxf(v, __builtin_bit_cast(float, dpp_get<0x140>(__builtin_bit_cast(int, v))));   // row_mirror
    if constexpr (W >= 32) v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F)));   // lane ^ 16
    return v;
}
template <int W>
__device__ __forceinline__ int lanes_sum_i(int v) {
    static_assert(W == 4 || W == 8 || W == 16 || W == 32, "aligned groups of 4, 8, 16 or 32 lanes");
    v += dpp_get<0xB1>(v);
    v += dpp_get<0x4E>(v);
    if constexpr (W >= 8) v += dpp_get<0x141>(v);
    if constexpr (W >= 16) v += dpp_get<0x140>(v);
    if constexpr (W >= 32) v += __builtin_amdgcn_ds_swizzle(v, 0x401F);
    return v;
}

// The largest 64-bit key (hi, lo) of the 64 lanes, to every lane: four DPP steps inside the 16-lane rows, then the four rows' winners
// through scalar registers.
__device__ __forceinline__ void wave_max_key(u32 &hi, u32 &lo) {
#define MI355_KEY_STEP(CTRL)                                                     \
    {                                                                            \
        const u32 oh = (u32)dpp_get<CTRL>((int)hi), ol = (u32)dpp_get<CTRL>((int)lo); \
        const bool take = oh > hi || (oh == hi && ol > lo);                      \
        hi = take ? oh : hi;                                                     \
        lo = take ? ol : lo;                                                     \
    }
    MI355_KEY_STEP(0xB1)
    MI355_KEY_STEP(0x4E)
    MI355_KEY_STEP(0x141)
    MI355_KEY_STEP(0x140)
#undef MI355_KEY_STEP
    u32 bh = (u32)__builtin_amdgcn_readlane((int)hi, 0), bl = (u32)__builtin_amdgcn_readlane((int)lo, 0);
#pragma unroll
    for (int r = 1; r < 4; r++) {
        const u32 oh = (u32)__builtin_amdgcn_readlane((int)hi, 16 * r), ol = (u32)__builtin_amdgcn_readlane((int)lo, 16 * r);
        const bool take = oh > bh || (oh == bh && ol > bl);
        bh = take ? oh : bh;
        bl = take ? ol : bl;
    }
    hi = bh;
    lo = bl;
}

// x / (1 + exp(-x)) for the fused SiLU * up launches: exp as v_exp_f32 of a scaled argument and the quotient as a multiplication
// by v_rcp_f32 (a few 1e-7 relative from the library forms, which cost ~35 instructions per element and made the 512-row
// launch compute-bound; the reference's own SiLU is a vectorized approximation, ggml-cpu.c:1868-1911).  The unary SILU node
// keeps the library forms.
__device__ __forceinline__ float silu_fast(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

__device__ __forceinline__ float wave_max_dpp(float v) {
    v = dpp_max<0xB1, 0xF>(v);
    v = dpp_max<0x4E, 0xF>(v);
    v = dpp_max<0x141, 0xF>(v);
    v = dpp_max<0x140, 0xF>(v);
    v = dpp_max<0x142, 0xA>(v);
    v = dpp_max<0x143, 0xC>(v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_max(float v) { return wave_max_dpp(v); }   // a maximum is the same in any order

// The values that a lane and the lane OFF away (lane ^ OFF; 8, 16 or 32) hold, as an unordered pair - the same pair, in the same
// order, in both lanes: v_permlane16_swap / v_permlane32_swap hand the halves of a register to each other in a few cycles (for 8 a
// rotation inside the 16-lane row), where __shfl_xor goes through the LDS crossbar.  For merges that are symmetric in the two.
struct lane_pair { float a, b; };
template <int OFF>
__device__ __forceinline__ lane_pair lanes_pair(float x) {
    static_assert(OFF == 8 || OFF == 16 || OFF == 32, "8, 16 or 32 lanes apart");
    const int xi = __builtin_bit_cast(int, x);
    if constexpr (OFF == 32) {
        const auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
        return lane_pair{__builtin_bit_cast(float, (int)r[0]), __builtin_bit_cast(float, (int)r[1])};
    } else if constexpr (OFF == 16) {
        const auto r = __builtin_amdgcn_permlane16_swap(xi, xi, false, false);
        return lane_pair{__builtin_bit_cast(float, (int)r[0]), __builtin_bit_cast(float, (int)r[1])};
    } else {
        const float o = __builtin_bit_cast(float, dpp_get<0x128>(xi));   // row_ror:8 = lane ^ 8 inside a row of 16
        const bool first = (threadIdx.x & 8) == 0;
        return lane_pair{first ? x : o, first ? o : x};
    }
}

// ---- host-side error plumbing
void set_error(const char *fmt, ...);

// every kernel launch of the library goes through this macro, which also counts it (mi355_launch_count)
void count_launch();
#define MI355_LAUNCH(...)               \
    do {                                \
        mi355::count_launch();          \
        hipLaunchKernelGGL(__VA_ARGS__); \
    } while (0)

#define MI355_CHECK_HIP(expr)                                                              \
    do {                                                                                   \
        hipError_t e_ = (expr);                                                            \
        if (e_ != hipSuccess) {                                                            \
            mi355::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
            return MI355_ERR_HIP;                                                          \
        }                                                                                  \
    } while (0)

#define MI355_REQUIRE(cond, ...)          \
    do {                                  \
        if (!(cond)) {                    \
            mi355::set_error(__VA_ARGS__); \
            return MI355_ERR_ARG;         \
        }                                 \
    } while (0)

inline int launch_status(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("launch of %s failed: %s", what, hipGetErrorString(e));
        return MI355_ERR_HIP;
    }
    return MI355_OK;
}

}  // namespace mi355
