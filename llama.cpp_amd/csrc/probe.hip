// Measurement aid: the shader clock the chip actually runs at while other work is in flight.
// One wave spins for a given time and reports how many shader-clock ticks (s_memtime) passed per tick of the constant
// 100 MHz reference counter (s_memrealtime).  Launched on a second stream next to a kernel under test it shows the clock that
// kernel gets: dense matrix-instruction kernels pull this part below its 2.4 GHz peak (power management), and rates quoted
// against the nominal peak then understate what the kernel does per clock.
#include "common.hpp"

namespace mi355 {

__global__ void __launch_bounds__(64) k_probe_clock(long long *out, long long ref_ticks) {
    const long long w0 = wall_clock64(), c0 = clock64();
    long long w = w0;
    while (w - w0 < ref_ticks) {
        __builtin_amdgcn_s_sleep(8);
        w = wall_clock64();
    }
    const long long c1 = clock64();
    if (threadIdx.x == 0) {
        out[0] = c1 - c0;   // shader clock ticks
        out[1] = w - w0;    // 100 MHz reference ticks
    }
}

// Measurement aid: the rate at which a compute unit pulls bytes into LDS with global_load_lds_dwordx4, the transfer the wide-tile
// GEMM feeds its operands with.  One 512-thread group per compute unit; every wave keeps `DEPTH` 1 KiB transfers in flight and
// walks its group's own region of `region` bytes round and round (64 KiB per group stays in L2, 4 MiB per group streams from
// HBM).  out[group] = shader-clock ticks the group took for iters * 8 KiB.
template <int DEPTH>
__global__ void __launch_bounds__(512) k_probe_lds_fill(const uint8_t *__restrict__ src, int64_t region, int iters, long long *out) {
    __shared__ __attribute__((aligned(1024))) uint8_t ring[8 * 8 * 1024];   // 8 waves x 8 slots of 1 KiB
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint8_t *base = src + (int64_t)blockIdx.x * region + wave * 1024 + lane * 16;
    const int wrap = (int)(region >> 13);
    auto fill = [&](int i) {
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)(base + (int64_t)(i % wrap) * 8192),
                                         (void __attribute__((address_space(3))) *)(ring + wave * 8192 + (i & 7) * 1024), 16, 0, 0);
    };
    const long long t0 = clock64();
    for (int i = 0; i < DEPTH; i++) fill(i);
    for (int i = DEPTH; i < iters; i++) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DEPTH - 1) : "memory");
        fill(i);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const long long t1 = clock64();
    if (threadIdx.x == 0) out[blockIdx.x] = t1 - t0 + (ring[lane] == 255 ? 1 : 0);   // the read keeps the transfers observable
}

}  // namespace mi355

extern "C" int mi355_probe_lds_fill(void *stream, const void *src, int64_t src_bytes, int64_t region, int n_groups, int iters, int64_t *out) {
    MI355_REQUIRE(src != nullptr && out != nullptr && ((uintptr_t)src & 15) == 0, "probe_lds_fill: bad pointers");
    MI355_REQUIRE(region >= 8192 && region % 8192 == 0 && n_groups > 0 && n_groups <= 4096 && iters >= 6 && iters <= (1 << 20), "probe_lds_fill: bad sizes");
    MI355_REQUIRE((int64_t)n_groups * region <= src_bytes, "probe_lds_fill: %d regions of %lld bytes do not fit the %lld-byte source", n_groups, (long long)region, (long long)src_bytes);
    MI355_LAUNCH(mi355::k_probe_lds_fill<6>, dim3((unsigned)n_groups), dim3(512), 0, (hipStream_t)stream, (const uint8_t *)src, region, iters, (long long *)out);
    return mi355::launch_status("k_probe_lds_fill");
}

extern "C" int mi355_probe_clock(void *stream, int64_t *out, int64_t micros) {
    MI355_REQUIRE(out != nullptr && micros > 0 && micros <= 1000000, "probe_clock: bad arguments");
    MI355_LAUNCH(mi355::k_probe_clock, dim3(1), dim3(64), 0, (hipStream_t)stream, (long long *)out, (long long)micros * 100);
    return mi355::launch_status("k_probe_clock");
}
