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

}  // namespace mi355

extern "C" int mi355_probe_clock(void *stream, int64_t *out, int64_t micros) {
    MI355_REQUIRE(out != nullptr && micros > 0 && micros <= 1000000, "probe_clock: bad arguments");
    MI355_LAUNCH(mi355::k_probe_clock, dim3(1), dim3(64), 0, (hipStream_t)stream, (long long *)out, (long long)micros * 100);
    return mi355::launch_status("k_probe_clock");
}
