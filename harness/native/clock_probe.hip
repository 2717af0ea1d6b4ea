// clock_probe.hip -- what clock the shader cores run at, sampled by a kernel: a fixed chain of
// dependent fused multiply-adds executed by one wavefront, bracketed by the shader-clock counter
// (clock64) and the constant-rate counter (wall_clock64, 100 MHz).  bench.py launches it on the
// benchmark's stream right after a batch of launches to report the clock that batch left behind
// (kernels bound by their vector instructions follow it).  Measurement only: not part of the library.
#include <hip/hip_runtime.h>
#include <stdint.h>

__global__ void clock_probe_kernel(uint64_t *out, int iters, float seed)
{
    float x = seed;
    const uint64_t w0 = wall_clock64();
    const uint64_t c0 = clock64();
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int k = 0; k < 64; k++) x = __builtin_fmaf(x, 0.999999f, 1e-7f);
    }
    const uint64_t c1 = clock64();
    const uint64_t w1 = wall_clock64();
    if (threadIdx.x == 0) {
        out[0] = c1 - c0;      // shader-clock ticks (if the counter follows the shader clock)
        out[1] = w1 - w0;      // constant-rate ticks
        out[2] = (uint64_t)(x != 12345.0f);   // keeps the chain alive
    }
}

extern "C" int clock_probe_launch(uint64_t *out_dev, int iters, void *stream)
{
    clock_probe_kernel<<<1, 64, 0, static_cast<hipStream_t>(stream)>>>(out_dev, iters, 0.5f);
    return (int)hipGetLastError();
}

extern "C" int clock_probe_wall_rate_khz(void)
{
    int khz = 0;
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, 0) != hipSuccess) return 0;
    return khz;
}
