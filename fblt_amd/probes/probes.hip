/*
 * Two measurement yardsticks, not part of the attention backend: they build
 * into their own small library (libfblt_probes.so) that only bench.py loads.
 *
 *  - the counter yardstick: a plain streaming COPY of a buffer.  It moves
 *    exactly `bytes` in and `bytes` out, so the hardware-counter readings
 *    (FETCH_SIZE, WRITE_SIZE) of the attention kernels are scaled by what the
 *    same counters read for it (bench.py --probe-copy-mib);
 *  - the launch floor: an empty kernel timed the way bench.py times every
 *    kernel (start / stop events attached to the dispatch) and by the host
 *    clock over back-to-back launches.  The first is what a kernel's reported
 *    duration cannot go below; the second is smaller, because the dispatch
 *    overhead inside an event-timed duration overlaps the previous kernel
 *    when launches follow each other -- which is why a short kernel's event
 *    duration can exceed the wall time per step of a back-to-back loop.
 */
#include "blt_fatal.h"
#include "hip_check.h"

#include <hip/hip_ext.h>

#include <stddef.h>
#include <stdint.h>

#include <algorithm>
#include <chrono>
#include <vector>

namespace {

__global__ __launch_bounds__(256) void stream_copy_kernel(float4 *__restrict__ dst, const float4 *__restrict__ src,
                                                          size_t n16) {
    for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256u) dst[i] = src[i];
}

__global__ void empty_kernel() {}

} // namespace

/* Plain device-to-device streaming copy of `bytes` (a multiple of 16) on the null stream. */
extern "C" void blt_probe_stream_copy(void *dst, const void *src, size_t bytes) {
    BLT_REQUIRE(dst != NULL && src != NULL && bytes % 16 == 0, "blt_probe_stream_copy: need 16-byte multiples");
    if (bytes == 0) return;
    hipLaunchKernelGGL(stream_copy_kernel, dim3(2048), dim3(256), 0, 0, static_cast<float4 *>(dst),
                       static_cast<const float4 *>(src), bytes / 16);
    HIP_CHECK_LAUNCH("blt_probe_stream_copy");
}

/* `launches` (at least 1) empty kernels of 256 workgroups x 256 threads on the null stream: the mean and the
 * median of their event-timed durations, and the wall time per launch of the same number issued
 * back to back without events; all in microseconds. */
extern "C" void blt_probe_launch_floor(int launches, float *event_us_mean, float *event_us_median, float *wall_us) {
    BLT_REQUIRE(launches >= 1 && event_us_mean && event_us_median && wall_us, "blt_probe_launch_floor: bad arguments");
    std::vector<hipEvent_t> e0(launches), e1(launches);
    for (int i = 0; i < launches; i++) {
        HIP_CHECK(hipEventCreate(&e0[i]));
        HIP_CHECK(hipEventCreate(&e1[i]));
    }
    for (int i = 0; i < 20; i++) hipLaunchKernelGGL(empty_kernel, dim3(256), dim3(256), 0, 0);
    HIP_CHECK(hipDeviceSynchronize());
    for (int i = 0; i < launches; i++) hipExtLaunchKernelGGL(empty_kernel, dim3(256), dim3(256), 0, 0, e0[i], e1[i], 0);
    HIP_CHECK(hipDeviceSynchronize());
    std::vector<float> us(launches);
    double sum = 0.0;
    for (int i = 0; i < launches; i++) {
        float ms = 0.f;
        HIP_CHECK(hipEventElapsedTime(&ms, e0[i], e1[i]));
        us[i] = ms * 1e3f;
        sum += us[i];
        HIP_CHECK(hipEventDestroy(e0[i]));
        HIP_CHECK(hipEventDestroy(e1[i]));
    }
    std::sort(us.begin(), us.end());
    *event_us_mean = (float)(sum / launches);
    *event_us_median = us[launches / 2];
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < launches; i++) hipLaunchKernelGGL(empty_kernel, dim3(256), dim3(256), 0, 0);
    HIP_CHECK(hipDeviceSynchronize());
    const auto t1 = std::chrono::steady_clock::now();
    *wall_us = (float)(std::chrono::duration<double, std::micro>(t1 - t0).count() / launches);
}
