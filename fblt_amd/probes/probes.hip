/*
 * Hardware yardsticks the kernel designs and the reported rooflines lean on.
 * They are measurement helpers, not part of the attention backend: they build
 * into their own small library (libfblt_probes.so) that only bench.py's
 * --probe-* modes load, so that the figures can be re-measured:
 *
 *  - a plain streaming COPY of a buffer (the yardstick hardware-counter
 *    readings of the attention kernels are scaled by: it moves exactly
 *    `bytes` in and `bytes` out);
 *  - a plain streaming READ of a buffer (what a purely bandwidth-bound kernel
 *    attains on this part, against the published HBM peak);
 *  - an issue probe: wavefronts that run only v_mfma_f32_32x32x2_f32, only
 *    v_fma_f32, or both kinds side by side on the same SIMDs.  It answers
 *    whether fp32 matrix instructions and ordinary vector instructions of
 *    different waves overlap on a SIMD (they do not on gfx950: the mixed run
 *    takes the sum of the two separate times).
 */
#include "blt_fatal.h"
#include "hip_check.h"

#include <stddef.h>

#include <stdint.h>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void stream_copy_kernel(float4 *__restrict__ dst, const float4 *__restrict__ src,
                                                          size_t n16) {
    for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256u) dst[i] = src[i];
}

__global__ __launch_bounds__(256) void stream_read_kernel(const float4 *__restrict__ src, size_t n16,
                                                          float *__restrict__ sink) {
    const size_t stride = (size_t)gridDim.x * 256u;
    size_t i = (size_t)blockIdx.x * 256u + threadIdx.x;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (; i + 7u * stride < n16; i += 8u * stride) {
        float4 t[8];
#pragma unroll
        for (int u = 0; u < 8; u++) t[u] = src[i + u * stride];
#pragma unroll
        for (int u = 0; u < 8; u++) acc.x += t[u].x, acc.y += t[u].y, acc.z += t[u].z, acc.w += t[u].w;
    }
    for (; i < n16; i += stride) {
        const float4 t = src[i];
        acc.x += t.x, acc.y += t.y, acc.z += t.z, acc.w += t.w;
    }
    if (acc.x + acc.y + acc.z + acc.w == 1234.5678f) sink[0] = 1.f; /* keeps the loads alive */
}

/* 512 threads = 8 waves = 2 per SIMD.  Waves 0-3 (one per SIMD) run the matrix
 * stream when mode & 1, waves 4-7 (again one per SIMD) the vector stream when
 * mode & 2; idle waves leave at once.  Per group of 8 MFMAs (512 cycles of
 * matrix pipe) the vector waves issue 64 dependent-free FMAs (256 cycles). */
__global__ __launch_bounds__(512) void issue_probe_kernel(float *__restrict__ sink, int groups, int mode, float a,
                                                          float b) {
    const int wave = threadIdx.x >> 6;
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = threadIdx.x * 0.001f;
    float v[8];
#pragma unroll
    for (int r = 0; r < 8; r++) v[r] = threadIdx.x * 0.5f + r;
    if (wave < 4) {
        if (mode & 1)
            for (int i = 0; i < groups; i++) {
#pragma unroll
                for (int u = 0; u < 8; u++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
            }
    } else if (mode & 2) {
        for (int i = 0; i < groups; i++) {
#pragma unroll
            for (int u = 0; u < 8; u++)
#pragma unroll
                for (int r = 0; r < 8; r++) v[r] = __builtin_fmaf(v[r], a, b);
        }
    }
    float s = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r++) s += acc[r];
#pragma unroll
    for (int r = 0; r < 8; r++) s += v[r];
    sink[(size_t)blockIdx.x * 512u + threadIdx.x] = s;
}

float timed_ms(hipEvent_t e0, hipEvent_t e1) {
    float ms = 0.f;
    HIP_CHECK(hipEventSynchronize(e1));
    HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
    return ms;
}

} // namespace

/* Plain device-to-device streaming copy of `bytes` (a multiple of 16) on the null stream. */
extern "C" void blt_probe_stream_copy(void *dst, const void *src, size_t bytes) {
    BLT_REQUIRE(dst != NULL && src != NULL && bytes % 16 == 0, "blt_probe_stream_copy: need 16-byte multiples");
    if (bytes == 0) return;
    hipLaunchKernelGGL(stream_copy_kernel, dim3(2048), dim3(256), 0, 0, static_cast<float4 *>(dst),
                       static_cast<const float4 *>(src), bytes / 16);
    HIP_CHECK_LAUNCH("blt_probe_stream_copy");
}

/* Plain streaming read of `bytes` device bytes, `launches` times back to back after one warm-up;
 * returns milliseconds per launch (HIP events). */
extern "C" float blt_probe_stream_read(const void *src, size_t bytes, int launches) {
    BLT_REQUIRE(src != NULL && bytes % 16 == 0 && bytes > 0 && launches >= 1,
                "blt_probe_stream_read: need a buffer of 16-byte multiples");
    float *sink = nullptr;
    HIP_CHECK(hipMalloc((void **)&sink, 64));
    hipEvent_t e0, e1;
    HIP_CHECK(hipEventCreate(&e0));
    HIP_CHECK(hipEventCreate(&e1));
    hipLaunchKernelGGL(stream_read_kernel, dim3(2048), dim3(256), 0, 0, static_cast<const float4 *>(src), bytes / 16,
                       sink);
    HIP_CHECK(hipEventRecord(e0, 0));
    for (int i = 0; i < launches; i++)
        hipLaunchKernelGGL(stream_read_kernel, dim3(2048), dim3(256), 0, 0, static_cast<const float4 *>(src),
                           bytes / 16, sink);
    HIP_CHECK(hipEventRecord(e1, 0));
    const float ms = timed_ms(e0, e1);
    HIP_CHECK(hipEventDestroy(e0));
    HIP_CHECK(hipEventDestroy(e1));
    HIP_CHECK(hipFree(sink));
    return ms / launches;
}

/* One launch of 256 workgroups of 8 waves (2 per SIMD) in which one wave per SIMD runs `groups` x 8
 * v_mfma_f32_32x32x2_f32 (mode & 1) and / or the other runs `groups` x 64 v_fma_f32 (mode & 2).
 * Returns the launch's milliseconds: mode 3 ~ mode 1 + mode 2 means the two do not overlap. */
extern "C" float blt_probe_issue(int mode, int groups) {
    BLT_REQUIRE(mode >= 1 && mode <= 3 && groups >= 1, "blt_probe_issue: mode is 1 (matrix), 2 (vector) or 3 (both)");
    float *sink = nullptr;
    HIP_CHECK(hipMalloc((void **)&sink, 256u * 512u * sizeof(float)));
    hipEvent_t e0, e1;
    HIP_CHECK(hipEventCreate(&e0));
    HIP_CHECK(hipEventCreate(&e1));
    hipLaunchKernelGGL(issue_probe_kernel, dim3(256), dim3(512), 0, 0, sink, 16, mode, 1.0f, 0.5f);
    HIP_CHECK(hipEventRecord(e0, 0));
    hipLaunchKernelGGL(issue_probe_kernel, dim3(256), dim3(512), 0, 0, sink, groups, mode, 1.0f, 0.5f);
    HIP_CHECK(hipEventRecord(e1, 0));
    const float ms = timed_ms(e0, e1);
    HIP_CHECK(hipEventDestroy(e0));
    HIP_CHECK(hipEventDestroy(e1));
    HIP_CHECK(hipFree(sink));
    return ms;
}
