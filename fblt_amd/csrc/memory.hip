/*
 * Device-memory shim of the HIP backend: the functions the reference's core
 * calls for device arenas and tensor transfers (reference contract:
 * csrc/core/cuda_shim.h:18-31; behaviour: csrc/ops/memory.cu:37-77).  Memset
 * and host-to-device copies are asynchronous on the null stream; the
 * device-to-host copy blocks and is the implicit synchronisation point.
 */
#include "blt_hip.h"
#include "hip_check.h"

extern "C" void *blt_hip_malloc(size_t bytes) {
    void *p = nullptr;
    HIP_CHECK(hipMalloc(&p, bytes));
    return p;
}

extern "C" void blt_hip_free(void *ptr) {
    if (!ptr) return;
    hipError_t e = hipFree(ptr);
    if (e != hipSuccess) BLT_WARN("HIP hipFree failed: %s", hipGetErrorString(e));
}

extern "C" void blt_hip_memset(void *dst, int value, size_t bytes) {
    if (bytes == 0) return;
    HIP_CHECK(hipMemsetAsync(dst, value, bytes, 0));
}

extern "C" void blt_hip_memcpy_h2d(void *dst, const void *src, size_t bytes) {
    if (bytes == 0) return;
    HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, 0));
}

extern "C" void blt_hip_memcpy_d2h(void *dst, const void *src, size_t bytes) {
    if (bytes == 0) return;
    HIP_CHECK(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
}

extern "C" void blt_backend_pass_sync_hip(void) {
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) BLT_FATAL("blt_backend_pass_sync: %s", hipGetErrorString(e));
}

extern "C" const char *blt_hip_build_info(void) { return "fblt_amd attention backend; kernels: gfx950"; }
