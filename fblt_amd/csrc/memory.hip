/*
 * Device-memory shim of the HIP backend: the functions the reference's core
 * calls for device arenas and tensor transfers (reference contract:
 * csrc/core/cuda_shim.h:18-31; behaviour: csrc/ops/memory.cu:37-77).  Memset
 * and host-to-device copies are asynchronous on the library's current stream
 * (the null stream unless blt_hip_set_stream chose another); the
 * device-to-host copy blocks and is the implicit synchronisation point.
 */
#include "blt_hip.h"
#include "blt_fatal.h"
#include "hip_check.h"
#include "launch.h"

#include <algorithm>
#include <stdint.h>

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

namespace {

/* Byte fill as a kernel: 16-byte stores over the aligned body, single bytes at the ragged ends. */
__global__ __launch_bounds__(256) void fill_bytes_kernel(unsigned char *dst, unsigned int pattern, size_t head,
                                                         size_t body16, size_t bytes) {
    const size_t t = (size_t)blockIdx.x * 256u + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256u;
    uint4 *body = reinterpret_cast<uint4 *>(dst + head);
    for (size_t i = t; i < body16; i += stride) body[i] = make_uint4(pattern, pattern, pattern, pattern);
    const size_t tail0 = head + 16u * body16;
    for (size_t i = t; i < head; i += stride) dst[i] = (unsigned char)pattern;
    for (size_t i = tail0 + t; i < bytes; i += stride) dst[i] = (unsigned char)pattern;
}

} // namespace

/* While a graph is being captured the fill is a kernel node: memset nodes recorded into a graph
 * have replayed wrongly on this platform, and blt_tensor_create (zero-filled tensors) reaches this
 * from inside captured calls. */
extern "C" void blt_hip_memset(void *dst, int value, size_t bytes) {
    if (bytes == 0) return;
    if (!blt_stream_capturing()) {
        HIP_CHECK(hipMemsetAsync(dst, value, bytes, blt_stream()));
        return;
    }
    const uintptr_t addr = reinterpret_cast<uintptr_t>(dst);
    const size_t head = std::min<size_t>(bytes, (16u - (addr & 15u)) & 15u);
    const size_t body16 = (bytes - head) / 16u;
    const unsigned int b = (unsigned int)(value & 0xFF), pattern = b | (b << 8) | (b << 16) | (b << 24);
    const unsigned blocks = (unsigned)std::min<size_t>(2048, std::max<size_t>(1, (body16 + 255) / 256));
    hipLaunchKernelGGL(fill_bytes_kernel, dim3(blocks), dim3(256), 0, blt_stream(), static_cast<unsigned char *>(dst),
                       pattern, head, body16, bytes);
    HIP_CHECK_LAUNCH("blt_hip_memset");
}


namespace {

/* Ring of pinned buffers, one event each: a slot is reused only after the copy
 * that read it has finished. */
struct PinnedRing {
    static constexpr int SLOTS = 8;
    struct Slot {
        void *host = nullptr;
        size_t capacity = 0;
        hipEvent_t copied = nullptr;
        bool in_flight = false;
    } slot[SLOTS];
    int next = 0;
};

} // namespace

void blt_upload_staged(void *dst, const void *src, size_t bytes) {
    if (bytes == 0) return;
    BLT_REQUIRE(!blt_stream_capturing(), "host data cannot be staged to the device while a graph is captured");
    static thread_local PinnedRing ring;
    PinnedRing::Slot &s = ring.slot[ring.next];
    ring.next = (ring.next + 1) % PinnedRing::SLOTS;
    if (!s.copied) HIP_CHECK(hipEventCreateWithFlags(&s.copied, hipEventDisableTiming));
    if (s.in_flight) {
        HIP_CHECK(hipEventSynchronize(s.copied));
        s.in_flight = false;
    }
    if (bytes > s.capacity) {
        if (s.host) HIP_CHECK(hipHostFree(s.host));
        s.capacity = bytes < 32768 ? 65536 : 2 * bytes; /* few re-allocations: pinning memory costs ~100 us */
        HIP_CHECK(hipHostMalloc(&s.host, s.capacity, hipHostMallocDefault));
    }
    __builtin_memcpy(s.host, src, bytes);
    HIP_CHECK(hipMemcpyAsync(dst, s.host, bytes, hipMemcpyHostToDevice, blt_stream()));
    HIP_CHECK(hipEventRecord(s.copied, blt_stream()));
    s.in_flight = true;
}

/* The reference's callers free or reuse the host buffer as soon as the upload call returns
 * (csrc/infer/kv_cache.c:237-238), so the source must be consumed before this returns: small
 * uploads go through the pinned ring (no wait), large ones wait for the copy. */
extern "C" void blt_hip_memcpy_h2d(void *dst, const void *src, size_t bytes) {
    if (bytes == 0) return;
    if (bytes <= (1u << 20) && !blt_stream_capturing()) {
        blt_upload_staged(dst, src, bytes);
        return;
    }
    HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, blt_stream()));
    HIP_CHECK(hipStreamSynchronize(blt_stream()));
}

extern "C" void blt_hip_memcpy_d2h(void *dst, const void *src, size_t bytes) {
    if (bytes == 0) return;
    /* the copy waits for the library's current stream, whichever it is */
    HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, blt_stream()));
    HIP_CHECK(hipStreamSynchronize(blt_stream()));
    blt_kv_check_device_errors();
}

extern "C" void blt_backend_pass_sync_hip(void) {
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) BLT_FATAL("blt_backend_pass_sync: %s", hipGetErrorString(e));
    blt_kv_check_device_errors();
}

extern "C" const char *blt_hip_build_info(void) { return "fblt_amd attention backend; kernels: gfx950"; }
