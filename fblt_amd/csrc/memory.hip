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
    HIP_CHECK(hipMemsetAsync(dst, value, bytes, blt_stream()));
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
}

extern "C" void blt_backend_pass_sync_hip(void) {
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) BLT_FATAL("blt_backend_pass_sync: %s", hipGetErrorString(e));
}

extern "C" const char *blt_hip_build_info(void) { return "fblt_amd attention backend; kernels: gfx950"; }
