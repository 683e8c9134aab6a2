/* HIP error handling in the fBLT fatal-error style (reference behaviour:
 * csrc/ops/memory.cu:7-11, attn_core.cu:19-25). */
#ifndef FBLT_AMD_HIP_CHECK_H
#define FBLT_AMD_HIP_CHECK_H

#include <hip/hip_runtime.h>
#include "blt_fatal.h"

#define HIP_CHECK(expr)                                                                                            \
    do {                                                                                                           \
        hipError_t blt_hip_err_ = (expr);                                                                          \
        if (blt_hip_err_ != hipSuccess) BLT_FATAL("HIP %s failed: %s", #expr, hipGetErrorString(blt_hip_err_));    \
    } while (0)

/* After a kernel launch: report a launch-time error (no synchronisation). */
#define HIP_CHECK_LAUNCH(what)                                                                                     \
    do {                                                                                                           \
        hipError_t blt_hip_err_ = hipGetLastError();                                                               \
        if (blt_hip_err_ != hipSuccess) BLT_FATAL("%s failed: %s", what, hipGetErrorString(blt_hip_err_));         \
    } while (0)

/* The calling wave's outstanding vector-memory operations have completed when this returns
 * (device-scope write-through stores are then visible to the other workgroups of the launch).
 * Placed between a workgroup's published data and the barrier before its ticket, so that the
 * order "data, then ticket" rests on a wait the source states rather than on one the compiler
 * happens to emit for the barrier. */
__device__ __forceinline__ void blt_vector_memory_done() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

#endif
