/*
 * Kernel launches of the library go through blt_launch(): a plain
 * hipLaunchKernelGGL normally; while a profile is open, the same launch with
 * a start and a stop event attached to the dispatch, so that the kernel's own
 * begin/end timestamps can be read back per launch and summed per kernel tag.
 * A stream argument of 0 means the calling thread's current stream.
 */
#ifndef FBLT_AMD_LAUNCH_H
#define FBLT_AMD_LAUNCH_H

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include "hip_check.h"

bool blt_profile_is_open();
/* The calling thread's current stream (null stream by default) and whether a
 * graph capture is open on it (stream.hip). */
hipStream_t blt_stream();
bool blt_stream_capturing();
/* The stream library-owned scratch is keyed by: the current stream, or, while a capture is open,
 * the stream the thread was on when it began (the one the graph will be replayed on). */
hipStream_t blt_stream_key();
/* Host-to-device copy that returns at once and lets the caller reuse `src`
 * right away: the bytes go through a small ring of pinned buffers owned by
 * the calling thread (memory.hip).  Not usable while a graph is captured. */
void blt_upload_staged(void *dst, const void *src, size_t bytes);
/* Turns a sticky error the KV step kernels raised on the device (a sequence outgrew what its
 * launch, slab or rotation tables hold) into the fatal error; costs one 4-byte read-back, and
 * only when such a step was issued since the last look.  Called after a host wait
 * (attn_decode.hip). */
void blt_kv_check_device_errors();
/* Makes the next call of blt_kv_check_device_errors read the word: for device-length steps that
 * are issued without passing through the step's entry point (replays of a captured graph). */
void blt_kv_arm_device_error_check();
/* Tells an open capture on this thread that it recorded a KV step with device-resident lengths
 * (stream.hip); no effect outside a capture. */
void blt_stream_note_device_length_step();
/* A fresh (start, stop) event pair owned by the open profile, booked under `tag`. */
void blt_profile_book(const char *tag, hipEvent_t *start, hipEvent_t *stop);

template <typename Kernel, typename... Args>
inline void blt_launch(const char *tag, Kernel kernel, dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream,
                       Args... args) {
    if (!stream) stream = blt_stream(); /* callers pass 0 for "the library's current stream" */
    if (blt_profile_is_open()) {
        hipEvent_t e0, e1;
        blt_profile_book(tag, &e0, &e1);
        hipExtLaunchKernelGGL(kernel, grid, block, (unsigned)lds_bytes, stream, e0, e1, 0, args...);
    } else {
        hipLaunchKernelGGL(kernel, grid, block, (unsigned)lds_bytes, stream, args...);
    }
}

#endif
