/*
 * Rotary position embedding of four consecutive elements (two pairs) of a row
 * at one position: (x0, x1) -> (x0*c - x1*s, x1*c + x0*s) with separately
 * rounded products (csrc/ops/reductions_cpu.c:219-226; the reference is built
 * without fused multiply-add, and rotated K rows are stored in the KV cache,
 * where they must match it bit for bit).  cs / sn point at the tables' entries
 * for the first of the two pairs.
 */
#ifndef FBLT_AMD_ROPE_DEVICE_H
#define FBLT_AMD_ROPE_DEVICE_H

#include <hip/hip_runtime.h>

__device__ __forceinline__ float4 rope_rotate4(float4 x, const float *cs, const float *sn) {
#pragma clang fp contract(off) /* no fused multiply-add in this block, also after inlining */
    const float2 c = *reinterpret_cast<const float2 *>(cs);
    const float2 s = *reinterpret_cast<const float2 *>(sn);
    float4 r;
    r.x = x.x * c.x - x.y * s.x;
    r.y = x.y * c.x + x.x * s.x;
    r.z = x.z * c.y - x.w * s.y;
    r.w = x.w * c.y + x.z * s.y;
    return r;
}

/* one pair */
__device__ __forceinline__ float2 rope_rotate2(float2 x, float c, float s) {
#pragma clang fp contract(off)
    float2 r;
    r.x = x.x * c - x.y * s;
    r.y = x.y * c + x.x * s;
    return r;
}

#endif
