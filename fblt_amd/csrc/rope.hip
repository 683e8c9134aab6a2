/*
 * Rotary position embedding on device rows (reference contracts:
 * csrc/ops/rope.h:19-27; CPU loops csrc/ops/reductions_cpu.c:199-229 and
 * csrc/core/backend.c:323-345; device twins csrc/ops/reductions.cu:253-340).
 * Element-wise and bit-identical to the reference's CPU loops: products and
 * sums are rounded separately.
 */
#include "blt_hip.h"
#include "blt_fatal.h"
#include "hip_check.h"
#include "launch.h"
#include "rope_device.h"

#include <stdint.h>

namespace {

/* One thread per (row t, head, pair i): src / dst row pitch and head pitch in elements. */
__global__ __launch_bounds__(256) void rope_pairs_kernel(const float *__restrict__ src, float *__restrict__ dst,
                                                         uint64_t row_pitch, uint64_t head_pitch, uint64_t rows,
                                                         uint32_t heads, uint32_t half, const float *__restrict__ cs,
                                                         const float *__restrict__ sn) {
    const uint64_t total = rows * heads * half;
    for (uint64_t e = (uint64_t)blockIdx.x * 256u + threadIdx.x; e < total; e += (uint64_t)gridDim.x * 256u) {
        const uint32_t i = (uint32_t)(e % half);
        const uint32_t hh = (uint32_t)((e / half) % heads);
        const uint64_t t = e / ((uint64_t)half * heads);
        const uint64_t at = t * row_pitch + hh * head_pitch + 2u * i;
        const float2 x = make_float2(src[at], src[at + 1]);
        const float2 r = rope_rotate2(x, cs[t * half + i], sn[t * half + i]);
        dst[at] = r.x;
        dst[at + 1] = r.y;
    }
}

void launch_pairs(const float *src, float *dst, uint64_t row_pitch, uint64_t head_pitch, uint64_t rows, uint32_t heads,
                  uint32_t half, const float *cs, const float *sn) {
    const uint64_t total = rows * heads * half;
    if (total == 0) return;
    const uint32_t blocks = (uint32_t)((total + 255u) / 256u < 4096u ? (total + 255u) / 256u : 4096u);
    blt_launch("rope_pairs", rope_pairs_kernel, dim3(blocks), dim3(256), 0, 0, src, dst, row_pitch, head_pitch, rows,
               heads, half, cs, sn);
}

void check_nd_fp32(const blt_tensor *t, size_t ndim, const char *what) {
    BLT_REQUIRE(t != NULL && t->data != NULL, "%s", what);
    BLT_REQUIRE(t->ndim == ndim && t->dtype == BLT_DTYPE_FP32, "%s", what);
    BLT_REQUIRE(t->backend == BLT_BACKEND_HIP, "%s (HIP implementation called with a non-HIP tensor)", what);
}

} // namespace

extern "C" void blt_rope_apply_hip(const blt_tensor *x, const blt_tensor *cos, const blt_tensor *sin,
                                   blt_tensor *out) {
    check_nd_fp32(x, 3, "rope: x must be 3D FP32");
    check_nd_fp32(cos, 2, "rope: cos shape mismatch");
    check_nd_fp32(sin, 2, "rope: sin shape mismatch");
    check_nd_fp32(out, 3, "rope: out shape mismatch");
    const size_t seq_len = x->shape[0], heads = x->shape[1], hd = x->shape[2];
    BLT_REQUIRE(hd % 2 == 0, "rope: head_dim must be even");
    BLT_REQUIRE(cos->shape[0] == seq_len && cos->shape[1] == hd / 2, "rope: cos shape mismatch");
    BLT_REQUIRE(sin->shape[0] == seq_len && sin->shape[1] == hd / 2, "rope: sin shape mismatch");
    BLT_REQUIRE(out->shape[0] == seq_len && out->shape[1] == heads && out->shape[2] == hd, "rope: out shape mismatch");
    BLT_REQUIRE(heads <= 0xFFFFFFFFu && hd <= 0xFFFFFFFFu, "rope: dimensions exceed 2^32-1");
    launch_pairs((const float *)x->data, (float *)out->data, heads * hd, hd, seq_len, (uint32_t)heads,
                 (uint32_t)(hd / 2), (const float *)cos->data, (const float *)sin->data);
    HIP_CHECK_LAUNCH("blt_rope_apply");
}

extern "C" void blt_rope_apply_packed_hip(float *qkv_data, size_t qkv_stride, size_t head_offset, size_t seq_len,
                                          size_t head_dim, const float *cos, const float *sin) {
    BLT_REQUIRE(qkv_data != NULL && cos != NULL && sin != NULL, "rope: buffers must not be NULL");
    BLT_REQUIRE(head_dim % 2 == 0 && head_dim <= 0xFFFFFFFFu, "rope: head_dim must be even");
    launch_pairs(qkv_data + head_offset, qkv_data + head_offset, qkv_stride, 0, seq_len, 1u, (uint32_t)(head_dim / 2),
                 cos, sin);
    HIP_CHECK_LAUNCH("blt_rope_apply_packed");
}
