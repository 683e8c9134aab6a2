/*
 * Small device utilities of the attention path: strided tile copy (head-slice
 * gather and KV-cache write-through), the masked row softmax and the dot
 * product (reference contracts: csrc/ops/vecmath.h:14-37).
 */
#include "blt_hip.h"
#include <cstdlib>
#include "blt_fatal.h"
#include "hip_check.h"
#include "launch.h"

#include <stdint.h>

namespace {

/* One thread per 4 consecutive columns when everything is 16-byte aligned,
 * else one thread per element.  Threads run along the column axis. */
template <bool VEC4>
__global__ __launch_bounds__(256) void strided_copy_kernel(float *__restrict__ dst, uint64_t dst_stride,
                                                           const float *__restrict__ src, uint64_t src_stride,
                                                           uint64_t rows, uint64_t cols) {
    const uint64_t per_row = VEC4 ? cols / 4u : cols;
    const uint64_t total = rows * per_row;
    for (uint64_t t = (uint64_t)blockIdx.x * 256u + threadIdx.x; t < total; t += (uint64_t)gridDim.x * 256u) {
        const uint64_t r = t / per_row, c = t % per_row;
        if (VEC4) {
            *reinterpret_cast<float4 *>(dst + r * dst_stride + 4u * c) =
                *reinterpret_cast<const float4 *>(src + r * src_stride + 4u * c);
        } else {
            dst[r * dst_stride + c] = src[r * src_stride + c];
        }
    }
}

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
    return x;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
    return x;
}

/* One workgroup of 256 threads owns the row: rewrite (scale, mask / causal
 * cut), maximum over finite entries, exponentials, sum, true division. */
__global__ __launch_bounds__(256) void softmax_row_kernel(float *__restrict__ row, uint64_t len, uint64_t row_idx,
                                                          int is_causal, const float *__restrict__ mask_row,
                                                          float scale) {
    __shared__ float red[4];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;

    float top = -__builtin_huge_valf();
    for (uint64_t c = threadIdx.x; c < len; c += 256u) {
        float x;
        if (mask_row) x = row[c] * scale + mask_row[c];
        else if (is_causal && c > row_idx) x = -__builtin_huge_valf();
        else x = row[c] * scale;
        row[c] = x;
        if (isfinite(x)) top = fmaxf(top, x);
    }
    top = wave_max(top);
    if (lane == 0) red[wave] = top;
    __syncthreads();
    top = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();

    float sum = 0.f;
    for (uint64_t c = threadIdx.x; c < len; c += 256u) {
        const float x = row[c];
        const float e = isfinite(x) ? expf(x - top) : 0.f;
        row[c] = e;
        sum += e;
    }
    sum = wave_sum(sum);
    if (lane == 0) red[wave] = sum;
    __syncthreads();
    sum = (red[0] + red[1]) + (red[2] + red[3]);
    if (sum > 0.f)
        for (uint64_t c = threadIdx.x; c < len; c += 256u) row[c] = row[c] / sum;
}

__global__ __launch_bounds__(256) void dot_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                  uint64_t n, float *__restrict__ out) {
    __shared__ float red[4];
    float acc = 0.f;
    for (uint64_t t = threadIdx.x; t < n; t += 256u) acc += a[t] * b[t];
    acc = wave_sum(acc);
    if ((threadIdx.x & 63u) == 0) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) *out = (red[0] + red[1]) + (red[2] + red[3]);
}

/* dst[r, :] = src[pos[r], :] for up to GATHER_ROWS rows per launch; the row numbers travel in the
 * kernel's argument block (the reference stages them in a device scratch arena, which this
 * library does not keep), so the call neither allocates nor synchronises. */
constexpr int GATHER_ROWS = 128;
struct GatherRows {
    uint64_t pos[GATHER_ROWS];
};

template <bool VEC>
__global__ __launch_bounds__(256) void rows_gather_kernel(const float *__restrict__ src, float *__restrict__ dst,
                                                          uint64_t row_len, GatherRows rows) {
    const float *s = src + rows.pos[blockIdx.x] * row_len;
    float *d = dst + (uint64_t)blockIdx.x * row_len;
    if (VEC) {
        for (uint64_t t = threadIdx.x; t < row_len / 4u; t += 256u)
            reinterpret_cast<float4 *>(d)[t] = reinterpret_cast<const float4 *>(s)[t];
    } else {
        for (uint64_t t = threadIdx.x; t < row_len; t += 256u) d[t] = s[t];
    }
}

} // namespace

extern "C" void blt_strided_copy_hip(blt_backend backend, float *dst, size_t dst_stride, const float *src,
                                     size_t src_stride, size_t rows, size_t cols) {
    BLT_REQUIRE(backend == BLT_BACKEND_HIP, "blt_strided_copy: HIP implementation called with non-HIP backend");
    if (rows == 0 || cols == 0) return;
    BLT_REQUIRE(dst != NULL && src != NULL, "blt_strided_copy: buffers must not be NULL");
    const bool vec = ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u) == 0 &&
                     dst_stride % 4 == 0 && src_stride % 4 == 0 && cols % 4 == 0;
    const uint64_t work = rows * (vec ? cols / 4 : cols);
    const unsigned blocks = (unsigned)((work + 255u) / 256u < 4096u ? (work + 255u) / 256u : 4096u);
    if (vec)
        hipLaunchKernelGGL(strided_copy_kernel<true>, dim3(blocks), dim3(256), 0, blt_stream(), dst, (uint64_t)dst_stride, src,
                           (uint64_t)src_stride, (uint64_t)rows, (uint64_t)cols);
    else
        hipLaunchKernelGGL(strided_copy_kernel<false>, dim3(blocks), dim3(256), 0, blt_stream(), dst, (uint64_t)dst_stride, src,
                           (uint64_t)src_stride, (uint64_t)rows, (uint64_t)cols);
    HIP_CHECK_LAUNCH("blt_strided_copy");
}

extern "C" void blt_rows_gather_hip(const blt_tensor *src, const size_t *pos_host, blt_tensor *dst) {
    BLT_REQUIRE(src != NULL && dst != NULL && pos_host != NULL, "blt_rows_gather: arguments cannot be NULL");
    BLT_REQUIRE(src->backend == BLT_BACKEND_HIP && dst->backend == BLT_BACKEND_HIP,
                "blt_rows_gather: HIP implementation called with non-HIP tensors");
    BLT_REQUIRE(src->dtype == BLT_DTYPE_FP32 && dst->dtype == BLT_DTYPE_FP32, "blt_rows_gather: tensors must be FP32");
    const size_t rows = dst->ndim >= 1 ? dst->shape[0] : 0;
    if (rows == 0 || dst->numel == 0) return;
    const size_t row_len = dst->numel / rows;
    BLT_REQUIRE(src->ndim >= 1 && src->shape[src->ndim - 1] != 0 && src->numel % src->shape[src->ndim - 1] == 0,
                "blt_rows_gather: src must be row-structured");
    BLT_REQUIRE(src->numel >= row_len, "blt_rows_gather: position out of range");
    for (size_t i = 0; i < rows; i++)
        BLT_REQUIRE(pos_host[i] <= (src->numel - row_len) / row_len, "blt_rows_gather: position out of range");
    const float *s = static_cast<const float *>(src->data);
    float *d = static_cast<float *>(dst->data);
    const bool vec = ((reinterpret_cast<uintptr_t>(s) | reinterpret_cast<uintptr_t>(d)) & 15u) == 0 && row_len % 4 == 0;
    for (size_t r0 = 0; r0 < rows; r0 += GATHER_ROWS) {
        const size_t n = rows - r0 < (size_t)GATHER_ROWS ? rows - r0 : (size_t)GATHER_ROWS;
        GatherRows g;
        for (size_t i = 0; i < (size_t)GATHER_ROWS; i++) g.pos[i] = i < n ? pos_host[r0 + i] : 0;
        if (vec)
            hipLaunchKernelGGL(rows_gather_kernel<true>, dim3((unsigned)n), dim3(256), 0, blt_stream(), s,
                               d + r0 * row_len, (uint64_t)row_len, g);
        else
            hipLaunchKernelGGL(rows_gather_kernel<false>, dim3((unsigned)n), dim3(256), 0, blt_stream(), s,
                               d + r0 * row_len, (uint64_t)row_len, g);
        HIP_CHECK_LAUNCH("blt_rows_gather");
    }
}

/* csrc/ops/gather_scatter_cpu.c:7-21: out row i = table row ids_host[i] */
extern "C" void blt_embedding_lookup_hip(const blt_tensor *table, const uint32_t *ids_host, blt_tensor *out) {
    BLT_REQUIRE(table != NULL && ids_host != NULL && out != NULL, "blt_embedding_lookup: arguments cannot be NULL");
    BLT_REQUIRE(table->backend == BLT_BACKEND_HIP && out->backend == BLT_BACKEND_HIP,
                "blt_embedding_lookup: HIP implementation called with non-HIP tensors");
    BLT_REQUIRE(table->ndim == 2 && out->ndim == 2 && table->dtype == BLT_DTYPE_FP32 && out->dtype == BLT_DTYPE_FP32,
                "blt_embedding_lookup: table and out must be 2D FP32 tensors");
    BLT_REQUIRE(table->shape[1] == out->shape[1], "blt_embedding_lookup: embed_dim mismatch");
    const size_t rows = out->shape[0];
    size_t *pos = (size_t *)malloc((rows ? rows : 1) * sizeof(size_t));
    BLT_REQUIRE(pos != NULL, "blt_embedding_lookup: out of host memory");
    for (size_t i = 0; i < rows; i++) {
        BLT_REQUIRE(ids_host[i] < table->shape[0], "blt_embedding_lookup: id out of range");
        pos[i] = ids_host[i];
    }
    blt_rows_gather_hip(table, pos, out);
    free(pos);
}

extern "C" void blt_softmax_masked_row_inplace_hip(blt_backend backend, float *row, size_t row_len, size_t row_idx,
                                                   bool is_causal, const float *mask_row, float scale) {
    BLT_REQUIRE(backend == BLT_BACKEND_HIP,
                "blt_softmax_masked_row_inplace: HIP implementation called with non-HIP backend");
    if (row_len == 0) return;
    BLT_REQUIRE(row != NULL, "blt_softmax_masked_row_inplace: row must not be NULL");
    hipLaunchKernelGGL(softmax_row_kernel, dim3(1), dim3(256), 0, blt_stream(), row, (uint64_t)row_len, (uint64_t)row_idx,
                       is_causal ? 1 : 0, mask_row, scale);
    HIP_CHECK_LAUNCH("blt_softmax_masked_row_inplace");
}

extern "C" float blt_vec_dot_hip(blt_backend backend, const float *a, const float *b, size_t n) {
    BLT_REQUIRE(backend == BLT_BACKEND_HIP, "blt_vec_dot: HIP implementation called with non-HIP backend");
    if (n == 0) return 0.f;
    BLT_REQUIRE(a != NULL && b != NULL, "blt_vec_dot: buffers must not be NULL");
    static thread_local float *slot = nullptr;
    if (!slot) HIP_CHECK(hipMalloc((void **)&slot, sizeof(float)));
    hipLaunchKernelGGL(dot_kernel, dim3(1), dim3(256), 0, blt_stream(), a, b, (uint64_t)n, slot);
    HIP_CHECK_LAUNCH("blt_vec_dot");
    float r = 0.f;
    HIP_CHECK(hipMemcpyAsync(&r, slot, sizeof(float), hipMemcpyDeviceToHost, blt_stream()));
    HIP_CHECK(hipStreamSynchronize(blt_stream()));
    return r;
}
