/*
 * The small row ops around the attention block in a decoder layer, and the
 * batched decode layer built from them (reference: csrc/infer/kv_cache.c:
 * 326-414 for one sequence; ops csrc/ops/reductions_cpu.c:325-352 RMSNorm,
 * csrc/ops/elementwise_cpu.c:9-18 add, 86-99 SwiGLU).
 *
 * RMSNorm keeps the reference's arithmetic exactly -- the squares are summed
 * in element order with separately rounded products, one lane per row, then
 * 1/sqrtf(mean + eps) and two multiplications per element -- so its result is
 * bit-identical to blt_rmsnorm_forward_cpu.  The rows of a decode step are
 * few and short; the serial sum costs a few microseconds.  add is exact by
 * nature; SwiGLU uses the device expf and is within fp32 tolerance.
 */
#include "blt_hip.h"
#include "blt_fatal.h"
#include "hip_check.h"
#include "launch.h"
#include "matmul.h"

#include <cmath>
#include <cstring>

namespace {

constexpr float RMSNORM_EPS = 1e-6f; /* csrc/ops/reductions_cpu.c:325 */

/* `parts` lanes (a power of two, 8..64) share a row's loads (coalesced, into
 * LDS), one of them then walks the row in element order.  256 / parts rows
 * per workgroup. */
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                           float *__restrict__ out, uint32_t rows, uint32_t dim,
                                                           uint32_t parts) {
#pragma clang fp contract(off) /* products and sums rounded separately, as the reference's loop */
    extern __shared__ __attribute__((aligned(16))) float stage[]; /* [256 / parts rows][pitch] */
    const uint32_t pitch = ((dim + 3u) & ~3u) + 4u; /* rows start 16-byte aligned, 4 banks apart */
    const uint32_t r_local = threadIdx.x / parts, part = threadIdx.x % parts;
    const uint32_t row = blockIdx.x * (256u / parts) + r_local;
    const bool ok = row < rows;
    const float *src = x + (size_t)(ok ? row : rows - 1u) * dim;
    for (uint32_t j = part; j < dim; j += parts) stage[r_local * pitch + j] = src[j];
    __syncthreads();
    float inv_rms = 0.f;
    if (part == 0) {
        float sumsq = 0.0f;
        const float *mine = stage + r_local * pitch;
        uint32_t j = 0;
        for (; j + 16u <= dim; j += 16u) { /* loads in bulk, then the sums in element order */
            float v[16];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4 t = *reinterpret_cast<const float4 *>(mine + j + 4 * q);
                v[4 * q + 0] = t.x, v[4 * q + 1] = t.y, v[4 * q + 2] = t.z, v[4 * q + 3] = t.w;
            }
#pragma unroll
            for (int q = 0; q < 16; q++) sumsq = sumsq + v[q] * v[q];
        }
        for (; j < dim; j++) sumsq = sumsq + mine[j] * mine[j];
        const float mean_sq = sumsq / (float)dim;
        inv_rms = 1.0f / sqrtf(mean_sq + RMSNORM_EPS);
    }
    inv_rms = __shfl(inv_rms, (int)((threadIdx.x & 63u) & ~(parts - 1u)), 64);
    if (!ok) return;
    float *dst = out + (size_t)row * dim;
    for (uint32_t j = part; j < dim; j += parts) dst[j] = stage[r_local * pitch + j] * inv_rms * w[j];
}

__global__ __launch_bounds__(256) void add_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                  float *__restrict__ out, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256u)
        out[i] = a[i] + b[i];
}

__global__ __launch_bounds__(256) void swiglu_kernel(const float *__restrict__ gate, const float *__restrict__ up,
                                                     float *__restrict__ out, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256u) {
        const float gv = gate[i];
        const float silu = gv / (1.0f + expf(-gv));
        out[i] = silu * up[i];
    }
}

uint32_t blocks_for(uint64_t n) { return (uint32_t)((n + 255u) / 256u < 2048u ? (n + 255u) / 256u : 2048u); }

void rmsnorm_launch(const float *x, const float *w, float *out, size_t rows, size_t dim) {
    if (rows == 0 || dim == 0) return;
    uint32_t parts = 8u; /* 32 rows per workgroup while they fit 48 KB of LDS, fewer for wide rows */
    const size_t pitch = ((dim + 3u) & ~(size_t)3u) + 4u;
    while (parts < 64u && (256u / parts) * pitch * sizeof(float) > 48u * 1024u) parts *= 2u;
    const uint32_t rpw = 256u / parts;
    const size_t lds = rpw * pitch * sizeof(float);
    BLT_REQUIRE(lds <= 64u * 1024u, "RMSNorm: embed_dim up to 4088 is supported by the HIP backend (got %zu)", dim);
    blt_launch("rmsnorm_rows", rmsnorm_rows_kernel, dim3((uint32_t)((rows + rpw - 1u) / rpw)), dim3(256), lds, 0, x, w,
               out, (uint32_t)rows, (uint32_t)dim, parts);
}
void add_launch(const float *a, const float *b, float *out, size_t n) {
    if (n) blt_launch("add", add_kernel, dim3(blocks_for(n)), dim3(256), 0, 0, a, b, out, (uint64_t)n);
}
void swiglu_launch(const float *g, const float *u, float *out, size_t n) {
    if (n) blt_launch("swiglu", swiglu_kernel, dim3(blocks_for(n)), dim3(256), 0, 0, g, u, out, (uint64_t)n);
}

void check_fp32_hip(const blt_tensor *t, const char *what) {
    BLT_REQUIRE(t != NULL && t->data != NULL && t->dtype == BLT_DTYPE_FP32, "%s", what);
    BLT_REQUIRE(t->backend == BLT_BACKEND_HIP, "%s (HIP implementation called with a non-HIP tensor)", what);
}

void check_weight(const blt_tensor *t, size_t rows, size_t cols, const char *what) {
    BLT_REQUIRE(t != NULL && t->data != NULL && t->ndim == 2 && t->shape[0] == rows && t->shape[1] == cols, "%s", what);
    BLT_REQUIRE(t->dtype == BLT_DTYPE_FP32 && t->backend == BLT_BACKEND_HIP,
                "%s (the HIP backend takes FP32 device weights only)", what);
}

/* out = a * b (+ residual), or silu(a * gate_w) .* (a * b) with gate_w set */
void gemm(const float *a, const float *b, float *out, size_t m, size_t k, size_t n, const float *residual = nullptr,
          const float *gate_w = nullptr, const float *norm_w = nullptr) {
    MatmulArgs g;
    std::memset(&g, 0, sizeof(g));
    g.a = a, g.b = b, g.out = out;
    g.residual = residual, g.b2 = gate_w, g.norm_w = norm_w;
    g.m = (uint32_t)m, g.k = (uint32_t)k, g.n = (uint32_t)n;
    g.lda = (uint32_t)k, g.ldb = (uint32_t)n, g.ldo = (uint32_t)n;
    matmul_f32_launch(g, 0);
}

} // namespace

extern "C" void blt_rmsnorm_forward_hip(const blt_tensor *x, const blt_tensor *weight, blt_tensor *out) {
    check_fp32_hip(x, "RMSNorm: input must be 2D FP32");
    check_fp32_hip(weight, "RMSNorm: weight must be [embed_dim] FP32");
    check_fp32_hip(out, "RMSNorm: output shape/dtype mismatch");
    BLT_REQUIRE(x->ndim == 2, "RMSNorm: input must be 2D FP32");
    const size_t rows = x->shape[0], dim = x->shape[1];
    BLT_REQUIRE(weight->ndim == 1 && weight->shape[0] == dim, "RMSNorm: weight must be [embed_dim] FP32");
    BLT_REQUIRE(out->ndim == 2 && out->shape[0] == rows && out->shape[1] == dim, "RMSNorm: output shape/dtype mismatch");
    BLT_REQUIRE(rows <= 0x7FFFFFFFu, "RMSNorm: too many rows");
    rmsnorm_launch((const float *)x->data, (const float *)weight->data, (float *)out->data, rows, dim);
    HIP_CHECK_LAUNCH("blt_rmsnorm_forward");
}

extern "C" void blt_add_hip(const blt_tensor *a, const blt_tensor *b, blt_tensor *out) {
    check_fp32_hip(a, "blt_add: input tensors must be FP32 with matching element count");
    check_fp32_hip(b, "blt_add: input tensors must be FP32 with matching element count");
    check_fp32_hip(out, "blt_add: output tensor must be FP32 with matching element count");
    BLT_REQUIRE(a->numel == b->numel && a->numel == out->numel,
                "blt_add: tensors must be FP32 with matching element count");
    add_launch((const float *)a->data, (const float *)b->data, (float *)out->data, a->numel);
    HIP_CHECK_LAUNCH("blt_add");
}

extern "C" void blt_swiglu_forward_hip(const blt_tensor *gate, const blt_tensor *up, blt_tensor *out) {
    check_fp32_hip(gate, "SwiGLU: gate/up must be FP32 with matching element count");
    check_fp32_hip(up, "SwiGLU: gate/up must be FP32 with matching element count");
    check_fp32_hip(out, "SwiGLU: output must be FP32 with matching element count");
    BLT_REQUIRE(gate->numel == up->numel && gate->numel == out->numel,
                "SwiGLU: tensors must be FP32 with matching element count");
    swiglu_launch((const float *)gate->data, (const float *)up->data, (float *)out->data, gate->numel);
    HIP_CHECK_LAUNCH("blt_swiglu_forward");
}

extern "C" void blt_kv_decode_layer_hip(const blt_kv_attn_cache *cache, const blt_transformer_weights *w,
                                        const float *rows_in, float *rows_out, const float *rope_cos,
                                        const float *rope_sin, size_t rope_positions, size_t n, int step_kind,
                                        int commit, size_t max_len_hint, blt_arena *arena) {
    BLT_REQUIRE(cache != NULL && w != NULL && rows_in != NULL && rows_out != NULL && arena != NULL,
                "blt_kv_decode_layer: arguments must not be NULL");
    BLT_REQUIRE(arena->backend == BLT_BACKEND_HIP, "blt_kv_decode_layer: needs a device arena");
    BLT_REQUIRE(w->norm1_bias == NULL && w->norm2_bias == NULL,
                "blt_kv_decode_layer: RMSNorm blocks only (norm biases must be NULL)");
    BLT_REQUIRE(w->ffn_gate_w != NULL, "blt_kv_decode_layer: SwiGLU blocks only (ffn_gate_w must be set)");
    const size_t E = cache->embed_dim, rows = cache->batch * n;
    BLT_REQUIRE(w->norm1_weight != NULL && w->norm1_weight->ndim == 1 && w->norm1_weight->shape[0] == E &&
                    w->norm2_weight != NULL && w->norm2_weight->ndim == 1 && w->norm2_weight->shape[0] == E,
                "blt_kv_decode_layer: norm weights must be [embed_dim]");
    check_fp32_hip(w->norm1_weight, "blt_kv_decode_layer: norm1_weight must be FP32");
    check_fp32_hip(w->norm2_weight, "blt_kv_decode_layer: norm2_weight must be FP32");
    check_weight(w->attn_qkv_w, E, 3 * E, "blt_kv_decode_layer: attn_qkv_w must be [embed_dim, 3*embed_dim]");
    check_weight(w->attn_proj_w, E, E, "blt_kv_decode_layer: attn_proj_w must be [embed_dim, embed_dim]");
    BLT_REQUIRE(w->ffn_up_w != NULL && w->ffn_up_w->ndim == 2, "blt_kv_decode_layer: ffn_up_w must be 2D");
    const size_t Hd = w->ffn_up_w->shape[1];
    check_weight(w->ffn_up_w, E, Hd, "blt_kv_decode_layer: ffn_up_w must be [embed_dim, hidden_dim]");
    check_weight(w->ffn_gate_w, E, Hd, "blt_kv_decode_layer: ffn_gate_w must be [embed_dim, hidden_dim]");
    check_weight(w->ffn_down_w, Hd, E, "blt_kv_decode_layer: ffn_down_w must be [hidden_dim, embed_dim]");
    if (rows == 0) return;

    auto f32 = [](const blt_tensor *t) { return (const float *)t->data; };
    float *normed = (float *)blt_arena_alloc(arena, rows * E * sizeof(float), 64);
    float *qkv = (float *)blt_arena_alloc(arena, rows * 3 * E * sizeof(float), 64);
    float *combined = (float *)blt_arena_alloc(arena, rows * E * sizeof(float), 64);
    float *resid1 = (float *)blt_arena_alloc(arena, rows * E * sizeof(float), 64);
    float *up = (float *)blt_arena_alloc(arena, rows * Hd * sizeof(float), 64);
    float *gate = (float *)blt_arena_alloc(arena, rows * Hd * sizeof(float), 64);

    MatmulArgs probe;
    std::memset(&probe, 0, sizeof(probe));
    probe.m = (uint32_t)rows, probe.k = (uint32_t)E;
    /* self-attention block, kv_cache.c:326-394 */
    probe.n = (uint32_t)(3 * E);
    if (matmul_takes_norm(probe)) {
        gemm(rows_in, f32(w->attn_qkv_w), qkv, rows, E, 3 * E, nullptr, nullptr, f32(w->norm1_weight));
    } else {
        rmsnorm_launch(rows_in, f32(w->norm1_weight), normed, rows, E);
        gemm(normed, f32(w->attn_qkv_w), qkv, rows, E, 3 * E);
    }
    blt_kv_rope_attend_step_hip(cache, qkv, 3 * E, qkv + E, 3 * E, qkv + 2 * E, 3 * E, rope_cos, rope_sin,
                                rope_positions, combined, E, n, step_kind, commit, max_len_hint);
    gemm(combined, f32(w->attn_proj_w), resid1, rows, E, E, rows_in); /* projection + residual in one pass */
    /* feed-forward block, kv_cache.c:396-414 */
    probe.n = (uint32_t)Hd;
    if (matmul_takes_norm(probe)) { /* RMSNorm, up, gate and SwiGLU in one pass */
        gemm(resid1, f32(w->ffn_up_w), gate, rows, E, Hd, nullptr, f32(w->ffn_gate_w), f32(w->norm2_weight));
    } else if (matmul_takes_gated(probe)) {
        rmsnorm_launch(resid1, f32(w->norm2_weight), normed, rows, E);
        gemm(normed, f32(w->ffn_up_w), gate, rows, E, Hd, nullptr, f32(w->ffn_gate_w)); /* up, gate, SwiGLU */
    } else {
        rmsnorm_launch(resid1, f32(w->norm2_weight), normed, rows, E);
        gemm(normed, f32(w->ffn_up_w), up, rows, E, Hd);
        gemm(normed, f32(w->ffn_gate_w), gate, rows, E, Hd);
        swiglu_launch(gate, up, gate, rows * Hd);
    }
    gemm(gate, f32(w->ffn_down_w), rows_out, rows, Hd, E, resid1); /* projection + residual */
    HIP_CHECK_LAUNCH("blt_kv_decode_layer");
}
