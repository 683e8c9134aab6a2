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
#include "cross_rows_device.h"
#include "rope_device.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <vector>

namespace {

constexpr float RMSNORM_EPS = 1e-6f; /* csrc/ops/reductions_cpu.c:325 */

/* `parts` lanes (a power of two, 8..64) share a row's loads (coalesced, into
 * LDS), one of them then walks the row in element order.  256 / parts rows
 * per workgroup.
 * VEC (dim a multiple of 4, 16-byte aligned pointers): a lane moves float4s, four requests in
 * flight; with the trip count unknown at compile time the scalar loops wait for memory once per
 * element instead. */
template <bool VEC>
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
    const uint32_t quads = dim / 4u;
    if constexpr (VEC) {
        const float4 *src4 = reinterpret_cast<const float4 *>(src);
        float4 *st4 = reinterpret_cast<float4 *>(stage + r_local * pitch);
        for (uint32_t j = part; j < quads; j += 4u * parts) {
            float4 t[4];
#pragma unroll
            for (uint32_t u = 0; u < 4u; u++) t[u] = src4[min(j + u * parts, quads - 1u)];
#pragma unroll
            for (uint32_t u = 0; u < 4u; u++)
                if (j + u * parts < quads) st4[j + u * parts] = t[u];
        }
    } else {
        for (uint32_t j = part; j < dim; j += parts) stage[r_local * pitch + j] = src[j];
    }
    float4 w_first[4]; /* the weights of the first round of stores, requested before the row walk */
    if constexpr (VEC) {
#pragma unroll
        for (uint32_t u = 0; u < 4u; u++)
            w_first[u] = reinterpret_cast<const float4 *>(w)[min(part + u * parts, quads - 1u)];
    }
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
    if constexpr (VEC) {
        const float4 *w4 = reinterpret_cast<const float4 *>(w);
        const float4 *st4 = reinterpret_cast<const float4 *>(stage + r_local * pitch);
        float4 *dst4 = reinterpret_cast<float4 *>(dst);
        for (uint32_t j = part; j < quads; j += 4u * parts) {
            float4 wv[4];
#pragma unroll
            for (uint32_t u = 0; u < 4u; u++) wv[u] = j == part ? w_first[u] : w4[min(j + u * parts, quads - 1u)];
#pragma unroll
            for (uint32_t u = 0; u < 4u; u++) {
                if (j + u * parts >= quads) continue;
                const float4 v = st4[j + u * parts];
                float4 o;
                o.x = v.x * inv_rms * wv[u].x, o.y = v.y * inv_rms * wv[u].y;
                o.z = v.z * inv_rms * wv[u].z, o.w = v.w * inv_rms * wv[u].w;
                dst4[j + u * parts] = o;
            }
        }
    } else {
        for (uint32_t j = part; j < dim; j += parts) dst[j] = stage[r_local * pitch + j] * inv_rms * w[j];
    }
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
    const bool vec = dim % 4u == 0u && (((uintptr_t)x | (uintptr_t)w | (uintptr_t)out) & 15u) == 0u;
    const dim3 grid((uint32_t)((rows + rpw - 1u) / rpw));
    if (vec)
        blt_launch("rmsnorm_rows", rmsnorm_rows_kernel<true>, grid, dim3(256), lds, 0, x, w, out, (uint32_t)rows,
                   (uint32_t)dim, parts);
    else
        blt_launch("rmsnorm_rows", rmsnorm_rows_kernel<false>, grid, dim3(256), lds, 0, x, w, out, (uint32_t)rows,
                   (uint32_t)dim, parts);
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

/* The decoder step and layer take their projections on the matrix cores whatever the row count
 * (fp32 tolerance, as they always did above 32 rows).  BLT_HIP_EXACT_STEP=1 keeps the exact
 * thread-per-column kernel for steps of up to 32 rows (results bit-identical to the CPU
 * reference, about 1.5 times the time). */
uint32_t step_tolerant() {
    static const uint32_t on = [] {
        const char *e = getenv("BLT_HIP_EXACT_STEP");
        return (e && atoi(e) == 1) ? 0u : 1u;
    }();
    return on;
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
    g.tolerant = step_tolerant();
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

namespace {

/* Prompt prefill through the step: `n` (> 32) new rows per sequence, causal.  The step kernels take
 * 32 rows at a time, one slice after the other with few workgroups each; here the rows are staged
 * once -- Q rotated into a scratch buffer, K rotated and V written through to the slabs, one small
 * launch -- and the attention of all of them runs as one batch of (sequence, head) problems of the
 * prefill kernels with the causal diagonal moved by the cached length (csrc/infer/kv_cache.c:
 * 229-236: j <= base + r, base + r - j < window).  Needs the lengths on the host. */
__global__ __launch_bounds__(256) void kv_chunk_stage_kernel(const float *__restrict__ qkv, float *__restrict__ q_rot,
                                                             float *__restrict__ cache_k, float *__restrict__ cache_v,
                                                             const uint32_t *__restrict__ self_len,
                                                             const float *__restrict__ rope_cos,
                                                             const float *__restrict__ rope_sin, uint32_t n, uint32_t E,
                                                             uint32_t hd, uint64_t max_seq_len) {
    const uint32_t row = blockIdx.x, b = row / n, r = row % n;
    const uint32_t pos = self_len[b] + r;
    const float *src = qkv + (size_t)row * 3u * E;
    float *kd = cache_k + ((size_t)b * max_seq_len + pos) * E;
    float *vd = cache_v + ((size_t)b * max_seq_len + pos) * E;
    for (uint32_t col = 4u * threadIdx.x; col < E; col += 1024u) {
        const size_t at = (size_t)pos * (hd / 2u) + (col % hd) / 2u;
        const float4 q4 = *reinterpret_cast<const float4 *>(src + col);
        const float4 k4 = *reinterpret_cast<const float4 *>(src + E + col);
        *reinterpret_cast<float4 *>(q_rot + (size_t)row * E + col) = rope_rotate4(q4, rope_cos + at, rope_sin + at);
        *reinterpret_cast<float4 *>(kd + col) = rope_rotate4(k4, rope_cos + at, rope_sin + at);
        *reinterpret_cast<float4 *>(vd + col) = *reinterpret_cast<const float4 *>(src + 2u * E + col);
    }
}

void long_chunk_attention(const blt_kv_attn_cache *cache, const float *qkv, const float *rope_cos,
                          const float *rope_sin, size_t rope_positions, size_t n, const size_t *host_base,
                          float *combined, blt_arena *arena) {
    const size_t E = cache->embed_dim, H = cache->num_heads, hd = E / H, rows = cache->batch * n;
    float *q_rot = (float *)blt_arena_alloc(arena, rows * E * sizeof(float), 64);
    for (size_t b = 0; b < cache->batch; b++)
        BLT_REQUIRE(host_base[b] + n <= rope_positions && host_base[b] + n <= cache->max_seq_len,
                    "blt_kv_decode_step: positions exceed the rotary tables or the cache");
    blt_launch("kv_chunk_stage", kv_chunk_stage_kernel, dim3((unsigned)rows), dim3(256), 0, 0, qkv, q_rot, cache->self_k,
               cache->self_v, cache->self_len, rope_cos, rope_sin, (uint32_t)n, (uint32_t)E, (uint32_t)hd,
               (uint64_t)cache->max_seq_len);
    std::vector<blt_attention_problem> pr(cache->batch * H);
    const float scale = 1.0f / sqrtf((float)hd);
    for (size_t b = 0; b < cache->batch; b++) {
        for (size_t head = 0; head < H; head++) {
            blt_attention_problem &p = pr[b * H + head];
            std::memset(&p, 0, sizeof(p));
            p.head.q = q_rot + b * n * E + head * hd;
            p.head.k = cache->self_k + b * cache->max_seq_len * E + head * hd;
            p.head.v = cache->self_v + b * cache->max_seq_len * E + head * hd;
            p.head.q_stride = p.head.k_stride = p.head.v_stride = E;
            p.head.combined = combined + b * n * E;
            p.head.combined_stride = E;
            p.head.combined_col_offset = head * hd;
            p.head.nq = n;
            p.head.nk = host_base[b] + n;
            p.head.head_dim = hd;
            p.head.scale = scale;
            p.mask_kind = BLT_ATTN_MASK_CAUSAL;
            p.causal_offset = host_base[b];
            p.window = cache->window;
        }
    }
    blt_attention_batch_hip(pr.data(), pr.size());
}

/* Q and K column blocks of packed [rows, 3E] projection rows rotated in place, row R at the
 * position positions[R] (block rows carry their own positions, csrc/models/block_diffusion.c:
 * 148-157; the arithmetic of csrc/ops/reductions_cpu.c:219-226). */
__global__ __launch_bounds__(256) void rope_rows_at_kernel(float *__restrict__ qkv, const uint32_t *__restrict__ positions,
                                                           const float *__restrict__ rope_cos,
                                                           const float *__restrict__ rope_sin, uint32_t E, uint32_t hd) {
    const uint32_t row = blockIdx.x;
    const uint32_t pos = positions[row];
    float *src = qkv + (size_t)row * 3u * E;
    for (uint32_t col = 4u * threadIdx.x; col < 2u * E; col += 1024u) { /* Q block, then K block */
        const size_t at = (size_t)pos * (hd / 2u) + (col % hd) / 2u;
        float4 *cell = reinterpret_cast<float4 *>(src + col);
        *cell = rope_rotate4(*cell, rope_cos + at, rope_sin + at);
    }
}

/* host_base: the sequences' lengths where the caller keeps them (NULL: device lengths in
 * cache->self_len); they then travel in the step kernels' arguments.  dev_positions: device array
 * [rows] of rotary positions when they are not base + r (NULL otherwise). */
void decode_layer_impl(const blt_kv_attn_cache *cache, const blt_transformer_weights *w, const float *rows_in,
                       float *rows_out, const float *rope_cos, const float *rope_sin, size_t rope_positions, size_t n,
                       int step_kind, int commit, size_t max_len_hint, blt_arena *arena, const size_t *host_base,
                       const uint32_t *dev_positions = nullptr) {
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
    probe.tolerant = step_tolerant();
    /* self-attention block, kv_cache.c:326-394 */
    probe.n = (uint32_t)(3 * E);
    if (matmul_takes_norm(probe)) {
        gemm(rows_in, f32(w->attn_qkv_w), qkv, rows, E, 3 * E, nullptr, nullptr, f32(w->norm1_weight));
    } else {
        rmsnorm_launch(rows_in, f32(w->norm1_weight), normed, rows, E);
        gemm(normed, f32(w->attn_qkv_w), qkv, rows, E, 3 * E);
    }
    if (host_base != nullptr && n > 32 && step_kind == BLT_KV_STEP_CAUSAL && commit == 0 && dev_positions == nullptr &&
        (E / cache->num_heads) % 4 == 0) {
        long_chunk_attention(cache, qkv, rope_cos, rope_sin, rope_positions, n, host_base, combined, arena);
    } else if (host_base != nullptr && commit == 0) {
        /* the caller keeps the lengths: they go into the kernel arguments */
        std::vector<uint32_t> lens(cache->batch);
        for (size_t b = 0; b < cache->batch; b++) lens[b] = (uint32_t)host_base[b];
        if (dev_positions != nullptr) { /* rows rotated at their own positions first, then a plain step */
            BLT_REQUIRE((E / cache->num_heads) % 4 == 0, "blt_kv_block_step: explicit row positions need head_dim %% 4 == 0");
            blt_launch("rope_rows_at", rope_rows_at_kernel, dim3((unsigned)rows), dim3(256), 0, 0, qkv, dev_positions,
                       rope_cos, rope_sin, (uint32_t)E, (uint32_t)(E / cache->num_heads));
            blt_kv_attend_step_lens_hip(cache, lens.data(), qkv, 3 * E, qkv + E, 3 * E, qkv + 2 * E, 3 * E, nullptr,
                                        nullptr, 0, combined, E, n, step_kind);
        } else {
            blt_kv_attend_step_lens_hip(cache, lens.data(), qkv, 3 * E, qkv + E, 3 * E, qkv + 2 * E, 3 * E, rope_cos,
                                        rope_sin, rope_positions, combined, E, n, step_kind);
        }
    } else {
        blt_kv_rope_attend_step_hip(cache, qkv, 3 * E, qkv + E, 3 * E, qkv + 2 * E, 3 * E, rope_cos, rope_sin,
                                    rope_positions, combined, E, n, step_kind, commit, max_len_hint);
    }
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

} // namespace

extern "C" void blt_kv_decode_layer_hip(const blt_kv_attn_cache *cache, const blt_transformer_weights *w,
                                        const float *rows_in, float *rows_out, const float *rope_cos,
                                        const float *rope_sin, size_t rope_positions, size_t n, int step_kind,
                                        int commit, size_t max_len_hint, blt_arena *arena) {
    decode_layer_impl(cache, w, rows_in, rows_out, rope_cos, rope_sin, rope_positions, n, step_kind, commit,
                      max_len_hint, arena, nullptr);
}

/* ===================================================================== */
/* The whole incremental decoder step (csrc/infer/kv_cache.c:112-416)     */
/* ===================================================================== */
namespace {

struct CrossRowsArgs {
    const float *q;     /* [rows, E] projected queries                               */
    const float *k;     /* tier-2 slabs [batch*slab_rows, E]                         */
    const float *v;
    float *out;         /* [rows, E] combined                                        */
    const uint32_t *lo; /* [rows] first visible sub-token of the row's own slab      */
    const uint32_t *hi; /* [rows] one past the last                                  */
    uint32_t n;         /* new rows per sequence: row R belongs to sequence R / n    */
    uint32_t E, xhd;
    uint64_t slab_rows;
    float scale;
};

/* One wave per (new row, head), see cross_rows_device.h. */
__global__ __launch_bounds__(64) void kv_cross_rows_kernel(CrossRowsArgs a) {
    const uint32_t R = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const uint32_t seq = R / a.n;
    cross_row_head(a.q + (size_t)R * a.E + head * a.xhd, a.k + (size_t)seq * a.slab_rows * a.E + head * a.xhd,
                   a.v + (size_t)seq * a.slab_rows * a.E + head * a.xhd, a.lo[R], a.hi[R], a.E, a.xhd, a.scale,
                   a.out + (size_t)R * a.E + head * a.xhd, lane);
}

bool cross_fires(const blt_local_decoder_config *c, size_t layer) {
    switch (c->cross_attn_placement) { /* csrc/models/local_common.c:49-64 */
    case BLT_XATTN_NONE: return false;
    case BLT_XATTN_LAST: return layer + 1 == c->num_layers;
    case BLT_XATTN_ALL: return true;
    case BLT_XATTN_FIRST: return layer == 0;
    default: return c->cross_attn_all_layers || layer + 1 == c->num_layers;
    }
}

void check_vec(const blt_tensor &t, size_t dim, const char *what) {
    BLT_REQUIRE(t.data != NULL && t.ndim == 1 && t.shape[0] == dim && t.dtype == BLT_DTYPE_FP32 &&
                    t.backend == BLT_BACKEND_HIP,
                "%s", what);
}

/* The step for `batch` sequences with n new rows each: base[b] is sequence b's
 * valid length, group[b*n + r] the latent patch of its row r.  Lengths and
 * group ranges travel to the device in one staged copy. */
/* step_kind / window: BLT_KV_STEP_CAUSAL with the decoder's local window for the incremental step;
 * the diffusion forward runs its clean rows causally without a window and its block rows as
 * BLT_KV_STEP_BLOCK.  positions (host, [batch*n]) when a row's rotary position is not base + r. */
void decode_step_run(const blt_kv_cache *cache, size_t batch, size_t n, const size_t *base, const size_t *group,
                     const float *d0_rows, float *logits, blt_arena *arena, int step_kind = BLT_KV_STEP_CAUSAL,
                     size_t window = SIZE_MAX, const size_t *positions = nullptr) {
    const blt_local_decoder *dec = cache->decoder;
    const blt_local_decoder_config *cfg = &dec->config;
    const size_t E = cache->embed_dim, L = cfg->num_layers, H = cfg->num_heads, XH = cfg->cross_attn_heads;
    const size_t V = cfg->vocab_size, rows = batch * n, hd = E / H, xhd = E / XH;
    BLT_REQUIRE(xhd <= 256, "blt_kv_decode_step: cross-attention heads wider than 256 columns are not supported");
    check_weight(&dec->lm_head_weight, E, V, "blt_kv_decode_step: lm_head_weight must be [embed_dim, vocab_size]");
    check_weight(&dec->rope_cos_cache, cfg->max_seq_len, hd / 2,
                 "blt_kv_decode_step: rope_cos_cache must be [max_seq_len, head_dim/2]");
    check_weight(&dec->rope_sin_cache, cfg->max_seq_len, hd / 2,
                 "blt_kv_decode_step: rope_sin_cache must be [max_seq_len, head_dim/2]");

    /* lengths, then lo / hi of every row's sub-token range, in one upload */
    bool own_positions = false; /* any row whose rotary position is not base + r */
    if (positions != nullptr)
        for (size_t b = 0; b < batch; b++)
            for (size_t r = 0; r < n; r++) {
                BLT_REQUIRE(positions[b * n + r] < cfg->max_seq_len, "rope_position_gather: position index out of range");
                own_positions = own_positions || positions[b * n + r] != base[b] + r;
            }
    std::vector<uint32_t> host(batch + 2 * rows + (own_positions ? rows : 0));
    if (own_positions)
        for (size_t i = 0; i < rows; i++) host[batch + 2 * rows + i] = (uint32_t)positions[i];
    size_t max_total = 0;
    for (size_t b = 0; b < batch; b++) {
        host[b] = (uint32_t)base[b];
        max_total = std::max(max_total, base[b] + n);
        for (size_t r = 0; r < n; r++) {
            host[batch + b * n + r] = (uint32_t)(group[b * n + r] * cache->k);
            host[batch + rows + b * n + r] = (uint32_t)((group[b * n + r] + 1) * cache->k);
        }
    }
    uint32_t *dev = (uint32_t *)blt_arena_alloc(arena, host.size() * sizeof(uint32_t), 64);
    blt_upload_staged(dev, host.data(), host.size() * sizeof(uint32_t));

    float *ping = (float *)blt_arena_alloc(arena, rows * E * sizeof(float), 64);
    float *pong = (float *)blt_arena_alloc(arena, rows * E * sizeof(float), 64);
    float *mid = (float *)blt_arena_alloc(arena, rows * E * sizeof(float), 64);
    float *xq = (float *)blt_arena_alloc(arena, rows * E * sizeof(float), 64);
    float *xnorm = (float *)blt_arena_alloc(arena, rows * E * sizeof(float), 64);
    float *xcomb = (float *)blt_arena_alloc(arena, rows * E * sizeof(float), 64);
    const size_t arena_mark = arena->offset;

    const float *cur = d0_rows;
    for (size_t l = 0; l < L; l++) {
        const blt_local_layer_storage *s = &dec->layers[l];
        const float *in = cur;
        if (cross_fires(cfg, l)) { /* kv_cache.c:303-341 */
            check_vec(s->cross_norm_weight, E, "blt_kv_decode_step: cross_norm_weight must be [embed_dim] FP32");
            check_weight(&s->cross_weight_q, E, E, "blt_kv_decode_step: cross_weight_q must be [embed_dim, embed_dim]");
            check_weight(&s->cross_weight_proj, E, E,
                         "blt_kv_decode_step: cross_weight_proj must be [embed_dim, embed_dim]");
            MatmulArgs probe;
            std::memset(&probe, 0, sizeof(probe));
            probe.m = (uint32_t)rows, probe.k = (uint32_t)E, probe.n = (uint32_t)E;
            probe.cross_head_dim = (uint32_t)xhd;
            probe.tolerant = step_tolerant();
            if (matmul_takes_norm(probe) && matmul_takes_cross(probe)) {
                /* norm, Q projection and the rows' cross attention in one launch: with more than 32
                 * rows a 32x32 tile of the projection is one 32-wide head of 32 rows; up to 32 rows
                 * one workgroup of the exact kernel holds the whole projected rows */
                MatmulArgs g;
                std::memset(&g, 0, sizeof(g));
                g.a = cur, g.b = (const float *)s->cross_weight_q.data, g.out = xq;
                g.norm_w = (const float *)s->cross_norm_weight.data;
                g.m = (uint32_t)rows, g.k = (uint32_t)E, g.n = (uint32_t)E;
                g.lda = g.ldb = g.ldo = (uint32_t)E;
                g.cross_k = (const float *)cache->cross_k[l].data, g.cross_v = (const float *)cache->cross_v[l].data;
                g.cross_out = xcomb, g.cross_lo = dev + batch, g.cross_hi = dev + batch + rows;
                g.cross_rows_per_seq = (uint32_t)n, g.cross_slab_rows = (uint32_t)cache->max_subtokens;
                g.cross_scale = 1.0f / sqrtf((float)xhd), g.cross_head_dim = (uint32_t)xhd;
                g.tolerant = step_tolerant();
                matmul_f32_launch(g, 0);
            } else {
            if (matmul_takes_norm(probe)) {
                gemm(cur, (const float *)s->cross_weight_q.data, xq, rows, E, E, nullptr, nullptr,
                     (const float *)s->cross_norm_weight.data);
            } else {
                rmsnorm_launch(cur, (const float *)s->cross_norm_weight.data, xnorm, rows, E);
                gemm(xnorm, (const float *)s->cross_weight_q.data, xq, rows, E, E);
            }
            CrossRowsArgs c;
            c.q = xq;
            c.k = (const float *)cache->cross_k[l].data;
            c.v = (const float *)cache->cross_v[l].data;
            c.out = xcomb;
            c.lo = dev + batch, c.hi = dev + batch + rows;
            c.n = (uint32_t)n, c.E = (uint32_t)E, c.xhd = (uint32_t)xhd;
            c.slab_rows = cache->max_subtokens;
            c.scale = 1.0f / sqrtf((float)xhd);
            blt_launch("kv_cross_rows", kv_cross_rows_kernel, dim3((unsigned)rows, (unsigned)XH), dim3(64), 0, 0, c);
            }
            gemm(xcomb, (const float *)s->cross_weight_proj.data, mid, rows, E, E, cur); /* + residual */
            in = mid;
        }
        blt_kv_attn_cache view;
        view.self_k = (float *)cache->self_k[l].data;
        view.self_v = (float *)cache->self_v[l].data;
        view.self_len = dev;
        view.batch = batch;
        view.max_seq_len = cache->max_seq_len;
        view.embed_dim = E;
        view.num_heads = H;
        view.window = window == SIZE_MAX ? cfg->local_window : window;
        blt_transformer_weights w;
        std::memset(&w, 0, sizeof(w));
        w.norm1_weight = &s->norm1_weight, w.attn_qkv_w = &s->attn_qkv_w, w.attn_proj_w = &s->attn_proj_w;
        w.norm2_weight = &s->norm2_weight, w.ffn_up_w = &s->ffn_up_w, w.ffn_gate_w = &s->ffn_gate_w;
        w.ffn_down_w = &s->ffn_down_w;
        float *next = (cur == ping) ? pong : ping;
        arena->offset = arena_mark; /* the layer's work buffers are reused by the next layer */
        decode_layer_impl(&view, &w, in, next, (const float *)dec->rope_cos_cache.data,
                          (const float *)dec->rope_sin_cache.data, cfg->max_seq_len, n, step_kind, 0, max_total, arena,
                          base, own_positions ? dev + batch + 2 * rows : nullptr);
        cur = next;
    }
    gemm(cur, (const float *)dec->lm_head_weight.data, logits, rows, E, V); /* kv_cache.c:416 */
    HIP_CHECK_LAUNCH("blt_kv_decode_step");
}

void check_cache(const blt_kv_cache *cache, const char *fn) {
    BLT_REQUIRE(cache != NULL && cache->decoder != NULL, "%s: cache cannot be NULL", fn);
    const blt_local_decoder_config *cfg = &cache->decoder->config;
    BLT_REQUIRE(cfg->num_heads != 0 && cfg->cross_attn_heads != 0 && cache->embed_dim == cfg->embed_dim &&
                    cfg->embed_dim % cfg->num_heads == 0 && cfg->embed_dim % cfg->cross_attn_heads == 0,
                "%s: decoder configuration is inconsistent", fn);
    BLT_REQUIRE(cache->self_k != NULL && cache->self_v != NULL && cache->cross_k != NULL && cache->cross_v != NULL,
                "%s: cache tiers are missing", fn);
    for (size_t l = 0; l < cfg->num_layers; l++)
        BLT_REQUIRE(cache->self_k[l].backend == BLT_BACKEND_HIP && cache->cross_k[l].backend == BLT_BACKEND_HIP,
                    "%s: HIP implementation called with a cache that is not in device memory", fn);
}

void refresh_cross_seq(blt_kv_cache *cache, size_t seq, const blt_tensor *patch_in, const blt_patch_info *patches,
                       size_t num_patches, size_t from_patch) {
    const blt_local_decoder *dec = cache->decoder;
    const size_t E = cache->embed_dim, L = dec->config.num_layers;
    const size_t first = from_patch * cache->k, count = (num_patches - from_patch) * cache->k;
    for (size_t l = 0; l < L; l++) {
        if (!cross_fires(&dec->config, l)) continue;
        const blt_local_layer_storage *s = &dec->layers[l];
        check_weight(&s->cross_weight_k, E, E, "blt_kv_cache_refresh_cross: cross_weight_k must be [embed_dim, embed_dim]");
        check_weight(&s->cross_weight_v, E, E, "blt_kv_cache_refresh_cross: cross_weight_v must be [embed_dim, embed_dim]");
        const size_t row0 = seq * cache->max_subtokens + first;
        MatmulArgs g;
        std::memset(&g, 0, sizeof(g));
        g.a = (const float *)patch_in->data + first * E;
        g.b = (const float *)s->cross_weight_k.data;
        g.out = (float *)cache->cross_k[l].data + row0 * E;
        g.m = (uint32_t)count, g.k = (uint32_t)E, g.n = (uint32_t)E;
        g.lda = g.ldb = g.ldo = (uint32_t)E;
        g.b2 = (const float *)s->cross_weight_v.data;
        g.out2 = (float *)cache->cross_v[l].data + row0 * E;
        g.tolerant = step_tolerant();
        if (matmul_takes_gated(g)) { /* K and V in one pass over the patch rows */
            matmul_f32_launch(g, 0);
        } else {
            g.b2 = nullptr, g.out2 = nullptr;
            matmul_f32_launch(g, 0);
            g.b = (const float *)s->cross_weight_v.data;
            g.out = (float *)cache->cross_v[l].data + row0 * E;
            matmul_f32_launch(g, 0);
        }
    }
    std::memcpy(&cache->cached_patches[seq * cache->max_seq_len + from_patch], &patches[from_patch],
                (num_patches - from_patch) * sizeof(blt_patch_info)); /* kv_cache.c:154-157 */
    HIP_CHECK_LAUNCH("blt_kv_cache_refresh_cross");
}

void check_refresh_args(const blt_kv_cache *cache, const blt_tensor *patch_in, const blt_patch_info *patches,
                        size_t num_patches, size_t from_patch, const blt_arena *arena) {
    BLT_REQUIRE(patch_in != NULL && patches != NULL && arena != NULL,
                "blt_kv_cache_refresh_cross: arguments cannot be NULL");
    BLT_REQUIRE(num_patches >= 1 && from_patch < num_patches,
                "blt_kv_cache_refresh_cross: need from_patch < num_patches");
    BLT_REQUIRE(patch_in->data != NULL && patch_in->ndim == 2 && patch_in->shape[0] == num_patches &&
                    patch_in->shape[1] == cache->patch_dim && patch_in->dtype == BLT_DTYPE_FP32,
                "blt_kv_cache_refresh_cross: patch_in must be [num_patches, patch_dim] FP32");
    BLT_REQUIRE(patch_in->backend == BLT_BACKEND_HIP,
                "blt_kv_cache_refresh_cross: HIP implementation called with a non-HIP tensor");
    BLT_REQUIRE(num_patches * cache->k <= cache->max_subtokens,
                "blt_kv_cache_refresh_cross: sub-token count exceeds cache capacity");
}

} // namespace

extern "C" void blt_kv_cache_refresh_cross_hip(blt_kv_cache *cache, const blt_tensor *patch_in,
                                               const blt_patch_info *patches, size_t num_patches, size_t from_patch,
                                               blt_arena *arena) {
    check_cache(cache, "blt_kv_cache_refresh_cross");
    check_refresh_args(cache, patch_in, patches, num_patches, from_patch, arena);
    BLT_REQUIRE(from_patch <= cache->cross_num_patches,
                "blt_kv_cache_refresh_cross: from_patch must not skip uncached patches "
                "(truncate to the LCP first)");
    refresh_cross_seq(cache, 0, patch_in, patches, num_patches, from_patch);
    cache->cross_num_patches = num_patches;
}

extern "C" void blt_kv_cache_refresh_cross_seq_hip(blt_kv_cache *cache, size_t seq, const blt_tensor *patch_in,
                                                   const blt_patch_info *patches, size_t num_patches,
                                                   size_t from_patch, blt_arena *arena) {
    check_cache(cache, "blt_kv_cache_refresh_cross");
    BLT_REQUIRE(seq < cache->batch_size, "blt_kv_cache_refresh_cross: sequence index out of range");
    check_refresh_args(cache, patch_in, patches, num_patches, from_patch, arena);
    refresh_cross_seq(cache, seq, patch_in, patches, num_patches, from_patch);
}

namespace {

/* blt_patch_decoder_latent_at (csrc/ops/patch_pool_cpu.c:114-131) for the consecutive positions
 * base .. base + n - 1: when the table tiles its range (each patch starts where the previous one
 * ends, the only kind the model builds) the owner only moves forward, so one walk serves all rows;
 * any other table goes row by row through the general rule. */
void latent_ids(const blt_patch_info *patches, size_t num_patches, size_t base, size_t n, size_t *out) {
    bool tiling = n > 4; /* a few rows: the general rule's own scan is as short as the check below */
    for (size_t p = 0; p < num_patches && tiling; p++)
        tiling = patches[p].length >= 1 &&
                 (p + 1 == num_patches || patches[p + 1].start_idx == patches[p].start_idx + patches[p].length);
    if (!tiling) {
        for (size_t r = 0; r < n; r++) out[r] = blt_patch_decoder_latent_at(patches, num_patches, base + r);
        return;
    }
    size_t p = 0;
    for (size_t r = 0; r < n; r++) {
        const size_t pos = base + r;
        if (pos < patches[0].start_idx) {
            out[r] = 0;
            continue;
        }
        while (p < num_patches && pos >= patches[p].start_idx + patches[p].length) p++;
        if (p == num_patches) {
            out[r] = num_patches - 1; /* past the last patch */
            continue;
        }
        const bool closes = pos - patches[p].start_idx + 1 == patches[p].length;
        out[r] = (closes && p + 1 < num_patches) ? p : (p == 0 ? 0 : p - 1);
    }
}

} // namespace

extern "C" void blt_kv_decode_step_hip(blt_kv_cache *cache, const blt_tensor *patch_in, const blt_patch_info *patches,
                                       size_t num_patches, const blt_tensor *d0_rows, int trailing_closed,
                                       blt_tensor *logits_out, blt_arena *arena) {
    check_cache(cache, "blt_kv_decode_step");
    const blt_local_decoder_config *cfg = &cache->decoder->config;
    const size_t E = cache->embed_dim, V = cfg->vocab_size, hd = E / cfg->num_heads;
    BLT_REQUIRE(hd > 0 && hd % 2 == 0, "blt_kv_decode_step: RoPE requires an even head_dim");
    BLT_REQUIRE(patch_in != NULL && patches != NULL && d0_rows != NULL && logits_out != NULL && arena != NULL,
                "blt_kv_decode_step: arguments cannot be NULL");
    BLT_REQUIRE(arena->backend == BLT_BACKEND_HIP, "blt_kv_decode_step: HIP implementation needs a device arena");
    BLT_REQUIRE(num_patches >= 1 && num_patches == cache->cross_num_patches,
                "blt_kv_decode_step: tier-2 cache must cover all patches (refresh first)");
    BLT_REQUIRE(d0_rows->data != NULL && d0_rows->ndim == 2 && d0_rows->shape[1] == E &&
                    d0_rows->dtype == BLT_DTYPE_FP32,
                "blt_kv_decode_step: d0_rows must be [n, embed_dim] FP32");
    BLT_REQUIRE(d0_rows->backend == BLT_BACKEND_HIP, "blt_kv_decode_step: HIP implementation called with a non-HIP tensor");
    const size_t n = d0_rows->shape[0];
    BLT_REQUIRE(n >= 1, "blt_kv_decode_step: need at least one row");
    const size_t base = cache->self_len, total = base + n;
    BLT_REQUIRE(total <= cache->max_seq_len, "blt_kv_decode_step: exceeds cache capacity");
    BLT_REQUIRE(logits_out->data != NULL && logits_out->ndim == 2 && logits_out->shape[0] == n &&
                    logits_out->shape[1] == V && logits_out->dtype == BLT_DTYPE_FP32 &&
                    logits_out->backend == BLT_BACKEND_HIP,
                "blt_kv_decode_step: logits_out must be [n, vocab_size] FP32");
    BLT_REQUIRE(num_patches * cache->k <= cache->max_subtokens,
                "blt_kv_decode_step: sub-token count exceeds cache capacity");
    std::vector<size_t> group(n); /* kv_cache.c:199-213 */
    latent_ids(patches, num_patches, base, n, group.data());
    if (trailing_closed) group[n - 1] = num_patches - 1;
    decode_step_run(cache, 1, n, &base, group.data(), (const float *)d0_rows->data, (float *)logits_out->data, arena);
    cache->self_len = total;
}

extern "C" void blt_kv_decode_step_batched_hip(blt_kv_cache *cache, size_t *self_len,
                                               const blt_patch_info *const *patches, const size_t *num_patches,
                                               const int *trailing_closed, const blt_tensor *d0_rows,
                                               blt_tensor *logits_out, blt_arena *arena) {
    check_cache(cache, "blt_kv_decode_step_batched");
    const blt_local_decoder_config *cfg = &cache->decoder->config;
    const size_t E = cache->embed_dim, V = cfg->vocab_size, hd = E / cfg->num_heads, batch = cache->batch_size;
    BLT_REQUIRE(hd > 0 && hd % 2 == 0, "blt_kv_decode_step_batched: RoPE requires an even head_dim");
    BLT_REQUIRE(self_len != NULL && patches != NULL && num_patches != NULL && d0_rows != NULL && logits_out != NULL &&
                    arena != NULL,
                "blt_kv_decode_step_batched: arguments cannot be NULL");
    BLT_REQUIRE(arena->backend == BLT_BACKEND_HIP, "blt_kv_decode_step_batched: HIP implementation needs a device arena");
    BLT_REQUIRE(d0_rows->data != NULL && d0_rows->ndim == 2 && d0_rows->shape[1] == E &&
                    d0_rows->dtype == BLT_DTYPE_FP32 && d0_rows->backend == BLT_BACKEND_HIP,
                "blt_kv_decode_step_batched: d0_rows must be [batch*n, embed_dim] FP32 in device memory");
    BLT_REQUIRE(batch >= 1 && d0_rows->shape[0] >= batch && d0_rows->shape[0] % batch == 0,
                "blt_kv_decode_step_batched: d0_rows must hold the same number n >= 1 of rows for every sequence");
    const size_t n = d0_rows->shape[0] / batch;
    BLT_REQUIRE(logits_out->data != NULL && logits_out->ndim == 2 && logits_out->shape[0] == batch * n &&
                    logits_out->shape[1] == V && logits_out->dtype == BLT_DTYPE_FP32 &&
                    logits_out->backend == BLT_BACKEND_HIP,
                "blt_kv_decode_step_batched: logits_out must be [batch*n, vocab_size] FP32 in device memory");
    std::vector<size_t> group(batch * n);
    for (size_t b = 0; b < batch; b++) {
        BLT_REQUIRE(patches[b] != NULL && num_patches[b] >= 1,
                    "blt_kv_decode_step_batched: every sequence needs at least one patch");
        BLT_REQUIRE(self_len[b] + n <= cache->max_seq_len, "blt_kv_decode_step_batched: exceeds cache capacity");
        BLT_REQUIRE(num_patches[b] * cache->k <= cache->max_subtokens,
                    "blt_kv_decode_step_batched: sub-token count exceeds cache capacity");
        latent_ids(patches[b], num_patches[b], self_len[b], n, group.data() + b * n);
        if (trailing_closed != NULL && trailing_closed[b]) group[b * n + n - 1] = num_patches[b] - 1;
    }
    decode_step_run(cache, batch, n, self_len, group.data(), (const float *)d0_rows->data,
                    (float *)logits_out->data, arena);
    for (size_t b = 0; b < batch; b++) self_len[b] += n;
}

/* ===================================================================== */
/* Inference-mode diffusion forward (csrc/models/block_diffusion.c:776-795) */
/* ===================================================================== */
namespace {

/* D_0 rows of the block section (block_diffusion.c:137-146): zeros, or row tokens[r] of the
 * learned table (csrc/ops/gather_scatter_cpu.c:7-29). */
const float *block_d0_rows(const blt_local_decoder *dec, const blt_block_batch *batch, blt_d0_mode d0_mode,
                           blt_arena *arena) {
    const size_t E = dec->config.embed_dim, R = batch->n_block_rows;
    const size_t shape[2] = {R, E};
    if (d0_mode != BLT_D0_LEARNED) {
        blt_tensor zeros = blt_tensor_create(arena, shape, 2, BLT_DTYPE_FP32); /* zero-filled */
        return (const float *)zeros.data;
    }
    BLT_REQUIRE(batch->tokens != NULL, "forward_diffusion_infer: batch->tokens cannot be NULL with the learned D_0 table");
    BLT_REQUIRE(dec->d0_embed_weight.data != NULL, "forward_diffusion_infer: the decoder has no learned D_0 table");
    blt_tensor out = blt_tensor_create_uninit(arena, shape, 2, BLT_DTYPE_FP32);
    blt_embedding_lookup_hip(&dec->d0_embed_weight, batch->tokens, &out);
    return (const float *)out.data;
}

void check_block_batch(const blt_block_batch *batch, const char *fn) {
    BLT_REQUIRE(batch != NULL, "%s: arguments cannot be NULL", fn);
    BLT_REQUIRE(batch->n_block_rows >= 1 && batch->positions != NULL && batch->groups != NULL,
                "%s: the batch needs at least one block row with positions and groups", fn);
    BLT_REQUIRE(batch->n_block_rows <= 32,
                "%s: at most 32 block rows (csrc/infer/block_generation.c:154); the rows of a block all see each "
                "other, so the block cannot be cut",
                fn);
}

/* The block rows over a cache whose sequence 0 holds the clean prefix. */
void block_step_run(const blt_kv_cache *cache, size_t num_patches, const blt_block_batch *batch, blt_d0_mode d0_mode,
                    float *logits, blt_arena *arena) {
    const size_t base = batch->num_clean, R = batch->n_block_rows;
    for (size_t r = 0; r < R; r++)
        BLT_REQUIRE(batch->groups[r] < num_patches, "forward_diffusion_infer: a block row's latent group is out of range");
    const float *d0 = block_d0_rows(cache->decoder, batch, d0_mode, arena);
    decode_step_run(cache, 1, R, &base, batch->groups, d0, logits, arena, BLT_KV_STEP_BLOCK, 0, batch->positions);
}

} // namespace

extern "C" void blt_kv_block_step_hip(blt_kv_cache *cache, size_t num_patches, const blt_block_batch *batch,
                                      blt_d0_mode d0_mode, blt_tensor *logits_out, blt_arena *arena) {
    check_cache(cache, "blt_kv_block_step");
    check_block_batch(batch, "blt_kv_block_step");
    const blt_local_decoder_config *cfg = &cache->decoder->config;
    const size_t hd = cache->embed_dim / cfg->num_heads;
    BLT_REQUIRE(hd > 0 && hd % 2 == 0, "blt_kv_block_step: RoPE requires an even head_dim");
    BLT_REQUIRE(logits_out != NULL && arena != NULL, "blt_kv_block_step: arguments cannot be NULL");
    BLT_REQUIRE(arena->backend == BLT_BACKEND_HIP, "blt_kv_block_step: HIP implementation needs a device arena");
    BLT_REQUIRE(batch->num_clean == cache->self_len,
                "blt_kv_block_step: the cache holds %zu byte rows, the batch says %zu clean rows", cache->self_len,
                batch->num_clean);
    BLT_REQUIRE(num_patches >= 1 && num_patches == cache->cross_num_patches,
                "blt_kv_block_step: tier-2 cache must cover all patches (refresh first)");
    BLT_REQUIRE(cache->self_len + batch->n_block_rows <= cache->max_seq_len, "blt_kv_block_step: exceeds cache capacity");
    BLT_REQUIRE(logits_out->data != NULL && logits_out->ndim == 2 && logits_out->shape[0] == batch->n_block_rows &&
                    logits_out->shape[1] == cfg->vocab_size && logits_out->dtype == BLT_DTYPE_FP32 &&
                    logits_out->backend == BLT_BACKEND_HIP,
                "blt_kv_block_step: logits_out must be [n_block_rows, vocab_size] FP32 in device memory");
    block_step_run(cache, num_patches, batch, d0_mode, (float *)logits_out->data, arena);
}

extern "C" void blt_local_decoder_forward_diffusion_infer_hip(const blt_local_decoder *model,
                                                              const blt_tensor *byte_hidden_in,
                                                              const blt_tensor *patch_in, const blt_patch_info *patches,
                                                              size_t num_patches, const blt_block_batch *batch,
                                                              blt_d0_mode d0_mode, blt_tensor *logits_out,
                                                              blt_arena *arena) {
    BLT_REQUIRE(model != NULL && logits_out != NULL && arena != NULL && batch != NULL,
                "forward_diffusion_infer: arguments cannot be NULL");
    const blt_local_decoder_config *cfg = &model->config;
    const size_t E = cfg->embed_dim, V = cfg->vocab_size, L = cfg->num_layers;
    const size_t N = batch->num_clean, R = batch->n_block_rows, S = N + R;
    const size_t pdim = cfg->patch_dim ? cfg->patch_dim : E, k = pdim / E;
    BLT_REQUIRE(cfg->num_heads != 0 && E % cfg->num_heads == 0 && (E / cfg->num_heads) % 2 == 0,
                "diffusion: RoPE requires an even head_dim");
    BLT_REQUIRE(byte_hidden_in != NULL && patch_in != NULL && patches != NULL, "diffusion: arguments cannot be NULL");
    BLT_REQUIRE(arena->backend == BLT_BACKEND_HIP && byte_hidden_in->backend == BLT_BACKEND_HIP &&
                    patch_in->backend == BLT_BACKEND_HIP,
                "forward_diffusion_infer: HIP implementation called with a non-HIP tensor");
    BLT_REQUIRE(byte_hidden_in->ndim == 2 && byte_hidden_in->shape[0] == N && byte_hidden_in->shape[1] == E && N >= 1,
                "diffusion: byte_hidden_in must be [N, embed_dim]");
    BLT_REQUIRE(patch_in->ndim == 2 && patch_in->shape[0] == num_patches && patch_in->shape[1] == pdim && num_patches >= 1,
                "diffusion: patch_in must be [num_patches, patch_dim]");
    BLT_REQUIRE(S >= 2 && S <= cfg->max_seq_len, "diffusion: total sequence length outside [2, decoder max_seq_len]");
    check_block_batch(batch, "forward_diffusion_infer");
    BLT_REQUIRE(logits_out->data != NULL && logits_out->ndim == 2 && logits_out->shape[0] == S &&
                    logits_out->shape[1] == V && logits_out->dtype == BLT_DTYPE_FP32 &&
                    logits_out->backend == BLT_BACKEND_HIP,
                "forward_diffusion_infer: logits_out must be [N + n_block_rows, vocab_size] FP32");

    /* A clean row never sees a block row (csrc/ops/mask_builder_cpu.c:128-131), so the clean rows
     * are the incremental step over an empty cache -- causal, no window (the INFER mask has none),
     * the last row on the last latent when the patch is closed -- and the block rows are one block
     * step over what that step cached (133-135: all clean rows plus the whole block).  The cache
     * lives in the caller's arena like every other work buffer of this forward; nothing of it needs
     * clearing, every row that is read was written first. */
    std::vector<blt_tensor> tiers(4 * L);
    const size_t subtokens = num_patches * k;
    for (size_t l = 0; l < L; l++) {
        const size_t self_shape[2] = {S, E}, cross_shape[2] = {subtokens, E};
        tiers[0 * L + l] = blt_tensor_create_uninit(arena, self_shape, 2, BLT_DTYPE_FP32);
        tiers[1 * L + l] = blt_tensor_create_uninit(arena, self_shape, 2, BLT_DTYPE_FP32);
        tiers[2 * L + l] = blt_tensor_create_uninit(arena, cross_shape, 2, BLT_DTYPE_FP32);
        tiers[3 * L + l] = blt_tensor_create_uninit(arena, cross_shape, 2, BLT_DTYPE_FP32);
    }
    std::vector<blt_patch_info> table(num_patches);
    blt_kv_cache cache;
    std::memset(&cache, 0, sizeof(cache));
    cache.decoder = model;
    cache.max_seq_len = S, cache.batch_size = 1, cache.max_subtokens = subtokens;
    cache.embed_dim = E, cache.k = k, cache.patch_dim = pdim;
    cache.self_k = tiers.data(), cache.self_v = tiers.data() + L;
    cache.cross_k = tiers.data() + 2 * L, cache.cross_v = tiers.data() + 3 * L;
    cache.cached_patches = table.data();
    check_cache(&cache, "forward_diffusion_infer");

    /* refresh_cross_seq indexes the snapshot by seq * max_seq_len: sequence 0 */
    refresh_cross_seq(&cache, 0, patch_in, patches, num_patches, 0);
    cache.cross_num_patches = num_patches;

    std::vector<size_t> group(N); /* block_diffusion.c:163-172 */
    latent_ids(patches, num_patches, 0, N, group.data());
    if (batch->trailing_closed) group[N - 1] = num_patches - 1;
    const size_t zero = 0;
    float *logits = (float *)logits_out->data;
    decode_step_run(&cache, 1, N, &zero, group.data(), (const float *)byte_hidden_in->data, logits, arena,
                    BLT_KV_STEP_CAUSAL, 0);
    cache.self_len = N;
    block_step_run(&cache, num_patches, batch, d0_mode, logits + N * V, arena);
}
