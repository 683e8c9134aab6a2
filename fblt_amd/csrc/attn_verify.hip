/*
 * Block kernel of the KV-cache step: a block of n query rows per sequence
 * (BLT-D/DV draft and verify blocks, chunked prefill) against the cached
 * prefix plus the n new rows, on the fp32 matrix cores.
 *
 * Same split-KV frame as the decode kernel (a workgroup owns one contiguous
 * span of a sequence's keys, its waves are the heads, per-split softmax states
 * are merged by the last workgroup of the sequence), but the inner product of
 * a 32-key sub-chunk with all query rows of the block is one transposed MFMA
 * tile, exactly as in the prefill kernel:
 *
 *   S^T[key, query] = K Q^T      (32 x 32 x head_dim,  v_mfma_f32_32x32x2_f32)
 *   O^T[d,   query] += V^T P^T   (head_dim x 32 x 32)
 *
 * The block's query rows (at most 32) are the N dimension of both products,
 * so K and V stream through once for the whole block; rows beyond n are
 * padding and never stored.  K rows are read coalesced and turned into MFMA
 * fragments through a per-wave LDS tile; V rows are read one dword per lane
 * (32 lanes = one 128-byte row segment).  The kernel is HBM-bound: ~8*head_dim
 * bytes of K/V per 2*head_dim MFMAs of a sub-chunk.
 */
#include "blt_hip.h"
#include "blt_fatal.h"
#include "hip_check.h"
#include "attn_device.h"
#include "kv_step.h"
#include "launch.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <type_traits>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int SLOTS = 32; /* query capacity of a launch = MFMA tile width */
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

__device__ __forceinline__ constexpr uint32_t acc_key(uint32_t r, uint32_t h) { return 8u * (r >> 2) + 4u * h + (r & 3u); }
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

/* One wavefront per (head, slice): blockDim.x = 64 * hpb * slices, head =
 * blockIdx.z * hpb + wave % hpb, slice = wave / hpb.  The slices of a head
 * take the span's 32-key sub-chunks round-robin and merge through LDS. */
template <int HD, int WAVES, bool KARG>
__global__ __launch_bounds__(64 * WAVES, 2) void kv_block_mfma_kernel(StepArgs a, LensArg<KARG> lens) {
    constexpr int HALF = HD / 2;
    constexpr int DB = HD / 32;
    constexpr int ROW = HD + 4;
    constexpr int PR = HD + 2;  /* a parked result row: HD columns, max, sum; 32 * PR fits a K tile */
    constexpr int LPR = HD / 4; /* lanes per row when a wave moves a K tile, 16 bytes each */

    __shared__ __attribute__((aligned(16))) float sm_k[WAVES][32 * ROW];
    __shared__ uint32_t sm_ticket;

    const uint32_t b = blockIdx.y;
    const uint32_t split = blockIdx.x;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t slice = wave / a.hpb;
    const uint32_t head = blockIdx.z * a.hpb + wave % a.hpb;
    const bool head_ok = head < a.num_heads;
    const uint32_t hsafe = head_ok ? head : 0u;
    const uint32_t h = lane >> 5;
    const uint32_t c = lane & 31u;

    const uint32_t len = kv_len_of(a, lens, b) + a.len_bias;
    const uint32_t nk = len + a.n;
    if (!KARG && kv_over_capacity(a, nk)) return; /* uniform over the sequence's workgroups */
    const size_t slab = (size_t)b * a.max_seq_len;
    const uint32_t span = kv_span_of(a, nk);
    const uint32_t k_begin = split * span;
    const uint32_t k_end = min(k_begin + span, nk);
    const size_t newrow0 = (size_t)b * a.n_seq;

    /* query fragment: row c of the block (clamped), floats [h*HALF, (h+1)*HALF) of the head */
    const uint32_t qi = a.q0 + c;
    const bool q_ok = qi < a.n;
    float qf[HALF];
    {
        const float *qrow = a.q_rows + (newrow0 + min(qi, a.n - 1u)) * a.q_stride + hsafe * HD + h * HALF;
#pragma unroll
        for (int s = 0; s < HALF; s += 4) {
            float4 t = *reinterpret_cast<const float4 *>(qrow + s);
            if (a.rope_cos) { /* the query sits at position len + qi */
                const size_t at = (size_t)(len + min(qi, a.n - 1u)) * HALF + (h * HALF + s) / 2;
                t = rope_rotate4(t, a.rope_cos + at, a.rope_sin + at);
            }
            qf[s + 0] = t.x, qf[s + 1] = t.y, qf[s + 2] = t.z, qf[s + 3] = t.w;
        }
    }
    /* keys this lane's query sees within the span, as [vis_lo, vis_lo + vis_len):
     * causal rows see keys up to their own position (kv_cache.c:229-236, with
     * the local window cut), block rows see everything; padding rows nothing */
    uint32_t vis_lo = 0, vis_hi = k_end;
    if (!a.block_kind) {
        const uint32_t qpos = len + qi; /* absolute position of this lane's query */
        vis_hi = min(vis_hi, qpos + 1u);
        if (a.window > 0u && qpos + 1u > a.window) vis_lo = qpos + 1u - a.window;
    }
    if (!q_ok) vis_hi = 0;
    const uint32_t vis_len = vis_hi > vis_lo ? vis_hi - vis_lo : 0u;
    const float scale2 = a.scale * LOG2E;

    floatx16 oacc[DB];
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[d][r] = 0.f;
    float m = neg_inf(), l = 0.f;

    float *my_k = sm_k[wave];

    /* row j of the sequence: cached rows come from the slab, new rows from the step's inputs.
     * (Argument fields are copied out first: a select between two fields read in place becomes a
     * per-lane load of the argument block itself.) */
    const float *const cache_k = a.cache_k, *const cache_v = a.cache_v;
    const float *const new_k = a.k_rows, *const new_v = a.v_rows;
    const size_t embed_dim = a.embed_dim, k_stride = a.k_stride, v_stride = a.v_stride;
    auto k_row = [&](uint32_t j) __attribute__((always_inline)) -> const float * {
        const size_t at = j < len ? (slab + j) * embed_dim : (newrow0 + (j - len)) * k_stride;
        return (j < len ? cache_k : new_k) + at;
    };
    auto v_row = [&](uint32_t j) __attribute__((always_inline)) -> const float * {
        const size_t at = j < len ? (slab + j) * embed_dim : (newrow0 + (j - len)) * v_stride;
        return (j < len ? cache_v : new_v) + at;
    };

    /* Requests for the K tile (HD/8 pieces of 16 bytes per lane) and the V
     * fragment of the sub-chunk at key cs.  A sub-chunk that lies entirely in
     * the cached prefix (the common case) is addressed from one per-lane base
     * with compile-time row steps; one that touches the new rows or the end
     * of the sequence selects row by row. */
    auto request_k = [&](auto cached_only, float (&kg)[HALF], uint32_t cs) __attribute__((always_inline)) {
        if (decltype(cached_only)::value || cs + 32u <= len) {
            const float *kb = cache_k + (slab + cs + lane / LPR) * embed_dim + hsafe * HD + 4u * (lane % LPR);
#pragma unroll
            for (int t = 0; t < HD / 8; t++) {
                const float4 x = *reinterpret_cast<const float4 *>(kb + (size_t)(t * (64 / LPR)) * embed_dim);
                kg[4 * t + 0] = x.x, kg[4 * t + 1] = x.y, kg[4 * t + 2] = x.z, kg[4 * t + 3] = x.w;
            }
        } else {
#pragma unroll
            for (int t = 0; t < HD / 8; t++) {
                const uint32_t r = t * (64 / LPR) + lane / LPR;
                const uint32_t j = min(cs + r, nk - 1u);
                const float4 x = *reinterpret_cast<const float4 *>(k_row(j) + hsafe * HD + 4u * (lane % LPR));
                kg[4 * t + 0] = x.x, kg[4 * t + 1] = x.y, kg[4 * t + 2] = x.z, kg[4 * t + 3] = x.w;
            }
        }
    };
    auto request_v = [&](auto cached_only, float (&vf)[DB][16], uint32_t cs) __attribute__((always_inline)) {
        if (decltype(cached_only)::value || cs + 32u <= len) {
            const float *vb = cache_v + (slab + cs + 4u * h) * embed_dim + hsafe * HD + c;
#pragma unroll
            for (int s = 0; s < 16; s++) {
                const float *vr = vb + (size_t)(8 * (s >> 2) + (s & 3)) * embed_dim;
#pragma unroll
                for (int d = 0; d < DB; d++) vf[d][s] = vr[32 * d];
            }
        } else {
#pragma unroll
            for (int s = 0; s < 16; s++) {
                const uint32_t j = min(cs + acc_key(s, h), nk - 1u);
                const float *vr = v_row(j) + hsafe * HD + c;
#pragma unroll
                for (int d = 0; d < DB; d++) vf[d][s] = vr[32 * d];
            }
        }
    };

    /* One 32-key sub-chunk at key c0 whose K tile and V fragment have been
     * requested into kg / vf.  As soon as kg is parked in LDS it is reused for
     * the K tile of the sub-chunk at cnext (when `more`), and vf for its V
     * fragment once the second product has consumed it, so those rows travel
     * while this and the following sub-chunks are worked on. */
    auto sub_chunk = [&](auto touches_new_rows, float (&kg)[HALF], float (&vf)[DB][16], uint32_t c0,
                         uint32_t cnext, bool more) __attribute__((always_inline)) {
        /* NEW = false: this sub-chunk and the one requested at cnext lie in the cached prefix: nothing
         * to rotate or write through, one address form.  That body has no branch around a load or a
         * store, so its waits stay exact. */
        constexpr bool NEW = decltype(touches_new_rows)::value;
        constexpr std::integral_constant<bool, !NEW> next_cached{};
        /* K tile: write-through of new rows, then LDS -> fragment (lane = key row) */
#pragma unroll
        for (int t = 0; t < HD / 8; t++) {
            const uint32_t r = t * (64 / LPR) + lane / LPR;
            float4 piece = make_float4(kg[4 * t + 0], kg[4 * t + 1], kg[4 * t + 2], kg[4 * t + 3]);
            if constexpr (NEW) {
                const uint32_t j = c0 + r;
                if (a.rope_cos && j >= len && j < nk) { /* a new key row is rotated at its position j */
                    const size_t at = (size_t)j * HALF + 2u * (lane % LPR);
                    piece = rope_rotate4(piece, a.rope_cos + at, a.rope_sin + at);
                }
                if (a.write_through && head_ok && j >= len && j < k_end)
                    *reinterpret_cast<float4 *>(a.cache_k + (slab + j) * a.embed_dim + head * HD +
                                                4u * (lane % LPR)) = piece;
            }
            *reinterpret_cast<float4 *>(my_k + r * ROW + 4u * (lane % LPR)) = piece;
        }
        float kf[HALF];
#pragma unroll
        for (int s = 0; s < HALF; s += 4) {
            const float4 t = *reinterpret_cast<const float4 *>(my_k + c * ROW + h * HALF + s);
            kf[s + 0] = t.x, kf[s + 1] = t.y, kf[s + 2] = t.z, kf[s + 3] = t.w;
        }
        if (more) request_k(next_cached, kg, cnext);
        /* the requests stay where they are written: left alone, the scheduler moves loads whose
         * results are not needed in this block to its end, which is the opposite of a prefetch */
        __builtin_amdgcn_sched_barrier(0);

        floatx16 sacc;
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[r] = 0.f;
#pragma unroll
        for (int s = 0; s < HALF; s++) sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[s], qf[s], sacc, 0, 0, 0);

        float x[16];
        float mt = neg_inf();
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float t = sacc[r] * scale2;
            /* one unsigned compare: vis_lo <= j < vis_lo + vis_len */
            const bool vis = (c0 + acc_key(r, h) - vis_lo) < vis_len && isfinite(t);
            x[r] = vis ? t : neg_inf();
            mt = fmaxf(mt, x[r]);
        }
        mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
        const float mn = fmaxf(m, mt);
        const float ms = mn == neg_inf() ? 0.f : mn;
        const float alpha = fast_exp2(m - ms);
        float ps = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            x[r] = fast_exp2(x[r] - ms);
            ps += x[r];
        }
        l = l * alpha + ps;
        m = mn;
#pragma unroll
        for (int d = 0; d < DB; d++) {
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[d][r] *= alpha;
#pragma unroll
            for (int s = 0; s < 16; s++) oacc[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(vf[d][s], x[s], oacc[d], 0, 0, 0);
        }

        /* V: write-through of new rows from the values just used, then the next rows */
        if constexpr (NEW) {
            if (a.write_through && head_ok) {
#pragma unroll
                for (int s = 0; s < 16; s++) {
                    const uint32_t j = c0 + acc_key(s, h);
                    if (j >= len && j < k_end) {
#pragma unroll
                        for (int d = 0; d < DB; d++)
                            a.cache_v[(slab + j) * a.embed_dim + head * HD + 32 * d + c] = vf[d][s];
                    }
                }
            }
        }
        if (more) request_v(next_cached, vf, cnext);
        __builtin_amdgcn_sched_barrier(0);
    };
    constexpr std::false_type CACHED{};
    constexpr std::true_type GENERAL{};

    const uint32_t step = a.slices * 32u;
    uint32_t c0 = k_begin + slice * 32u;
    float kg[HALF];
    float vf[DB][16];
    if (c0 < k_end) {
        request_k(std::false_type{}, kg, c0);
        request_v(std::false_type{}, vf, c0);
    }
    while (c0 + step + 32u <= len && c0 + step < k_end) { /* this and the next sub-chunk are cached rows */
        sub_chunk(CACHED, kg, vf, c0, c0 + step, true);
        c0 += step;
    }
    while (c0 < k_end) {
        const uint32_t cn = c0 + step;
        sub_chunk(GENERAL, kg, vf, c0, cn, cn < k_end);
        c0 = cn;
    }

    l += __shfl_xor(l, 32, 64);

    /* lane (h, c) holds O^T[d = 32*db + acc_key(r, h)][query c].  The wave
     * turns that into rows [query][HD columns, max, sum] in its LDS tile; then
     * the workgroup merges the slices of each head with consecutive threads
     * on consecutive floats of a row, which is also the order of the output
     * rows and of the per-split records in the partial buffer. */
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
        for (int r = 0; r < 16; r++) my_k[c * PR + 32 * d + acc_key(r, h)] = oacc[d][r];
    if (h == 0) {
        my_k[c * PR + HD + 0] = m * LN2; /* merges work in natural units */
        my_k[c * PR + HD + 1] = l;
    }
    __syncthreads();
    /* every wave of the workgroup has long read the old length: draw the ticket now, look at it last */
    const uint32_t early_ticket = kv_draw_early_ticket(a, b);

    const uint32_t rows = a.n - a.q0 < (uint32_t)SLOTS ? a.n - a.q0 : (uint32_t)SLOTS;
    const uint32_t cells = a.hpb * rows * PR;
    for (uint32_t t = threadIdx.x; t < cells; t += blockDim.x) {
        const uint32_t col = t % PR;
        const uint32_t r = (t / PR) % rows;
        const uint32_t hl = t / (PR * rows);
        const uint32_t hh = blockIdx.z * a.hpb + hl;
        if (hh >= a.num_heads) continue;
        float M = neg_inf();
        for (uint32_t s = 0; s < a.slices; s++) M = fmaxf(M, sm_k[s * a.hpb + hl][r * PR + HD]);
        float L = 0.f, acc = 0.f;
        for (uint32_t s = 0; s < a.slices; s++) {
            const float *ps = sm_k[s * a.hpb + hl] + r * PR;
            const float f = ps[HD] == neg_inf() ? 0.f : softmax_exp(ps[HD] - M);
            L += ps[HD + 1] * f;
            if (col < (uint32_t)HD) acc += ps[col] * f;
        }
        if (a.splits == 1u) {
            if (col < (uint32_t)HD)
                a.combined[(newrow0 + a.q0 + r) * a.out_stride + hh * HD + col] = L > 0.f ? acc / L : 0.f;
        } else {
            float *dst = a.partial + ((((size_t)b * a.splits + split) * a.num_heads + hh) * SLOTS + r) * PR;
            publish(dst + col, col < (uint32_t)HD ? acc : (col == (uint32_t)HD ? M : L));
        }
    }

    kv_finish_sequence<HD>(a, (uint32_t)SLOTS, b, nk, &sm_ticket, early_ticket);
}

typedef float floatx4 __attribute__((ext_vector_type(4)));

/* The same step for blocks of at most 16 rows on 16x16x4 tiles
 * (v_mfma_f32_16x16x4_f32: A[i = lane % 16][k = lane / 16], B[k = lane / 16][j = lane % 16],
 * D[i = 4 * (lane / 16) + r][j = lane % 16]), so that no half of a tile is padding:
 *
 *   S^T[key, query]: two 16-key tiles per sub-chunk; lane group g = lane / 16 contracts the
 *                    head's columns [g * HD/4, (g + 1) * HD/4), one per step;
 *   O^T[d, query]:   HD/16 tiles; the contraction runs over the keys, lane group g taking key
 *                    16 t + 4 g + r at step (t, r) -- exactly the key whose weight its S^T
 *                    register (t, r) holds, so P^T needs no exchange.
 *
 * Half the matrix-core cycles and half the softmax arithmetic of the 32-wide kernel per
 * sub-chunk.  K and V fragments come straight from global memory in fragment layout (a K row's
 * 128 bytes are shared by the four lane groups), nothing is staged through LDS. */
template <int HD, int WAVES, bool KARG>
__global__ __launch_bounds__(64 * WAVES, 2) void kv_block16_mfma_kernel(StepArgs a, LensArg<KARG> lens) {
    constexpr int HALF = HD / 2;
    constexpr int QD = HD / 4;  /* columns of the head one lane group contracts */
    constexpr int DT = HD / 16; /* 16-row tiles of O^T */
    constexpr int PR = HD + 2;  /* a parked result row: HD columns, max, sum */
    constexpr uint32_t ROWS = 16;

    __shared__ float sm_o[WAVES][ROWS * PR];
    __shared__ uint32_t sm_ticket;

    const uint32_t b = blockIdx.y;
    const uint32_t split = blockIdx.x;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t slice = wave / a.hpb;
    const uint32_t head = blockIdx.z * a.hpb + wave % a.hpb;
    const bool head_ok = head < a.num_heads;
    const uint32_t hsafe = head_ok ? head : 0u;
    const uint32_t g = lane >> 4;
    const uint32_t c = lane & 15u;

    const uint32_t len = kv_len_of(a, lens, b) + a.len_bias;
    const uint32_t nk = len + a.n;
    if (!KARG && kv_over_capacity(a, nk)) return; /* uniform over the sequence's workgroups */
    const size_t slab = (size_t)b * a.max_seq_len;
    const uint32_t span = kv_span_of(a, nk);
    const uint32_t k_begin = split * span;
    const uint32_t k_end = min(k_begin + span, nk);
    const size_t newrow0 = (size_t)b * a.n_seq;

    /* query fragment: row c of the block (clamped), columns [g*QD, (g+1)*QD) of the head */
    const uint32_t qi = a.q0 + c;
    const bool q_ok = qi < a.n;
    float qf[QD];
    {
        const float *qrow = a.q_rows + (newrow0 + min(qi, a.n - 1u)) * a.q_stride + hsafe * HD + g * QD;
#pragma unroll
        for (int s = 0; s < QD; s += 4) {
            float4 t = *reinterpret_cast<const float4 *>(qrow + s);
            if (a.rope_cos) { /* the query sits at position len + qi */
                const size_t at = (size_t)(len + min(qi, a.n - 1u)) * HALF + (g * QD + s) / 2;
                t = rope_rotate4(t, a.rope_cos + at, a.rope_sin + at);
            }
            qf[s + 0] = t.x, qf[s + 1] = t.y, qf[s + 2] = t.z, qf[s + 3] = t.w;
        }
    }
    uint32_t vis_lo = 0, vis_hi = k_end;
    if (!a.block_kind) {
        const uint32_t qpos = len + qi;
        vis_hi = min(vis_hi, qpos + 1u);
        if (a.window > 0u && qpos + 1u > a.window) vis_lo = qpos + 1u - a.window;
    }
    if (!q_ok) vis_hi = 0;
    const uint32_t vis_len = vis_hi > vis_lo ? vis_hi - vis_lo : 0u;
    const float scale2 = a.scale * LOG2E;

    floatx4 oacc[DT];
#pragma unroll
    for (int d = 0; d < DT; d++)
#pragma unroll
        for (int r = 0; r < 4; r++) oacc[d][r] = 0.f;
    float m = neg_inf(), l = 0.f;

    const float *const cache_k = a.cache_k, *const cache_v = a.cache_v;
    const float *const new_k = a.k_rows, *const new_v = a.v_rows;
    const size_t embed_dim = a.embed_dim, k_stride = a.k_stride, v_stride = a.v_stride;
    auto k_row = [&](uint32_t j) __attribute__((always_inline)) -> const float * {
        const size_t at = j < len ? (slab + j) * embed_dim : (newrow0 + (j - len)) * k_stride;
        return (j < len ? cache_k : new_k) + at;
    };
    auto v_row = [&](uint32_t j) __attribute__((always_inline)) -> const float * {
        const size_t at = j < len ? (slab + j) * embed_dim : (newrow0 + (j - len)) * v_stride;
        return (j < len ? cache_v : new_v) + at;
    };

    /* K fragment of the sub-chunk at key cs: tile t holds key cs + 16 t + c, columns g*QD ...;
     * V fragment: element (d, 4 t + r) is column 16 d + c of key cs + 16 t + 4 g + r */
    auto request_k = [&](auto cached_only, float (&kf)[2][QD], uint32_t cs) __attribute__((always_inline)) {
        if (decltype(cached_only)::value || cs + 32u <= len) {
            const float *kb = cache_k + (slab + cs + c) * embed_dim + hsafe * HD + g * QD;
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int s = 0; s < QD; s += 4) {
                    const float4 x = *reinterpret_cast<const float4 *>(kb + (size_t)(16 * t) * embed_dim + s);
                    kf[t][s + 0] = x.x, kf[t][s + 1] = x.y, kf[t][s + 2] = x.z, kf[t][s + 3] = x.w;
                }
        } else {
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const uint32_t j = min(cs + 16u * t + c, nk - 1u);
                const float *kr = k_row(j) + hsafe * HD + g * QD;
#pragma unroll
                for (int s = 0; s < QD; s += 4) {
                    const float4 x = *reinterpret_cast<const float4 *>(kr + s);
                    kf[t][s + 0] = x.x, kf[t][s + 1] = x.y, kf[t][s + 2] = x.z, kf[t][s + 3] = x.w;
                }
            }
        }
    };
    auto request_v = [&](auto cached_only, float (&vf)[DT][8], uint32_t cs) __attribute__((always_inline)) {
        if (decltype(cached_only)::value || cs + 32u <= len) {
            const float *vb = cache_v + (slab + cs + 4u * g) * embed_dim + hsafe * HD + c;
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const float *vr = vb + (size_t)(16 * (u >> 2) + (u & 3)) * embed_dim;
#pragma unroll
                for (int d = 0; d < DT; d++) vf[d][u] = vr[16 * d];
            }
        } else {
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const uint32_t j = min(cs + 16u * (u >> 2) + 4u * g + (u & 3), nk - 1u);
                const float *vr = v_row(j) + hsafe * HD + c;
#pragma unroll
                for (int d = 0; d < DT; d++) vf[d][u] = vr[16 * d];
            }
        }
    };

    auto sub_chunk = [&](auto touches_new_rows, float (&kf)[2][QD], float (&vf)[DT][8], uint32_t c0, uint32_t cnext,
                         bool more) __attribute__((always_inline)) {
        constexpr bool NEW = decltype(touches_new_rows)::value;
        constexpr std::integral_constant<bool, !NEW> next_cached{};
        float kc[2][QD]; /* this sub-chunk's K values; kf is handed to the next request at once */
#pragma unroll
        for (int t = 0; t < 2; t++) {
#pragma unroll
            for (int s = 0; s < QD; s += 4) {
                float4 piece = make_float4(kf[t][s + 0], kf[t][s + 1], kf[t][s + 2], kf[t][s + 3]);
                if constexpr (NEW) {
                    const uint32_t j = c0 + 16u * t + c;
                    if (a.rope_cos && j >= len && j < nk) { /* a new key row is rotated at its position j */
                        const size_t at = (size_t)j * HALF + (g * QD + s) / 2;
                        piece = rope_rotate4(piece, a.rope_cos + at, a.rope_sin + at);
                    }
                    if (a.write_through && head_ok && j >= len && j < k_end)
                        *reinterpret_cast<float4 *>(a.cache_k + (slab + j) * a.embed_dim + head * HD + g * QD + s) =
                            piece;
                }
                kc[t][s + 0] = piece.x, kc[t][s + 1] = piece.y, kc[t][s + 2] = piece.z, kc[t][s + 3] = piece.w;
            }
        }
        if (more) request_k(next_cached, kf, cnext);
        __builtin_amdgcn_sched_barrier(0); /* the requests stay ahead of the arithmetic */

        floatx4 sacc[2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
#pragma unroll
            for (int r = 0; r < 4; r++) sacc[t][r] = 0.f;
#pragma unroll
            for (int s = 0; s < QD; s++) sacc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kc[t][s], qf[s], sacc[t], 0, 0, 0);
        }

        float x[8];
        float mt = neg_inf();
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const float t = sacc[u >> 2][u & 3] * scale2;
            const uint32_t j = c0 + 16u * (u >> 2) + 4u * g + (u & 3);
            const bool vis = ((j - vis_lo) < vis_len) & isfinite(t);
            x[u] = vis ? t : neg_inf();
            mt = fmaxf(mt, x[u]);
        }
        mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
        mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
        const float mn = fmaxf(m, mt);
        const float ms = mn == neg_inf() ? 0.f : mn;
        const float alpha = fast_exp2(m - ms);
        float ps = 0.f;
#pragma unroll
        for (int u = 0; u < 8; u++) {
            x[u] = fast_exp2(x[u] - ms);
            ps += x[u];
        }
        l = l * alpha + ps;
        m = mn;
#pragma unroll
        for (int d = 0; d < DT; d++) {
#pragma unroll
            for (int r = 0; r < 4; r++) oacc[d][r] *= alpha;
#pragma unroll
            for (int u = 0; u < 8; u++) oacc[d] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[d][u], x[u], oacc[d], 0, 0, 0);
        }

        if constexpr (NEW) {
            if (a.write_through && head_ok) {
#pragma unroll
                for (int u = 0; u < 8; u++) {
                    const uint32_t j = c0 + 16u * (u >> 2) + 4u * g + (u & 3);
                    if (j >= len && j < k_end) {
#pragma unroll
                        for (int d = 0; d < DT; d++)
                            a.cache_v[(slab + j) * a.embed_dim + head * HD + 16 * d + c] = vf[d][u];
                    }
                }
            }
        }
        if (more) request_v(next_cached, vf, cnext);
        __builtin_amdgcn_sched_barrier(0);
    };
    constexpr std::false_type CACHED{};
    constexpr std::true_type GENERAL{};

    const uint32_t step = a.slices * 32u;
    uint32_t c0 = k_begin + slice * 32u;
    float kf[2][QD];
    float vf[DT][8];
    if (c0 < k_end) {
        request_k(std::false_type{}, kf, c0);
        request_v(std::false_type{}, vf, c0);
    }
    while (c0 + step + 32u <= len && c0 + step < k_end) { /* this and the next sub-chunk are cached rows */
        sub_chunk(CACHED, kf, vf, c0, c0 + step, true);
        c0 += step;
    }
    while (c0 < k_end) {
        const uint32_t cn = c0 + step;
        sub_chunk(GENERAL, kf, vf, c0, cn, cn < k_end);
        c0 = cn;
    }

    /* the four lane groups of a column carry the same m, their sums add */
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);

    /* lane (g, c) holds O^T[d = 16 dt + 4 g + r][query c]: park rows [query][HD columns, max, sum]
     * in the wave's LDS tile, then merge the slices of each head as the 32-wide kernel does */
    float *mine = sm_o[wave];
#pragma unroll
    for (int d = 0; d < DT; d++)
#pragma unroll
        for (int r = 0; r < 4; r++) mine[c * PR + 16 * d + 4 * g + r] = oacc[d][r];
    if (g == 0) {
        mine[c * PR + HD + 0] = m * LN2; /* merges work in natural units */
        mine[c * PR + HD + 1] = l;
    }
    __syncthreads();
    const uint32_t early_ticket = kv_draw_early_ticket(a, b); /* as in the 32-wide kernel */

    const uint32_t rows = a.n - a.q0 < ROWS ? a.n - a.q0 : ROWS;
    const uint32_t cells = a.hpb * rows * PR;
    for (uint32_t t = threadIdx.x; t < cells; t += blockDim.x) {
        const uint32_t col = t % PR;
        const uint32_t r = (t / PR) % rows;
        const uint32_t hl = t / (PR * rows);
        const uint32_t hh = blockIdx.z * a.hpb + hl;
        if (hh >= a.num_heads) continue;
        float M = neg_inf();
        for (uint32_t s = 0; s < a.slices; s++) M = fmaxf(M, sm_o[s * a.hpb + hl][r * PR + HD]);
        float L = 0.f, acc = 0.f;
        for (uint32_t s = 0; s < a.slices; s++) {
            const float *ps = sm_o[s * a.hpb + hl] + r * PR;
            const float f = ps[HD] == neg_inf() ? 0.f : softmax_exp(ps[HD] - M);
            L += ps[HD + 1] * f;
            if (col < (uint32_t)HD) acc += ps[col] * f;
        }
        if (a.splits == 1u) {
            if (col < (uint32_t)HD)
                a.combined[(newrow0 + a.q0 + r) * a.out_stride + hh * HD + col] = L > 0.f ? acc / L : 0.f;
        } else {
            float *dst = a.partial + ((((size_t)b * a.splits + split) * a.num_heads + hh) * SLOTS + r) * PR;
            publish(dst + col, col < (uint32_t)HD ? acc : (col == (uint32_t)HD ? M : L));
        }
    }

    kv_finish_sequence<HD>(a, (uint32_t)SLOTS, b, nk, &sm_ticket, early_ticket);
}

template <int HD, int WAVES>
void launch_block(StepArgs a, uint32_t batch, const uint32_t *host_lens, hipStream_t s) {
    /* a.hpb heads per workgroup (the caller's choice, see kv_block_heads_per_group); the other waves are slices */
    a.hpb = std::max(1u, std::min<uint32_t>(std::min<uint32_t>(a.hpb, a.num_heads), (uint32_t)WAVES));
    const uint32_t subs = (a.span + 31u) / 32u;
    a.slices = std::max(1u, std::min<uint32_t>((uint32_t)WAVES / a.hpb, subs));
    dim3 grid(a.splits, batch, (a.num_heads + a.hpb - 1) / a.hpb);
    /* blocks of up to 16 rows on 16-wide tiles; BLT_HIP_BLOCK_TILE=32 keeps the 32-wide kernel (test hook) */
    static const bool wide_only = [] {
        const char *e = getenv("BLT_HIP_BLOCK_TILE");
        return e && strcmp(e, "32") == 0;
    }();
    const dim3 block(64 * a.hpb * a.slices);
    const bool narrow = a.n - a.q0 <= 16u && !wide_only;
    if (host_lens) {
        KargLens lens;
        for (uint32_t b = 0; b < batch; b++) lens.v[b] = host_lens[b];
        if (narrow) blt_launch("kv_block16_mfma", kv_block16_mfma_kernel<HD, WAVES, true>, grid, block, 0, s, a, lens);
        else blt_launch("kv_block_mfma", kv_block_mfma_kernel<HD, WAVES, true>, grid, block, 0, s, a, lens);
    } else {
        const DeviceLens lens{0u};
        if (narrow) blt_launch("kv_block16_mfma", kv_block16_mfma_kernel<HD, WAVES, false>, grid, block, 0, s, a, lens);
        else blt_launch("kv_block_mfma", kv_block_mfma_kernel<HD, WAVES, false>, grid, block, 0, s, a, lens);
    }
}

} // namespace

/* Heads per workgroup for `batch` sequences of `subs` 32-key sub-chunks: one
 * head (all waves are slices of it, which keeps short launches free of the
 * cross-workgroup merge) when there are enough sub-chunks to occupy the
 * slices and one workgroup per (sequence, head) does not exceed what the
 * chip holds at once (one 8-wave workgroup per compute unit); else two. */
uint32_t kv_block_heads_per_group(uint32_t batch, uint32_t subs, uint32_t num_heads) {
    if (num_heads == 1u) return 1u;
    return subs >= 4u && (uint64_t)batch * num_heads <= 256u ? 1u : 2u;
}

/* Takes head_dim 32 and 64 (the K tiles of four waves fit the static LDS
 * budget); the caller falls back to the VALU kernel otherwise.  Handles up to
 * 32 query rows per launch: a.q0 .. a.q0 + 31. */
bool kv_block_mfma_launch(const StepArgs &a, uint32_t batch, uint32_t head_dim, const uint32_t *host_lens,
                          hipStream_t s) {
    /* the per-wave K tiles bound the workgroup: 8 waves of 4.6 KB or 4 of 8.7 KB */
    if (head_dim == 32u) launch_block<32, 8>(a, batch, host_lens, s);
    else if (head_dim == 64u) launch_block<64, 4>(a, batch, host_lens, s);
    else return false;
    return true;
}
