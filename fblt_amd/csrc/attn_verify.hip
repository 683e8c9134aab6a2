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
#include "lane_ops.h"

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
    kv_fetch_arguments(a);
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

/* Merge of the slices of each head after the waves have parked rows [query][HD columns .. max,
 * sum] (row pitch LPR floats, maxima in natural units) in sm_o[wave].  A cell is (local head, row,
 * column quad); a wave takes 64 / WAVES cells and spreads each over WAVES lanes, one per slice:
 * a lane reads its slice's (max, sum) and quad, the common maximum and the weighted sums are
 * cross-lane operations in the vector ALU, and the lane of slice 0 stores.  The serial work per
 * lane does not grow with the number of slices (a loop over the slices in one thread did: 1900
 * cycles at 8 slices, by cycle marks).  With one split the output rows are written, otherwise the
 * workgroup's per-split records. */
template <int HD, int WAVES, int LPR, int ROWCAP, int STRIDE = ROWCAP * LPR> /* STRIDE: floats between the waves' tiles */
__device__ __forceinline__ void kv_merge_slices(const StepArgs &a, const float (*sm_o)[STRIDE], uint32_t hshift,
                                                uint32_t wave, uint32_t b, uint32_t split, size_t newrow0,
                                                const uint32_t zblock) {
    static_assert(WAVES == 4 || WAVES == 8 || WAVES == 16, "slices map onto lane groups of a wave");
    constexpr int PR = HD + 2; /* a per-split record in global memory: HD columns, max, sum */
    constexpr uint32_t QUADS = HD / 4;
    constexpr uint32_t CPW = 64 / WAVES; /* cells per wave and pass */
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t s = lane / CPW; /* this lane's slice */
    const uint32_t rows = a.n - a.q0 < (uint32_t)ROWCAP ? a.n - a.q0 : (uint32_t)ROWCAP;
    const uint32_t cells = a.hpb * rows * QUADS;
    const uint32_t nwaves = a.hpb * a.slices;
    for (uint32_t cell0 = wave * CPW; cell0 < cells; cell0 += nwaves * CPW) { /* uniform over the wave */
        const uint32_t cell = cell0 + lane % CPW;
        const bool live = cell < cells && s < a.slices;
        const uint32_t cc = min(cell, cells - 1u);
        const uint32_t quad = cc % QUADS;
        const uint32_t r = (cc / QUADS) % rows;
        const uint32_t hl = cc / (QUADS * rows);
        const uint32_t hh = zblock * a.hpb + hl;
        const float *ps = sm_o[(min(s, a.slices - 1u) << hshift) + hl] + r * LPR;
        const float2 ml = *reinterpret_cast<const float2 *>(ps + HD);
        const float4 o4 = *reinterpret_cast<const float4 *>(ps + 4u * quad);
        const float mine = live ? ml.x : neg_inf();
        const float M = across_keys<(int)CPW>(mine, OpMax());
        const float f = mine == neg_inf() ? 0.f : softmax_exp(mine - M);
        const float L = across_keys<(int)CPW>(ml.y * f, OpSum());
        float4 acc;
        acc.x = across_keys<(int)CPW>(o4.x * f, OpSum());
        acc.y = across_keys<(int)CPW>(o4.y * f, OpSum());
        acc.z = across_keys<(int)CPW>(o4.z * f, OpSum());
        acc.w = across_keys<(int)CPW>(o4.w * f, OpSum());
        if (s != 0u || cell >= cells || hh >= a.num_heads) continue;
        if (a.splits == 1u) {
            const float inv = L > 0.f ? 1.0f / L : 0.f;
            *reinterpret_cast<float4 *>(a.combined + (newrow0 + a.q0 + r) * a.out_stride + hh * HD + 4u * quad) =
                make_float4(acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv);
        } else {
            float *dst = a.partial + ((((size_t)b * a.splits + split) * a.num_heads + hh) * SLOTS + r) * PR;
            publish(dst + 4u * quad + 0, acc.x), publish(dst + 4u * quad + 1, acc.y);
            publish(dst + 4u * quad + 2, acc.z), publish(dst + 4u * quad + 3, acc.w);
            if (quad == 0) publish(dst + HD, M), publish(dst + HD + 1, L);
        }
    }
}

/* The same step for blocks of at most 16 rows on 16x16x4 tiles
 * (v_mfma_f32_16x16x4_f32: A[i = lane % 16][k = lane / 16], B[k = lane / 16][j = lane % 16],
 * D[i = 4 * (lane / 16) + r][j = lane % 16]), so that no half of a tile is padding:
 *
 *   S^T[key, query]: two 16-key tiles per sub-chunk; lane group g = lane / 16 contracts the
 *                    head's columns [g * HD/4, (g + 1) * HD/4), one per step;
 *   O^T[d, query]:   HD/16 tiles; the contraction runs over the keys, lane group g taking key
 *                    16 t + 4 g + r at step (t, r) -- exactly the key whose weight its S^T
 *                    register (t, r) holds, so P^T needs no exchange.  Row i of tile e is column
 *                    (HD/16) i + e of the head: a lane's HD/16 operands of one key are
 *                    consecutive floats, one 8- or 16-byte load, and the sixteen lanes of a group
 *                    read the key's row as one contiguous piece.
 *
 * Half the matrix-core cycles and half the softmax arithmetic of the 32-wide kernel per
 * sub-chunk.  K and V fragments come straight from global memory in fragment layout (a K row's
 * 128 bytes are shared by the four lane groups), nothing is staged through LDS.
 *
 * At the sizes this kernel is used for, a workgroup's time is issue time and dependent trips to
 * memory, not bandwidth (cycle marks at 64 sequences x 4 heads x <= 524 keys: 1300 cycles of
 * address arithmetic per sub-chunk request with per-row 64-bit selects, 3100 cycles in a merge
 * loop of dependent LDS reads).  Hence:
 *   - the sequence is walked as ceil(len / 32) sub-chunks of cached rows followed by ONE
 *     sub-chunk that holds the step's new rows.  Which of the two a sub-chunk is, is uniform
 *     over the wave, so base pointer, row stride and row limit are scalar selects and every
 *     load is `scalar base + 32-bit lane offset` (two vector instructions per row, no branch);
 *   - the first sub-chunk is requested before the query rows; the next one before this one is
 *     worked on, unconditionally (past the end the clamped rows hit the cache), so the wait in
 *     between counts exactly the newer requests;
 *   - cross-lane maxima and sums use the row swaps of the vector ALU, not the LDS crossbar;
 *   - the slices meet once in LDS; the merge issues all of a cell's reads before it adds. */
template <int HD, int WAVES, bool KARG>
__global__ __launch_bounds__(64 * WAVES, 1) void kv_block16_mfma_kernel(StepArgs a, LensArg<KARG> lens) {
    kv_fetch_arguments(a);
    constexpr int HALF = HD / 2;
    constexpr int QD = HD / 4;  /* columns of the head one lane group contracts */
    constexpr int DT = HD / 16; /* 16-row tiles of O^T */
    constexpr int LPR = HD + 4; /* a result row [HD columns, max, sum] parked in LDS, rows 16-byte aligned */
    constexpr uint32_t ROWS = 16;
    constexpr int KROW = HD + 4;      /* a K row on its way to fragments: the same padded row */
    constexpr int KL = HD / 4;        /* lanes per K row when the wave moves a sub-chunk, 16 bytes each */
    constexpr int KRI = 64 / KL;      /* K rows one load instruction covers */
    constexpr int KNV = 32 / KRI;     /* load instructions per 32-key sub-chunk */

    /* per wave: the sub-chunk's 32 K rows between their coalesced loads and the fragment reads; after the
     * loop the first half of the same area holds the wave's result rows */
    __shared__ __attribute__((aligned(16))) float sm_kt[WAVES][32 * KROW];
    float(*const sm_o)[32 * KROW] = sm_kt;
    static_assert(ROWS * LPR <= 32 * KROW, "the result rows fit the K tile they overlay");
    __shared__ uint32_t sm_ticket;

    /* Which (sequence, head group) the workgroup takes.  Launches by length walk the pairs sequence
     * by sequence, longest first, in the order workgroups are handed out (y before z): with more
     * pairs than compute units the units that finish the shortest of the first round pick up the
     * longest of the rest, so every unit ends up with about the same number of keys. */
    uint32_t b = blockIdx.y, zblock = blockIdx.z;
    if constexpr (KARG) {
        if (a.by_length) {
            const uint32_t at = blockIdx.y + gridDim.y * blockIdx.z;
            zblock = at % gridDim.z;
            b = lens.order[at / gridDim.z];
        }
    }
    const uint32_t split = blockIdx.x;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); /* uniform, and known to be */
    const uint32_t hshift = (uint32_t)__builtin_ctz(a.hpb);                 /* heads per workgroup: a power of two */
    const uint32_t slice = wave >> hshift;
    const uint32_t head = zblock * a.hpb + (wave & (a.hpb - 1u));
    const bool head_ok = head < a.num_heads;
    const uint32_t hsafe = head_ok ? head : 0u;
    const uint32_t g = lane >> 4;
    const uint32_t c = lane & 15u;

    const uint32_t len = kv_len_of(a, lens, b) + a.len_bias;
    const uint32_t nk = len + a.n;
    if (!KARG && kv_over_capacity(a, nk)) return; /* uniform over the sequence's workgroups */
    const size_t slab = (size_t)b * a.max_seq_len;
    const size_t newrow0 = (size_t)b * a.n_seq;
    /* sub-chunks of this sequence: the cached ones, then the one with the new rows; this
     * workgroup's share [s_begin, s_end), its waves' slices round-robin */
    const uint32_t cached_subs = (len + 31u) / 32u;
    const uint32_t total_subs = cached_subs + 1u;
    const uint32_t per_split = a.splits == 1u ? total_subs : (total_subs + a.splits - 1u) / a.splits;
    const uint32_t s_begin = split * per_split;
    const uint32_t s_end = min(s_begin + per_split, total_subs);

    const float *const cache_k = a.cache_k + slab * a.embed_dim + hsafe * HD;
    const float *const cache_v = a.cache_v + slab * a.embed_dim + hsafe * HD;
    const float *const new_k = a.k_rows + newrow0 * a.k_stride + hsafe * HD;
    const float *const new_v = a.v_rows + newrow0 * a.v_stride + hsafe * HD;
    const uint32_t cache_pitch = a.embed_dim * 4u, newk_pitch = a.k_stride * 4u, newv_pitch = a.v_stride * 4u;
    const uint32_t last_cached = len > 0u ? len - 1u : 0u, last_new = a.n - 1u;
    const uint32_t lane_k = g * (QD * 4u); /* byte offset inside a row */

    /* K rows of sub-chunk si as the wave moves them: load v covers rows KRI v ... KRI v + KRI - 1 with
     * consecutive lanes on consecutive 16-byte pieces of a row (lanes that each touch another row
     * are served at a quarter of the rate); they become fragments through the wave's LDS tile.
     * The V rows the same way (as fragments -- element (e, 4 t + r) is column DT c + e of row
     * 16 t + 4 g + r -- a load moves half the bytes per instruction at head width 32, and the
     * compute unit's vector memory path is what a long sequence waits for). */
    const uint32_t krow_l = lane / KL, kpiece = lane % KL;
    auto request = [&](floatx4 (&kg)[KNV], floatx4 (&vg)[KNV], uint32_t si) __attribute__((always_inline)) {
        const bool fresh = si >= cached_subs; /* wave-uniform: scalar selects */
        const char *kb = reinterpret_cast<const char *>(fresh ? new_k : cache_k);
        const char *vb = reinterpret_cast<const char *>(fresh ? new_v : cache_v);
        const uint32_t kp = fresh ? newk_pitch : cache_pitch, vp = fresh ? newv_pitch : cache_pitch;
        const uint32_t row0 = fresh ? 0u : si * 32u, limit = fresh ? last_new : last_cached;
#pragma unroll
        for (int v = 0; v < KNV; v++) {
            const uint32_t off = min(row0 + (uint32_t)(KRI * v) + krow_l, limit) * kp + 16u * kpiece;
            kg[v] = *reinterpret_cast<const floatx4 *>(kb + off);
        }
#pragma unroll
        for (int v = 0; v < KNV; v++) {
            const uint32_t off = min(row0 + (uint32_t)(KRI * v) + krow_l, limit) * vp + 16u * kpiece;
            vg[v] = *reinterpret_cast<const floatx4 *>(vb + off);
        }
    };

    /* the first sub-chunk's rows are requested before anything else waits for memory */
    uint32_t si = s_begin + slice;
    floatx4 kg[KNV], vg[KNV];
    request(kg, vg, si);

    /* query fragment: row c of the block (clamped), columns [g*QD, (g+1)*QD) of the head */
    const uint32_t qi = a.q0 + c;
    const bool q_ok = qi < a.n;
    float qf[QD];
    {
        const char *qb = reinterpret_cast<const char *>(a.q_rows + newrow0 * a.q_stride + hsafe * HD);
        const uint32_t off = min(qi, a.n - 1u) * (a.q_stride * 4u) + lane_k;
#pragma unroll
        for (int s = 0; s < QD; s += 4) {
            float4 t = *reinterpret_cast<const float4 *>(qb + off + 4 * s);
            if (a.rope_cos) { /* the query sits at position len + qi */
                const size_t at = (size_t)(len + min(qi, a.n - 1u)) * HALF + (g * QD + s) / 2;
                t = rope_rotate4(t, a.rope_cos + at, a.rope_sin + at);
            }
            qf[s + 0] = t.x, qf[s + 1] = t.y, qf[s + 2] = t.z, qf[s + 3] = t.w;
        }
    }
    /* the keys this lane's query row sees, as absolute positions [vis_lo, vis_hi): block rows
     * see everything, causal rows up to their own position inside the window (kv_cache.c:
     * 229-236), padding rows nothing */
    uint32_t vis_lo = 0, vis_hi = nk;
    if (!a.block_kind) {
        const uint32_t qpos = len + qi;
        vis_hi = min(vis_hi, qpos + 1u);
        if (a.window > 0u && qpos + 1u > a.window) vis_lo = qpos + 1u - a.window;
    }
    if (!q_ok) vis_hi = 0;
    const float scale2 = a.scale * LOG2E;

    floatx4 oacc[DT];
#pragma unroll
    for (int d = 0; d < DT; d++)
#pragma unroll
        for (int r = 0; r < 4; r++) oacc[d][r] = 0.f;
    float m = neg_inf(), l = 0.f;

    float *const my_kt = sm_kt[wave];
    while (si < s_end) {
        const bool fresh = si >= cached_subs;
        const uint32_t j0 = fresh ? len : si * 32u; /* absolute position of the sub-chunk's first key */
        const uint32_t j_end = fresh ? nk : len;    /* rows past it are clamped repeats */
        if (fresh) { /* the new rows: rotate their keys at their own positions, write keys and values through */
#pragma unroll
            for (int v = 0; v < KNV; v++) {
                const uint32_t r = (uint32_t)(KRI * v) + krow_l;
                const bool real = r < a.n;
                if (a.rope_cos && real) {
                    const size_t at = (size_t)(len + r) * HALF + 2u * kpiece;
                    const float4 t = rope_rotate4(make_float4(kg[v][0], kg[v][1], kg[v][2], kg[v][3]), a.rope_cos + at,
                                                  a.rope_sin + at);
                    kg[v][0] = t.x, kg[v][1] = t.y, kg[v][2] = t.z, kg[v][3] = t.w;
                }
                if (a.write_through && head_ok && real) {
                    const size_t at = (slab + len + r) * a.embed_dim + head * HD + 4u * kpiece;
                    *reinterpret_cast<floatx4 *>(a.cache_k + at) = kg[v];
                    *reinterpret_cast<floatx4 *>(a.cache_v + at) = vg[v];
                }
            }
        }
        /* rows -> fragments through the wave's own tile (LDS serves a wave's requests in order: no
         * barrier): tile t holds row 16 t + c, columns g QD ... */
#pragma unroll
        for (int v = 0; v < KNV; v++)
            *reinterpret_cast<floatx4 *>(my_kt + ((uint32_t)(KRI * v) + krow_l) * KROW + 4u * kpiece) = kg[v];
        float kf[2][QD];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int s = 0; s < QD; s += 4) {
                const float4 x = *reinterpret_cast<const float4 *>(my_kt + (16u * t + c) * KROW + g * QD + s);
                kf[t][s + 0] = x.x, kf[t][s + 1] = x.y, kf[t][s + 2] = x.z, kf[t][s + 3] = x.w;
            }
        float vf[DT][8];
#pragma unroll
        for (int v = 0; v < KNV; v++)
            *reinterpret_cast<floatx4 *>(my_kt + ((uint32_t)(KRI * v) + krow_l) * KROW + 4u * kpiece) = vg[v];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const float *vrow = my_kt + (16u * (u >> 2) + (u & 3) + 4u * g) * KROW + DT * c;
            if constexpr (DT == 2) {
                const float2 x = *reinterpret_cast<const float2 *>(vrow);
                vf[0][u] = x.x, vf[1][u] = x.y;
            } else {
                static_assert(DT == 4, "head widths 32 and 64");
                const float4 x = *reinterpret_cast<const float4 *>(vrow);
                vf[0][u] = x.x, vf[1][u] = x.y, vf[2][u] = x.z, vf[3][u] = x.w;
            }
        }
        /* the next sub-chunk's rows travel while this one is worked on: the raw rows have left their
         * registers */
        request(kg, vg, si + a.slices);
        __builtin_amdgcn_sched_barrier(0); /* the requests stay ahead of the arithmetic */

        floatx4 sacc[2];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) sacc[t][r] = 0.f;
#pragma unroll
        for (int s = 0; s < QD; s++) /* the two tiles' chains interleaved: neither waits for its own result */
#pragma unroll
            for (int t = 0; t < 2; t++)
                sacc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t][s], qf[s], sacc[t], 0, 0, 0);

        /* one unsigned compare per key: lo <= j < hi */
        const uint32_t hi = min(vis_hi, j_end);
        const uint32_t span = hi > vis_lo ? hi - vis_lo : 0u;
        const uint32_t rel = j0 + 4u * g - vis_lo;
        float x[8];
        float mt = neg_inf();
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const float t = sacc[u >> 2][u & 3] * scale2;
            const bool vis = ((rel + (16u * (u >> 2) + (u & 3))) < span) & isfinite(t);
            x[u] = vis ? t : neg_inf();
            mt = fmaxf(mt, x[u]);
        }
        mt = swap32(swap16(mt, OpMax()), OpMax());
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
        for (int d = 0; d < DT; d++)
#pragma unroll
            for (int r = 0; r < 4; r++) oacc[d][r] *= alpha;
#pragma unroll
        for (int u = 0; u < 8; u++)
#pragma unroll
            for (int d = 0; d < DT; d++)
                oacc[d] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[d][u], x[u], oacc[d], 0, 0, 0);
        si += a.slices;
    }

    /* the four lane groups of a column carry the same m, their sums add */
    l = swap32(swap16(l, OpSum()), OpSum());

    /* lane (g, c) holds O^T[column DT (4 g + r) + e][query c] in oacc[e][r], i.e. the 4 DT
     * consecutive columns from 4 DT g on: park rows [query][HD columns, max, sum] in the wave's
     * LDS tile */
    float *mine = sm_o[wave];
    if constexpr (DT == 2) {
#pragma unroll
        for (int r = 0; r < 4; r += 2)
            *reinterpret_cast<float4 *>(mine + c * LPR + 8 * g + 2 * r) =
                make_float4(oacc[0][r], oacc[1][r], oacc[0][r + 1], oacc[1][r + 1]);
    } else {
#pragma unroll
        for (int r = 0; r < 4; r++)
            *reinterpret_cast<float4 *>(mine + c * LPR + 16 * g + 4 * r) =
                make_float4(oacc[0][r], oacc[1][r], oacc[2][r], oacc[3][r]);
    }
    if (g == 0) *reinterpret_cast<float2 *>(mine + c * LPR + HD) = make_float2(m * LN2, l); /* merges work in natural units */
    __syncthreads();
    const uint32_t early_ticket = kv_draw_early_ticket(a, b); /* as in the 32-wide kernel */

    kv_merge_slices<HD, WAVES, LPR, (int)ROWS, 32 * KROW>(a, sm_o, hshift, wave, b, split, newrow0, zblock);

    kv_finish_sequence<HD>(a, (uint32_t)SLOTS, b, nk, &sm_ticket, early_ticket);
}

/* The same step for blocks of at most 4 rows and head width 32 on 4x4x1 tiles
 * (v_mfma_f32_4x4x1_16b_f32: 16 independent blocks; lane = 4 * block + i supplies A[i], lane =
 * 4 * block + j supplies B[j], D[i][j] sits in register i of lane 4 * block + j; with cbsz:3 the
 * A operand of block `abid` of each group of eight blocks is used by all eight).  A 16-wide tile
 * with four real query rows spends three quarters of its matrix-core cycles and of its softmax
 * arithmetic on padding; at these sizes a workgroup's time is the number of instructions its
 * waves issue, so a wave takes 64 keys per sub-chunk with nothing padded:
 *
 *   S^T[key, query]: block = 4 consecutive keys, lane = key: the lane holds its K row whole (eight
 *                    16-byte loads) and the row of query lane % 4; one instruction per head
 *                    column; register r of lane (block, j) ends up with key 4 block + r, query j;
 *   O[query, d]:     instruction (beta, r) broadcasts the weights of key 4 beta + r (lower eight
 *                    blocks) and key 32 + 4 beta + r (upper eight) as A; lane l supplies column
 *                    l % 32 of that key's V row as B (the V rows reach the lanes like the K rows:
 *                    coalesced loads, then the wave's LDS tile); register i of lane l accumulates
 *                    O[query i][column l % 32] over the lane's half of the keys.  One accumulator of four registers; the two halves
 *                    meet once, after the loop, with one row swap.
 *
 * The sequence is walked as ceil(len / 64) sub-chunks of cached rows followed by one with the new
 * rows; which of the two a sub-chunk is, is uniform over the wave. */
template <int WAVES, int MAXW, bool LOOP, bool KARG> /* WAVES: slots of the merge (a power of two), MAXW <= WAVES: most waves launched */
__global__ __launch_bounds__(64 * MAXW, 1) void kv_block4_mfma_kernel(StepArgs a, LensArg<KARG> lens) {
    kv_fetch_arguments(a);
    constexpr int HD = 32, HALF = 16;
    constexpr int LPR = HD + 4; /* a parked result row in LDS, 16-byte aligned */
    constexpr uint32_t ROWS = 4, CH = 64;

    constexpr int KROW = HD + 4; /* a K row on its way from its coalesced load to the lane that contracts it */
    __shared__ __attribute__((aligned(16))) float sm_o[WAVES][ROWS * LPR];
    __shared__ uint32_t sm_ticket;
    extern __shared__ __attribute__((aligned(16))) float sm_kt4[]; /* per wave: 32 K rows, KROW floats each */

    const uint32_t b = blockIdx.y;
    const uint32_t split = blockIdx.x;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t hshift = (uint32_t)__builtin_ctz(a.hpb);
    const uint32_t slice = wave >> hshift;
    const uint32_t head = blockIdx.z * a.hpb + (wave & (a.hpb - 1u));
    const bool head_ok = head < a.num_heads;
    const uint32_t hsafe = head_ok ? head : 0u;
    const uint32_t blk = lane >> 2;  /* block of four keys */
    const uint32_t li = lane & 3u;   /* i of the A operand, j (query) of B and D in S^T */
    const uint32_t half = lane >> 5; /* which 32 keys of a sub-chunk this lane contracts in O */
    const uint32_t dcol = lane & 31u;

    const uint32_t len = kv_len_of(a, lens, b) + a.len_bias;
    const uint32_t nk = len + a.n;
    if (!KARG && kv_over_capacity(a, nk)) return; /* uniform over the sequence's workgroups */
    const size_t slab = (size_t)b * a.max_seq_len;
    const size_t newrow0 = (size_t)b * a.n_seq;
    const uint32_t cached_subs = (len + CH - 1u) / CH;
    const uint32_t total_subs = cached_subs + 1u;
    uint32_t s_begin = 0u, s_end = total_subs;
    if (a.splits > 1u) {
        const uint32_t per_split = (total_subs + a.splits - 1u) / a.splits;
        s_begin = split * per_split;
        s_end = min(s_begin + per_split, total_subs);
    }

    const char *const cache_k = reinterpret_cast<const char *>(a.cache_k + slab * a.embed_dim + hsafe * HD);
    const char *const cache_v = reinterpret_cast<const char *>(a.cache_v + slab * a.embed_dim + hsafe * HD);
    const char *const new_k = reinterpret_cast<const char *>(a.k_rows + newrow0 * a.k_stride + hsafe * HD);
    const char *const new_v = reinterpret_cast<const char *>(a.v_rows + newrow0 * a.v_stride + hsafe * HD);
    const uint32_t cache_pitch = a.embed_dim * 4u, newk_pitch = a.k_stride * 4u, newv_pitch = a.v_stride * 4u;
    const uint32_t last_cached = len > 0u ? len - 1u : 0u, last_new = a.n - 1u;

    /* kg[v]: piece lane % 8 of the sub-chunk's row 8 v + lane / 8 -- consecutive lanes on consecutive
     * 16-byte pieces of a row; a load whose lanes each touch another row (lane = key, as the S^T
     * product wants the rows) is served at a quarter of the rate, and eight of those per sub-chunk
     * were most of what the longest sequences waited for.  vg[v]: the same piece of the same row of V
     * (the O product wants column dcol of row 32 half + 4 beta + r in lane (half, dcol): a load of that
     * shape moves 256 bytes per instruction, and thirty-two of them per sub-chunk kept the compute
     * unit's vector memory path busier than the K rows did).  Rows past the last one are clamped to it
     * (their weights are zero).  Base, pitch and limit are scalar selects: every load is scalar base +
     * 32-bit lane offset. */
    const uint32_t krow_l = lane >> 3, kpiece = lane & 7u;
    auto request = [&](floatx4 (&kg)[8], floatx4 (&vg)[8], uint32_t si) __attribute__((always_inline)) {
        const bool fresh = si >= cached_subs;
        const char *kb = fresh ? new_k : cache_k, *vb = fresh ? new_v : cache_v;
        const uint32_t kp = fresh ? newk_pitch : cache_pitch, vp = fresh ? newv_pitch : cache_pitch;
        const uint32_t row0 = fresh ? 0u : si * CH, limit = fresh ? last_new : last_cached;
#pragma unroll
        for (int v = 0; v < 8; v++)
            kg[v] = *reinterpret_cast<const floatx4 *>(kb + __umul24(min(row0 + 8u * v + krow_l, limit), kp) + 16u * kpiece);
#pragma unroll
        for (int v = 0; v < 8; v++)
            vg[v] = *reinterpret_cast<const floatx4 *>(vb + __umul24(min(row0 + 8u * v + krow_l, limit), vp) + 16u * kpiece);
    };

    /* The query rows: lanes 0..3 (block 0) hold row `lane` whole; the S^T instructions hand block
     * 0's A operand to all sixteen blocks, so no other lane needs them (a copy per lane would move
     * as many bytes through the vector memory path as a K sub-chunk does).  Requested first: 4
     * active lanes cost next to nothing and S^T cannot start without them. */
    float4 qr[8];
#pragma unroll
    for (int e = 0; e < 8; e++) qr[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (lane < 4u) {
        const uint32_t row = min(a.q0 + lane, a.n - 1u);
        const char *qp = reinterpret_cast<const char *>(a.q_rows + newrow0 * a.q_stride + hsafe * HD);
        const uint32_t qoff = __umul24(row, a.q_stride * 4u);
#pragma unroll
        for (int e = 0; e < 8; e++) qr[e] = *reinterpret_cast<const float4 *>(qp + qoff + 16 * e);
        if (a.rope_cos) { /* the query sits at position len + row */
            const size_t at = (size_t)(len + row) * HALF;
#pragma unroll
            for (int e = 0; e < 8; e++) qr[e] = rope_rotate4(qr[e], a.rope_cos + at + 2 * e, a.rope_sin + at + 2 * e);
        }
    }
    /* LOOP = false: the launch has a wave for every sub-chunk of every sequence (the host sized it
     * so).  A wave then has one sub-chunk or none; those with none request nothing -- the compute
     * unit's vector memory path (64 bytes a cycle) is what the longest sequences wait for -- and
     * park a neutral record.  LOOP = true: sub-chunks round-robin, the next one requested ahead. */
    uint32_t si = s_begin + slice;
    floatx4 kg[8], vg[8];
    if (LOOP || si < s_end) request(kg, vg, si); /* before anything waits for memory */
    float *const my_kt = sm_kt4 + wave * (32 * KROW);

    const uint32_t qi = a.q0 + li;
    const bool q_ok = qi < a.n;
    uint32_t vis_lo = 0, vis_hi = nk;
    if (!a.block_kind) {
        const uint32_t qpos = len + qi;
        vis_hi = min(vis_hi, qpos + 1u);
        if (a.window > 0u && qpos + 1u > a.window) vis_lo = qpos + 1u - a.window;
    }
    if (!q_ok) vis_hi = 0;
    const float scale2 = a.scale * LOG2E;

    floatx4 oacc; /* register i: O[query i][column dcol], this half's keys */
#pragma unroll
    for (int r = 0; r < 4; r++) oacc[r] = 0.f;
    float m = neg_inf(), l = 0.f;

    /* one sub-chunk whose rows sit in kg / vg */
    auto attend = [&](floatx4 (&kg)[8], floatx4 (&vg)[8], uint32_t si) __attribute__((always_inline)) {
        const bool fresh = si >= cached_subs;
        const uint32_t j0 = fresh ? len : si * CH; /* absolute position of the sub-chunk's first key */
        const uint32_t j_end = fresh ? nk : len;   /* rows past it are clamped repeats */
        if (fresh) { /* the new rows (wave-uniform): rotate their keys, write keys and values through */
#pragma unroll
            for (int v = 0; v < 8; v++) {
                const uint32_t r = 8u * v + krow_l;
                const bool real = r < a.n;
                if (a.rope_cos && real) {
                    const size_t at = (size_t)(len + r) * HALF + 2u * kpiece;
                    const float4 t = rope_rotate4(make_float4(kg[v][0], kg[v][1], kg[v][2], kg[v][3]), a.rope_cos + at,
                                                  a.rope_sin + at);
                    kg[v][0] = t.x, kg[v][1] = t.y, kg[v][2] = t.z, kg[v][3] = t.w;
                }
                if (a.write_through && head_ok && real) {
                    const size_t at = (slab + len + r) * a.embed_dim + head * HD + 4u * kpiece;
                    *reinterpret_cast<floatx4 *>(a.cache_k + at) = kg[v];
                    *reinterpret_cast<floatx4 *>(a.cache_v + at) = vg[v];
                }
            }
        }
        /* rows -> the lanes that contract them, 32 rows at a time through the wave's own LDS tile (LDS
         * serves a wave's requests in order: no barrier): lane l ends up with row l whole */
        float4 kr[8];
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++) {
#pragma unroll
            for (int v = 0; v < 4; v++)
                *reinterpret_cast<floatx4 *>(my_kt + (8u * v + krow_l) * KROW + 4u * kpiece) = kg[4 * h2 + v];
            if (half == (uint32_t)h2) {
#pragma unroll
                for (int e = 0; e < 8; e++) kr[e] = *reinterpret_cast<const float4 *>(my_kt + (lane & 31u) * KROW + 4 * e);
            }
        }
        /* the V rows the same way: lane (half, dcol) ends up with column dcol of rows 32 half ... 32 half + 31 */
        float vr[32];
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++) {
#pragma unroll
            for (int v = 0; v < 4; v++)
                *reinterpret_cast<floatx4 *>(my_kt + (8u * v + krow_l) * KROW + 4u * kpiece) = vg[4 * h2 + v];
            if (half == (uint32_t)h2) {
#pragma unroll
                for (int t = 0; t < 32; t++) vr[t] = my_kt[t * KROW + dcol];
            }
        }

        /* S[query, key]: A = block 0's query rows for every block (cbsz:4 abid:0), B = the lane's K
         * row; two chains (even and odd columns) so that no instruction waits for the one before.
         * Register i of lane (blk, j) ends up with query i against key j0 + 4 blk + j. */
        floatx4 s0, s1;
#pragma unroll
        for (int r = 0; r < 4; r++) s0[r] = 0.f, s1[r] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            s0 = __builtin_amdgcn_mfma_f32_4x4x1f32(qr[e].x, kr[e].x, s0, 4, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_4x4x1f32(qr[e].y, kr[e].y, s1, 4, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_4x4x1f32(qr[e].z, kr[e].z, s0, 4, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_4x4x1f32(qr[e].w, kr[e].w, s1, 4, 0, 0);
        }
        /* 4 x 4 transpose inside each quad of lanes (two exchange steps), so that register r of lane
         * (blk, j) holds key j0 + 4 blk + r against query j: the layout the weights are needed in */
        float sc[4];
#pragma unroll
        for (int r = 0; r < 4; r++) sc[r] = s0[r] + s1[r];
        {
            const bool odd = (li & 1u) != 0u, upper = (li & 2u) != 0u;
#pragma unroll
            for (int p = 0; p < 4; p += 2) { /* registers (p, p + 1) across lanes (j, j ^ 1) */
                const float got = dpp_mov<DPP_XOR1>(odd ? sc[p] : sc[p + 1]);
                sc[p] = odd ? got : sc[p];
                sc[p + 1] = odd ? sc[p + 1] : got;
            }
#pragma unroll
            for (int p = 0; p < 2; p++) { /* registers (p, p + 2) across lanes (j, j ^ 2) */
                const float got = dpp_mov<DPP_XOR2>(upper ? sc[p] : sc[p + 2]);
                sc[p] = upper ? got : sc[p];
                sc[p + 2] = upper ? sc[p + 2] : got;
            }
        }
        /* one unsigned compare per key */
        const uint32_t hi = min(vis_hi, j_end);
        const uint32_t span = hi > vis_lo ? hi - vis_lo : 0u;
        const uint32_t rel = j0 + 4u * blk - vis_lo;
        float x[4];
        float mt = neg_inf();
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float t = sc[r] * scale2;
            const bool vis = ((rel + (uint32_t)r) < span) & isfinite(t);
            x[r] = vis ? t : neg_inf();
            mt = fmaxf(mt, x[r]);
        }
        mt = across_keys<4>(mt, OpMax()); /* over the sixteen blocks, query by query */
        const float mn = fmaxf(m, mt);
        const float ms = mn == neg_inf() ? 0.f : mn;
        const float alpha = fast_exp2(m - ms);
        float ps = 0.f;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            x[r] = fast_exp2(x[r] - ms);
            ps += x[r];
        }
        l = l * alpha + ps; /* this block's keys only */
        m = mn;
        /* accumulator register i belongs to query i, whose factor the lanes with li == i hold */
        oacc[0] *= dpp_mov<0x00>(alpha); /* quad_perm [0,0,0,0] */
        oacc[1] *= dpp_mov<0x55>(alpha); /* quad_perm [1,1,1,1] */
        oacc[2] *= dpp_mov<0xAA>(alpha);
        oacc[3] *= dpp_mov<0xFF>(alpha);
#define BLT_O_STEP(BETA)                                                                                         \
    oacc = __builtin_amdgcn_mfma_f32_4x4x1f32(x[0], vr[4 * BETA + 0], oacc, 3, BETA, 0);                           \
    oacc = __builtin_amdgcn_mfma_f32_4x4x1f32(x[1], vr[4 * BETA + 1], oacc, 3, BETA, 0);                           \
    oacc = __builtin_amdgcn_mfma_f32_4x4x1f32(x[2], vr[4 * BETA + 2], oacc, 3, BETA, 0);                           \
    oacc = __builtin_amdgcn_mfma_f32_4x4x1f32(x[3], vr[4 * BETA + 3], oacc, 3, BETA, 0);
        BLT_O_STEP(0) BLT_O_STEP(1) BLT_O_STEP(2) BLT_O_STEP(3) BLT_O_STEP(4) BLT_O_STEP(5) BLT_O_STEP(6) BLT_O_STEP(7)
#undef BLT_O_STEP
    };

    if constexpr (!LOOP) {
        if (si < s_end) attend(kg, vg, si);
    } else {
        while (si < s_end) {
            floatx4 kn[8], vn[8];
            request(kn, vn, si + a.slices); /* past the end the clamped rows hit the cache; no branch */
            __builtin_amdgcn_sched_barrier(0);
            attend(kg, vg, si);
#pragma unroll
            for (int e = 0; e < 8; e++) kg[e] = kn[e], vg[e] = vn[e];
            si += a.slices;
        }
    }

    /* the two halves of the keys meet; the sixteen blocks' sums of weights meet; m is already common */
#pragma unroll
    for (int r = 0; r < 4; r++) oacc[r] = swap32(oacc[r], OpSum());
    l = across_keys<4>(l, OpSum());

    float *mine = sm_o[wave];
    if (half == 0u) {
#pragma unroll
        for (int i = 0; i < 4; i++) mine[i * LPR + dcol] = oacc[i];
        if (blk == 0u) *reinterpret_cast<float2 *>(mine + li * LPR + HD) = make_float2(m * LN2, l);
    }
    __syncthreads();
    const uint32_t early_ticket = kv_draw_early_ticket(a, b);
    kv_merge_slices<HD, WAVES, LPR, (int)ROWS>(a, sm_o, hshift, wave, b, split, newrow0, blockIdx.z);
    kv_finish_sequence<HD>(a, (uint32_t)SLOTS, b, nk, &sm_ticket, early_ticket);
}

template <int HD, int WAVES, bool NARROW>
void launch_block_as(StepArgs a, uint32_t batch, const uint32_t *host_lens, hipStream_t s) {
    /* a.hpb heads per workgroup (the caller's choice, see kv_block_heads_per_group; a power of two);
     * the other waves are slices */
    a.hpb = std::max(1u, std::min<uint32_t>(std::min<uint32_t>(a.hpb, a.num_heads), (uint32_t)WAVES));
    while (a.hpb & (a.hpb - 1u)) a.hpb &= a.hpb - 1u;
    const uint32_t subs = (a.span + 31u) / 32u;
    /* Long sequences of unequal lengths, more (sequence, head) pairs than compute units, lengths
     * known here: a launch of one workgroup per sequence and head pair ends with its longest
     * sequence (2032 keys against a mean of 1528 is a quarter of the time lost), so the pairs
     * become workgroups of their own, handed out longest first. */
    KargLens lens;
    a.by_length = 0;
    if (NARROW && host_lens && a.splits == 1u && a.num_heads >= 2u && batch >= 2u) {
        uint32_t shortest = host_lens[0], longest = host_lens[0];
        for (uint32_t b = 1; b < batch; b++)
            shortest = std::min(shortest, host_lens[b]), longest = std::max(longest, host_lens[b]);
        const bool pays = (uint64_t)batch * a.num_heads > 256u && subs >= 32u && (longest - shortest) * 5u >= longest;
        if (pays) {
            a.by_length = 1;
            a.hpb = 1;
            uint32_t idx[KARG_SEQS];
            for (uint32_t b = 0; b < batch; b++) idx[b] = b;
            std::stable_sort(idx, idx + batch, [&](uint32_t x, uint32_t y) { return host_lens[x] > host_lens[y]; });
            for (uint32_t b = 0; b < batch; b++) lens.order[b] = (uint8_t)idx[b];
        }
    }
    a.slices = std::max(1u, std::min<uint32_t>((uint32_t)WAVES / a.hpb, subs));
    dim3 grid(a.splits, batch, (a.num_heads + a.hpb - 1) / a.hpb);
    const dim3 block(64 * a.hpb * a.slices);
    if (host_lens) {
        for (uint32_t b = 0; b < batch; b++) lens.v[b] = host_lens[b];
        if constexpr (NARROW) blt_launch("kv_block16_mfma", kv_block16_mfma_kernel<HD, WAVES, true>, grid, block, 0, s, a, lens);
        else blt_launch("kv_block_mfma", kv_block_mfma_kernel<HD, WAVES, true>, grid, block, 0, s, a, lens);
    } else {
        const DeviceLens lens{0u};
        if constexpr (NARROW) blt_launch("kv_block16_mfma", kv_block16_mfma_kernel<HD, WAVES, false>, grid, block, 0, s, a, lens);
        else blt_launch("kv_block_mfma", kv_block_mfma_kernel<HD, WAVES, false>, grid, block, 0, s, a, lens);
    }
}

template <int WAVES, int MAXW, bool LOOP>
void launch_block4_as(const StepArgs &a, uint32_t batch, const uint32_t *host_lens, hipStream_t s) {
    dim3 grid(a.splits, batch, (a.num_heads + a.hpb - 1) / a.hpb);
    const dim3 block(64 * a.hpb * a.slices);
    /* the waves' K tiles: 32 rows of 36 floats each; with sixteen waves more than the 64 KB a kernel
     * may use without asking (the static result rows come on top) */
    constexpr size_t kt_bytes = (size_t)MAXW * 32 * 36 * sizeof(float);
    if (host_lens) {
        static const bool raised = [] {
            HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&kv_block4_mfma_kernel<WAVES, MAXW, LOOP, true>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)kt_bytes));
            return true;
        }();
        (void)raised;
        KargLens lens;
        for (uint32_t b = 0; b < batch; b++) lens.v[b] = host_lens[b];
        blt_launch("kv_block4_mfma", kv_block4_mfma_kernel<WAVES, MAXW, LOOP, true>, grid, block, kt_bytes, s, a, lens);
    } else {
        static const bool raised = [] {
            HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&kv_block4_mfma_kernel<WAVES, MAXW, LOOP, false>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)kt_bytes));
            return true;
        }();
        (void)raised;
        blt_launch("kv_block4_mfma", kv_block4_mfma_kernel<WAVES, MAXW, LOOP, false>, grid, block, kt_bytes, s, a,
                   DeviceLens{0u});
    }
}

void launch_block4(StepArgs a, uint32_t batch, const uint32_t *host_lens, hipStream_t s) {
    a.hpb = std::max(1u, std::min<uint32_t>(std::min<uint32_t>(a.hpb, a.num_heads), 8u));
    while (a.hpb & (a.hpb - 1u)) a.hpb &= a.hpb - 1u;
    /* 64-key sub-chunks of the longest sequence's share, and the one with the new rows */
    const uint32_t subs = (a.span + 63u) / 64u + 1u;
    if (a.splits == 1u && subs * a.hpb <= 16u) { /* a wave for every sub-chunk: no loop, nothing requested ahead */
        a.slices = subs;
        /* the register budget follows the waves actually launched: 256 / 170 / 128 per lane */
        if (subs * a.hpb <= 8u) launch_block4_as<8, 8, false>(a, batch, host_lens, s);
        else if (subs * a.hpb <= 12u) launch_block4_as<16, 12, false>(a, batch, host_lens, s);
        else launch_block4_as<16, 16, false>(a, batch, host_lens, s);
    } else {
        a.slices = std::max(1u, std::min<uint32_t>(8u / a.hpb, subs));
        launch_block4_as<8, 8, true>(a, batch, host_lens, s);
    }
}

/* blocks of up to 16 rows on 16-wide tiles; BLT_HIP_BLOCK_TILE=32 keeps the 32-wide kernel (test hook) */
bool narrow_block(const StepArgs &a) {
    static const bool wide_only = [] {
        const char *e = getenv("BLT_HIP_BLOCK_TILE");
        return e && strcmp(e, "32") == 0;
    }();
    return a.n - a.q0 <= 16u && !wide_only;
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
    /* the per-wave K tiles bound the workgroups: 8 waves of 4.6 KB or 4 of 8.7 KB */
    /* BLT_HIP_BLOCK_TILE=16 keeps blocks of up to four rows on the 16-wide tiles, =4 keeps the looping
     * kernels (4x4x1 tiles up to four rows, 16-wide above), =once takes the all-at-once kernel wherever
     * the shape allows (test hooks) */
    static const int pin = [] {
        const char *e = getenv("BLT_HIP_BLOCK_TILE");
        return !e ? 0 : strcmp(e, "once") == 0 ? 1 : strcmp(e, "4") == 0 ? 4 : strcmp(e, "16") == 0 ? 16 : strcmp(e, "32") == 0 ? 32 : 0;
    }();
    const bool no_tile4 = pin == 16 || pin == 32;
    /* All at once wherever the shape allows, ahead of the looping 16-wide kernel (64 sequences x 4 heads
     * over 64 ... 508 cached keys: 7.0 against 8.0 us at 8 rows, 7.2 against 8.6 at 16); up to four rows
     * of head width 32 the 4x4x1 kernel, which has no padding rows to multiply, stays ahead (6.4 against
     * 6.9 us). */
    const bool small = head_dim == 32u && a.n - a.q0 <= 4u;
    if ((pin == 1 || (pin == 0 && !small)) && kv_block_once_launch(a, batch, head_dim, host_lens, s)) return true;
    if (head_dim == 32u) {
        if (a.n - a.q0 <= 4u && !no_tile4) launch_block4(a, batch, host_lens, s);
        else if (!narrow_block(a)) launch_block_as<32, 8, false>(a, batch, host_lens, s);
        else launch_block_as<32, 8, true>(a, batch, host_lens, s);
    } else if (head_dim == 64u) {
        if (!narrow_block(a)) launch_block_as<64, 4, false>(a, batch, host_lens, s);
        else launch_block_as<64, 4, true>(a, batch, host_lens, s);
    } else {
        return false;
    }
    return true;
}
