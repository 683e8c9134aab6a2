/*
 * Single-row decode kernel of the KV-cache step: one new row per sequence
 * (csrc/infer/kv_cache.c:343-390 with n = 1), one workgroup per (sequence,
 * head).  Built around the latency chain of a step that moves a few tens of
 * megabytes: at these sizes the time is not bandwidth but the number of
 * dependent trips between kernel entry and the last store.
 *
 *   - the W waves of a workgroup take the sequence's key groups round-robin;
 *     G = head_dim / 4 lanes own one key per 16-byte load, as in the split
 *     kernel, so every fetched line is used whole;
 *   - every address is a select, not a branch: the new row comes from the
 *     step's inputs, cached rows from the slab, rows past the end are clamped
 *     and masked.  The loop body has no branch around a load, so the rows of
 *     the next round are in flight while this round is worked on;
 *   - lengths come from the kernel arguments when the host has them (the
 *     reference keeps self_len on the host, csrc/infer/kv_cache.h:56-60):
 *     the first K/V requests then depend on nothing but the argument block.
 *     The device-length form reads self_len[b] and commits through the ticket;
 *   - cross-lane arithmetic stays in the vector ALU: sums over the lanes of a
 *     key with DPP row operations, across keys of a wave with DPP rotations
 *     and the gfx950 row swaps (v_permlane16_swap / v_permlane32_swap) -- no
 *     trip through the LDS crossbar;
 *   - one maximum per wave and round (wave-uniform), so the merge of a wave's
 *     key groups is five plain sums, no exponentials;
 *   - the waves meet once: each parks (max, sum, output) in LDS, one barrier,
 *     wave 0 rescales and adds the W records and stores the row.
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

namespace {

__device__ __forceinline__ float dot4(float4 a, float4 b) { return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w; }

/* G lanes per key, W waves per workgroup; KARG: lengths from the argument block, no commit.
 * A wave takes 32 keys per round with at most four 16-byte loads each of K and V per lane (eight
 * loads per lane and round were measured too: no gain at 4 and 8 waves, register spills at 16). */
template <int G, int W, bool KARG>
__global__ __launch_bounds__(64 * W) void kv_row_kernel(StepArgs a, LensArg<KARG> lens) {
    constexpr int KPL = 64 / G; /* keys per load instruction of a wave */
    constexpr int LOADS = SUB / KPL < 1 ? 1 : (SUB / KPL > 4 ? 4 : SUB / KPL);
    constexpr int STEP = LOADS * KPL; /* keys a wave takes per round */
    constexpr int HD = 4 * G;
    constexpr int PR = HD + 2;

    __shared__ float sm[W * PR]; /* per wave: HD output columns, max, sum */

    const uint32_t b = blockIdx.y;
    const uint32_t head = blockIdx.x;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t g = lane % G;
    const uint32_t grp = lane / G;

    const uint32_t len = kv_len_of(a, lens, b);
    const uint32_t nk = len + 1u;
    if (!KARG && kv_over_capacity(a, nk)) return; /* uniform over the sequence's workgroups */

    const size_t slab = (size_t)b * a.max_seq_len;
    const uint32_t col = head * HD + 4u * g;
    const float *const cache_k = a.cache_k + slab * a.embed_dim + col;
    const float *const cache_v = a.cache_v + slab * a.embed_dim + col;
    const float *const new_k = a.k_rows + (size_t)b * a.k_stride + col;
    const float *const new_v = a.v_rows + (size_t)b * a.v_stride + col;
    const uint32_t E = a.embed_dim;

    /* the keys the row sees: [vlo, nk) -- its own position is len (kv_cache.c:229-236) */
    uint32_t vlo = 0u;
    if (a.window > 0u && nk > a.window) vlo = nk - a.window;
    const uint32_t vlen = nk - vlo;
    constexpr uint32_t ROUND = (uint32_t)(W * STEP);
    const uint32_t first = (vlo / ROUND) * ROUND; /* whole rounds before the window are skipped */

    auto fetch = [&](uint32_t c0, float4 (&kf)[LOADS], float4 (&vf)[LOADS]) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < LOADS; t++) {
            const uint32_t j = min(c0 + grp + KPL * t, len);
            const bool cached = j < len;
            const float *kp = cached ? cache_k + (size_t)j * E : new_k;
            const float *vp = cached ? cache_v + (size_t)j * E : new_v;
            kf[t] = *reinterpret_cast<const float4 *>(kp);
            vf[t] = *reinterpret_cast<const float4 *>(vp);
        }
    };

    uint32_t c0 = first + wave * STEP;
    float4 kf[LOADS], vf[LOADS];
    fetch(c0, kf, vf); /* unconditional: rows past the end are clamped to the new row */
    float4 q = *reinterpret_cast<const float4 *>(a.q_rows + (size_t)b * a.q_stride + col);
    float2 rc = make_float2(1.f, 1.f), rs = make_float2(0.f, 0.f);
    if (a.rope_cos) { /* the query and the new key both sit at position len */
        const size_t at = (size_t)len * (HD / 2) + 2u * g;
        rc = *reinterpret_cast<const float2 *>(a.rope_cos + at);
        rs = *reinterpret_cast<const float2 *>(a.rope_sin + at);
        q = rope_rotate4(q, &rc.x, &rs.x);
    }

    float m = neg_inf(), l = 0.f;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    while (c0 < nk) {
        const uint32_t cn = c0 + ROUND;
        float4 kn[LOADS], vn[LOADS];
        fetch(cn, kn, vn); /* no branch around the requests: the wait below counts exactly these */
        __builtin_amdgcn_sched_barrier(0); /* the requests stay ahead of the work */

        float x[LOADS];
        float mt = neg_inf();
#pragma unroll
        for (int t = 0; t < LOADS; t++) {
            const uint32_t j = c0 + grp + KPL * t;
            if (j == len) { /* the new row: rotate, write through (one lane group of one wave) */
                if (a.rope_cos) kf[t] = rope_rotate4(kf[t], &rc.x, &rs.x);
                *reinterpret_cast<float4 *>(a.cache_k + (slab + len) * E + col) = kf[t];
                *reinterpret_cast<float4 *>(a.cache_v + (slab + len) * E + col) = vf[t];
            }
            const float s = key_sum<G>(dot4(q, kf[t])) * a.scale;
            const bool vis = ((j - vlo) < vlen) & isfinite(s);
            x[t] = vis ? s : neg_inf();
            mt = fmaxf(mt, x[t]);
        }
        mt = across_keys<G>(mt, OpMax());
        const float mn = fmaxf(m, mt);
        const float ms = mn == neg_inf() ? 0.f : mn; /* nothing seen yet: keep the differences defined */
        const float alpha = softmax_exp(m - ms);     /* exp(-inf) = 0 on the first round */
        l *= alpha;
        o.x *= alpha, o.y *= alpha, o.z *= alpha, o.w *= alpha;
#pragma unroll
        for (int t = 0; t < LOADS; t++) {
            const float w = softmax_exp(x[t] - ms);
            l += w;
            o.x += w * vf[t].x;
            o.y += w * vf[t].y;
            o.z += w * vf[t].z;
            o.w += w * vf[t].w;
        }
        m = mn;
#pragma unroll
        for (int t = 0; t < LOADS; t++) kf[t] = kn[t], vf[t] = vn[t];
        c0 = cn;
    }

    /* the keys of the wave: plain sums (one maximum for all of them).  Every lane of a key
     * carries the same l; the output columns differ by g. */
    l = across_keys<G>(l, OpSum());
    o.x = across_keys<G>(o.x, OpSum());
    o.y = across_keys<G>(o.y, OpSum());
    o.z = across_keys<G>(o.z, OpSum());
    o.w = across_keys<G>(o.w, OpSum());
    float *mine = sm + wave * PR;
    if (grp == 0) {
        *reinterpret_cast<float2 *>(mine + 4u * g) = make_float2(o.x, o.y);
        *reinterpret_cast<float2 *>(mine + 4u * g + 2u) = make_float2(o.z, o.w);
        if (g == 0) {
            mine[HD] = m;
            mine[HD + 1] = l;
        }
    }
    __syncthreads();
    if (wave != 0) return;

    /* every wave has read the old length: commit (device lengths only), then merge the W records */
    if (!KARG && a.commit && lane == 0) {
        if (gridDim.x == 1u) {
            a.self_len[b] = nk;
        } else {
            const uint32_t ticket = __hip_atomic_fetch_add(&a.tickets[b], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (ticket == gridDim.x - 1u) {
                a.tickets[b] = 0u; /* re-armed for the next launch */
                a.self_len[b] = nk;
            }
        }
    }
    const float mw = lane < (uint32_t)W ? sm[lane * PR + HD] : neg_inf();
    const float lw = lane < (uint32_t)W ? sm[lane * PR + HD + 1] : 0.f;
    const float M = first_lane(row0_all(mw, OpMax()));
    const float f = mw == neg_inf() ? 0.f : softmax_exp(mw - M);
    const float L = first_lane(row0_all(f * lw, OpSum()));
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    float *out = a.combined + (size_t)b * a.out_stride + head * HD;
    for (uint32_t d = lane; d < (uint32_t)HD; d += 64u) {
        float acc = 0.f;
#pragma unroll
        for (int s = 0; s < W; s++) acc += lane_value(f, s) * sm[s * PR + d];
        out[d] = acc * inv;
    }
}

template <int G, int W>
void launch_row(const StepArgs &a, uint32_t batch, const uint32_t *host_lens, hipStream_t s) {
    dim3 grid(a.num_heads, batch, 1);
    if (host_lens) {
        KargLens lens;
        for (uint32_t b = 0; b < batch; b++) lens.v[b] = host_lens[b];
        blt_launch("kv_row", kv_row_kernel<G, W, true>, grid, dim3(64 * W), 0, s, a, lens);
    } else {
        blt_launch("kv_row", kv_row_kernel<G, W, false>, grid, dim3(64 * W), 0, s, a, DeviceLens{0u});
    }
}

template <int G>
void launch_row_waves(const StepArgs &a, uint32_t batch, const uint32_t *host_lens, uint32_t waves, hipStream_t s) {
    if (waves >= 16) launch_row<G, 16>(a, batch, host_lens, s);
    else if (waves >= 8) launch_row<G, 8>(a, batch, host_lens, s);
    else launch_row<G, 4>(a, batch, host_lens, s);
}

} // namespace

/* One new row per sequence, one workgroup per (sequence, head).  `host_lens` (batch entries, at
 * most KARG_SEQS) or NULL for the device lengths in a.self_len.  max_keys sizes the
 * workgroups (measured at 64 sequences x 4 heads x <= 790 keys: 5.2 us with 8 waves, 5.5 with 16,
 * 6.0 with 4; at 128 sequences x 1024..2048 keys: 33.8 us with 16 waves, 34.4 with 8, 35.8 with 4). */
bool kv_row_launch(const StepArgs &a, uint32_t batch, uint32_t head_dim, const uint32_t *host_lens, uint32_t max_keys,
                   hipStream_t s) {
    const uint32_t keys_per_wave = head_dim >= 128 ? 8u : head_dim >= 64 ? 16u : head_dim >= 8 ? 32u : 64u;
    const uint32_t rounds = (max_keys + keys_per_wave - 1) / keys_per_wave;
    const uint32_t waves = rounds > 32 ? 16u : rounds > 4 ? 8u : 4u;
    switch (head_dim) {
    case 4: launch_row_waves<1>(a, batch, host_lens, waves, s); break;
    case 8: launch_row_waves<2>(a, batch, host_lens, waves, s); break;
    case 16: launch_row_waves<4>(a, batch, host_lens, waves, s); break;
    case 32: launch_row_waves<8>(a, batch, host_lens, waves, s); break;
    case 64: launch_row_waves<16>(a, batch, host_lens, waves, s); break;
    case 128: launch_row_waves<32>(a, batch, host_lens, waves, s); break;
    default: return false;
    }
    return true;
}
