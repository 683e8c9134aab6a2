/*
 * "decode" kernel family: the attention statements of one KV-cache step for a
 * whole batch of sequences in one launch -- write the new K/V rows through to
 * the cache, then attend the new query rows over the cached prefix plus the
 * new rows (reference order of operations: csrc/infer/kv_cache.c:343-390).
 *
 * Memory-bound split-KV design, no matrix cores:
 *   - a workgroup owns 32 consecutive cache rows (keys) of one sequence; its
 *     wavefronts are the heads, so together they read whole 4*E-byte rows;
 *   - inside a wave, groups of G = head_dim/4 lanes own one key each per
 *     16-byte load: one load instruction of the wave covers 64/G consecutive
 *     keys, every byte of the fetched lines is used;
 *   - all K and V loads of the chunk are issued before any arithmetic, so a
 *     wave has its whole 32-key chunk in flight at once;
 *   - dot products are reduced across the G lanes with wavefront shuffles,
 *     the per-group partial softmax states (max, sum, output) are merged
 *     across the wave with shuffles too, and one partial per (sequence,
 *     chunk, head, query) goes to a scratch buffer;
 *   - the last workgroup of a sequence to finish (device-scope ticket) merges
 *     that sequence's partials, writes the output rows, and advances the
 *     sequence's length when the step commits.
 */
#include "blt_hip.h"
#include "blt_fatal.h"
#include "hip_check.h"
#include "attn_device.h"
#include "launch.h"

#include <algorithm>

namespace {

/* keys per workgroup: 32, or one full load instruction of the wave if that is more */
constexpr int chunk_keys(int G) { return 64 / G > 32 ? 64 / G : 32; }

struct StepArgs {
    float *cache_k;
    float *cache_v;
    uint32_t *self_len;
    const float *q_rows;
    const float *k_rows;
    const float *v_rows;
    float *combined;
    float *partial;    /* [batch][chunks][heads][NQ][hd + 2] */
    uint32_t *tickets; /* [batch] */
    uint32_t q_stride, k_stride, v_stride, out_stride;
    uint32_t max_seq_len, embed_dim, num_heads, head_dim;
    uint32_t window;
    uint32_t n;        /* new rows per sequence */
    uint32_t q0;       /* first query row this launch handles */
    uint32_t chunks;   /* gridDim.x */
    float scale;
    int block_kind;    /* every new row sees all keys */
    int write_through; /* this launch stores the new rows into the cache */
    int commit;        /* advance self_len when the sequence is done */
};

template <int G>
__device__ __forceinline__ float group_sum(float x) {
#pragma unroll
    for (int o = 1; o < G; o <<= 1) x += __shfl_xor(x, o, 64);
    return x;
}

__device__ __forceinline__ float dot4(float4 a, float4 b) { return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w; }

/* merge softmax state (m2, l2, o2) into (m, l, o) */
__device__ __forceinline__ void merge_state(float &m, float &l, float4 &o, float m2, float l2, float4 o2) {
    const float mn = fmaxf(m, m2);
    const float a = m == neg_inf() ? 0.f : softmax_exp(m - mn);
    const float b = m2 == neg_inf() ? 0.f : softmax_exp(m2 - mn);
    l = l * a + l2 * b;
    o.x = o.x * a + o2.x * b;
    o.y = o.y * a + o2.y * b;
    o.z = o.z * a + o2.z * b;
    o.w = o.w * a + o2.w * b;
    m = mn;
}

/* G lanes per key (head_dim = 4*G), NQ query rows per sequence in this launch,
 * blockDim.x = 64 * heads-per-block, head = blockIdx.z * (blockDim.x/64) + wave. */
template <int G, int NQ>
__global__ __launch_bounds__(256) void kv_step_kernel(StepArgs a) {
    constexpr int KPL = 64 / G;          /* keys per load instruction of a wave */
    constexpr int CHUNK = chunk_keys(G);
    constexpr int LOADS = CHUNK / KPL;   /* loads per lane for K (and for V)   */
    constexpr int HD = 4 * G;
    constexpr int DPL = (HD + 63) / 64;  /* output columns per lane in the final merge */

    __shared__ uint32_t sm_ticket;

    const uint32_t b = blockIdx.y;
    const uint32_t chunk = blockIdx.x;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t head = blockIdx.z * (blockDim.x >> 6) + wave;
    const uint32_t g = lane % G;
    const uint32_t grp = lane / G;
    const bool head_ok = head < a.num_heads;

    const uint32_t len = a.self_len[b];
    const uint32_t nk = len + a.n;
    const uint32_t c0 = chunk * CHUNK;
    const size_t slab = (size_t)b * a.max_seq_len;
    const uint32_t col = head * HD + 4u * g;

    if (c0 < nk && head_ok) {
        /* ---- issue every load of the chunk ---- */
        float4 kf[LOADS], vf[LOADS];
#pragma unroll
        for (int t = 0; t < LOADS; t++) {
            const uint32_t j = min(c0 + grp + KPL * t, nk - 1u);
            if (j < len) {
                kf[t] = *reinterpret_cast<const float4 *>(a.cache_k + (slab + j) * a.embed_dim + col);
                vf[t] = *reinterpret_cast<const float4 *>(a.cache_v + (slab + j) * a.embed_dim + col);
            } else {
                const size_t r = (size_t)b * a.n + (j - len);
                kf[t] = *reinterpret_cast<const float4 *>(a.k_rows + r * a.k_stride + col);
                vf[t] = *reinterpret_cast<const float4 *>(a.v_rows + r * a.v_stride + col);
            }
        }
        float4 q[NQ];
#pragma unroll
        for (int r = 0; r < NQ; r++) {
            const uint32_t qi = min(a.q0 + r, a.n - 1u);
            q[r] = *reinterpret_cast<const float4 *>(a.q_rows + ((size_t)b * a.n + qi) * a.q_stride + col);
        }

        /* ---- write-through of the new rows this chunk holds ---- */
        if (a.write_through) {
#pragma unroll
            for (int t = 0; t < LOADS; t++) {
                const uint32_t j = c0 + grp + KPL * t;
                if (j >= len && j < nk) {
                    *reinterpret_cast<float4 *>(a.cache_k + (slab + j) * a.embed_dim + col) = kf[t];
                    *reinterpret_cast<float4 *>(a.cache_v + (slab + j) * a.embed_dim + col) = vf[t];
                }
            }
        }

        /* ---- scores, chunk-local softmax, PV, merge across the wave ---- */
#pragma unroll
        for (int r = 0; r < NQ; r++) {
            const uint32_t qi = a.q0 + r;
            const uint32_t p = len + qi; /* absolute position of the query */
            float x[LOADS];
            float m = neg_inf();
#pragma unroll
            for (int t = 0; t < LOADS; t++) {
                const uint32_t j = c0 + grp + KPL * t;
                const float s = group_sum<G>(dot4(q[r], kf[t])) * a.scale;
                bool vis = j < nk && qi < a.n;
                if (!a.block_kind) vis = vis && j <= p && (a.window == 0u || p - j < a.window);
                vis = vis && isfinite(s);
                x[t] = vis ? s : neg_inf();
                m = fmaxf(m, x[t]);
            }
            float l = 0.f;
            float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int t = 0; t < LOADS; t++) {
                const float w = x[t] == neg_inf() ? 0.f : softmax_exp(x[t] - m);
                l += w;
                o.x += w * vf[t].x;
                o.y += w * vf[t].y;
                o.z += w * vf[t].z;
                o.w += w * vf[t].w;
            }
#pragma unroll
            for (int off = G; off < 64; off <<= 1) {
                const float m2 = __shfl_xor(m, off, 64);
                const float l2 = __shfl_xor(l, off, 64);
                float4 o2;
                o2.x = __shfl_xor(o.x, off, 64);
                o2.y = __shfl_xor(o.y, off, 64);
                o2.z = __shfl_xor(o.z, off, 64);
                o2.w = __shfl_xor(o.w, off, 64);
                merge_state(m, l, o, m2, l2, o2);
            }
            if (grp == 0) {
                float *dst = a.partial +
                             ((((size_t)b * a.chunks + chunk) * a.num_heads + head) * NQ + r) * (HD + 2);
                *reinterpret_cast<float4 *>(dst + 4u * g) = o;
                if (g == 0) {
                    dst[HD + 0] = m;
                    dst[HD + 1] = l;
                }
            }
        }
    }

    /* ---- ticket: the last workgroup of the sequence merges ---- */
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) sm_ticket = atomicAdd(&a.tickets[b], 1u);
    __syncthreads();
    if (sm_ticket != gridDim.x * gridDim.z - 1u) return;
    __threadfence();

    const uint32_t used = (nk + CHUNK - 1) / CHUNK;
    const uint32_t heads_per_block = blockDim.x >> 6;
    /* this block's waves sweep all heads (other z-blocks have finished) */
    for (uint32_t hh = wave; hh < a.num_heads; hh += heads_per_block) {
        for (uint32_t r = 0; r < (uint32_t)NQ; r++) {
            const uint32_t qi = a.q0 + r;
            if (qi >= a.n) break;
            const float *base = a.partial + (((size_t)b * a.chunks * a.num_heads + hh) * NQ + r) * (HD + 2);
            const size_t cstride = (size_t)a.num_heads * NQ * (HD + 2);
            float M = neg_inf();
            for (uint32_t c = 0; c < used; c++) M = fmaxf(M, base[c * cstride + HD]);
            float L = 0.f, acc[DPL];
#pragma unroll
            for (int e = 0; e < DPL; e++) acc[e] = 0.f;
            for (uint32_t c = 0; c < used; c++) {
                const float *pc = base + c * cstride;
                const float mc = pc[HD];
                const float f = mc == neg_inf() ? 0.f : softmax_exp(mc - M);
                L += pc[HD + 1] * f;
#pragma unroll
                for (int e = 0; e < DPL; e++)
                    if (lane + 64u * e < (uint32_t)HD) acc[e] += pc[lane + 64u * e] * f;
            }
#pragma unroll
            for (int e = 0; e < DPL; e++)
                if (lane + 64u * e < (uint32_t)HD)
                    a.combined[((size_t)b * a.n + qi) * a.out_stride + hh * HD + lane + 64u * e] =
                        L > 0.f ? acc[e] / L : 0.f;
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        a.tickets[b] = 0u;
        if (a.commit) a.self_len[b] = nk;
    }
}

/* scratch the family owns: partial softmax states and per-sequence tickets */
struct Scratch {
    float *partial = nullptr;
    size_t partial_floats = 0;
    uint32_t *tickets = nullptr;
    size_t ticket_count = 0;
};

Scratch &scratch() {
    static thread_local Scratch s;
    return s;
}

template <int G, int NQ>
void launch_step(const StepArgs &a, uint32_t batch, hipStream_t s) {
    const uint32_t hpb = std::min<uint32_t>(a.num_heads, 4u);
    dim3 grid(a.chunks, batch, (a.num_heads + hpb - 1) / hpb);
    blt_launch("kv_step", kv_step_kernel<G, NQ>, grid, dim3(64 * hpb), 0, s, a);
}

template <int G>
void dispatch_nq(const StepArgs &a, uint32_t nq, uint32_t batch, hipStream_t s) {
    if (nq <= 1) launch_step<G, 1>(a, batch, s);
    else if (nq <= 2) launch_step<G, 2>(a, batch, s);
    else if (nq <= 4) launch_step<G, 4>(a, batch, s);
    else if (nq <= 8) launch_step<G, 8>(a, batch, s);
    else launch_step<G, 16>(a, batch, s);
}

} // namespace

extern "C" void blt_kv_attend_step_hip(const blt_kv_attn_cache *cache, const float *q_rows, size_t q_stride,
                                       const float *k_rows, size_t k_stride, const float *v_rows, size_t v_stride,
                                       float *combined, size_t combined_stride, size_t n, int step_kind, int commit,
                                       size_t max_len_hint) {
    BLT_REQUIRE(cache != NULL && cache->self_k != NULL && cache->self_v != NULL && cache->self_len != NULL,
                "blt_kv_attend_step: cache buffers must not be NULL");
    BLT_REQUIRE(q_rows != NULL && k_rows != NULL && v_rows != NULL && combined != NULL,
                "blt_kv_attend_step: row buffers must not be NULL");
    BLT_REQUIRE(n >= 1, "blt_kv_attend_step: need at least one row");
    BLT_REQUIRE(n <= 32, "blt_kv_attend_step: at most 32 new rows per sequence and step "
                         "(longer prefill chunks go through blt_attention_batch_hip)");
    BLT_REQUIRE(step_kind == BLT_KV_STEP_CAUSAL || step_kind == BLT_KV_STEP_BLOCK,
                "blt_kv_attend_step: unknown step_kind");
    const size_t E = cache->embed_dim, H = cache->num_heads;
    BLT_REQUIRE(H >= 1 && E % H == 0, "blt_kv_attend_step: embed_dim must be divisible by num_heads");
    const size_t hd = E / H;
    BLT_REQUIRE(hd == 4 || hd == 8 || hd == 16 || hd == 32 || hd == 64 || hd == 128 || hd == 256,
                "blt_kv_attend_step: head_dim must be a power of two in [4, 256]");
    BLT_REQUIRE(max_len_hint >= n && max_len_hint <= cache->max_seq_len, "blt_kv_attend_step: exceeds cache capacity");
    BLT_REQUIRE(cache->batch >= 1 && cache->batch <= 65535, "blt_kv_attend_step: batch must be in [1, 65535]");
    BLT_REQUIRE(q_stride % 4 == 0 && k_stride % 4 == 0 && v_stride % 4 == 0 && combined_stride >= E &&
                    q_stride >= E && k_stride >= E && v_stride >= E,
                "blt_kv_attend_step: row strides must be multiples of 4 and at least embed_dim");
    BLT_REQUIRE(((reinterpret_cast<uintptr_t>(q_rows) | reinterpret_cast<uintptr_t>(k_rows) |
                  reinterpret_cast<uintptr_t>(v_rows) | reinterpret_cast<uintptr_t>(cache->self_k) |
                  reinterpret_cast<uintptr_t>(cache->self_v)) & 15u) == 0,
                "blt_kv_attend_step: buffers must be 16-byte aligned");

    StepArgs a;
    a.cache_k = cache->self_k;
    a.cache_v = cache->self_v;
    a.self_len = cache->self_len;
    a.q_rows = q_rows;
    a.k_rows = k_rows;
    a.v_rows = v_rows;
    a.combined = combined;
    a.q_stride = (uint32_t)q_stride;
    a.k_stride = (uint32_t)k_stride;
    a.v_stride = (uint32_t)v_stride;
    a.out_stride = (uint32_t)combined_stride;
    a.max_seq_len = (uint32_t)cache->max_seq_len;
    a.embed_dim = (uint32_t)E;
    a.num_heads = (uint32_t)H;
    a.head_dim = (uint32_t)hd;
    a.window = (uint32_t)cache->window;
    a.n = (uint32_t)n;
    const size_t chunk = (size_t)chunk_keys((int)(hd / 4));
    a.chunks = (uint32_t)((max_len_hint + chunk - 1) / chunk);
    a.scale = 1.0f / sqrtf((float)hd);
    a.block_kind = step_kind == BLT_KV_STEP_BLOCK;

    Scratch &sc = scratch();
    const size_t need = cache->batch * (size_t)a.chunks * H * 16u * (hd + 2);
    if (need > sc.partial_floats) {
        if (sc.partial) {
            HIP_CHECK(hipDeviceSynchronize());
            HIP_CHECK(hipFree(sc.partial));
        }
        sc.partial_floats = need;
        HIP_CHECK(hipMalloc((void **)&sc.partial, need * sizeof(float)));
    }
    if (cache->batch > sc.ticket_count) {
        if (sc.tickets) {
            HIP_CHECK(hipDeviceSynchronize());
            HIP_CHECK(hipFree(sc.tickets));
        }
        sc.ticket_count = std::max<size_t>(cache->batch, 1024);
        HIP_CHECK(hipMalloc((void **)&sc.tickets, sc.ticket_count * sizeof(uint32_t)));
        HIP_CHECK(hipMemsetAsync(sc.tickets, 0, sc.ticket_count * sizeof(uint32_t), 0));
    }
    a.partial = sc.partial;
    a.tickets = sc.tickets;

    /* query rows go in slices of at most 16; every slice reads the new rows
     * from the inputs, so only the first one stores them and only the last
     * one may advance the lengths */
    for (uint32_t q0 = 0; q0 < a.n; q0 += 16u) {
        const uint32_t nq = std::min<uint32_t>(16u, a.n - q0);
        a.q0 = q0;
        a.write_through = q0 == 0;
        a.commit = commit && (q0 + 16u >= a.n);
        switch (hd) {
        case 4: dispatch_nq<1>(a, nq, (uint32_t)cache->batch, 0); break;
        case 8: dispatch_nq<2>(a, nq, (uint32_t)cache->batch, 0); break;
        case 16: dispatch_nq<4>(a, nq, (uint32_t)cache->batch, 0); break;
        case 32: dispatch_nq<8>(a, nq, (uint32_t)cache->batch, 0); break;
        case 64: dispatch_nq<16>(a, nq, (uint32_t)cache->batch, 0); break;
        case 128: dispatch_nq<32>(a, nq, (uint32_t)cache->batch, 0); break;
        default: dispatch_nq<64>(a, nq, (uint32_t)cache->batch, 0); break;
        }
    }
    HIP_CHECK_LAUNCH("blt_kv_attend_step");
}
