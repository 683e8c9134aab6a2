/*
 * "decode" kernel family: the attention statements of one KV-cache step for a
 * whole batch of sequences in one launch -- write the new K/V rows through to
 * the cache, then attend the new query rows over the cached prefix plus the
 * new rows (reference order of operations: csrc/infer/kv_cache.c:343-390).
 *
 * Memory-bound split-KV design, no matrix cores:
 *   - the keys of a sequence are cut into `splits` contiguous spans, one
 *     workgroup each, so that batch x splits workgroups fill the chip;
 *   - a workgroup has one wavefront per (head, slice): the waves of one slice
 *     are the heads and read whole 4*E-byte cache rows between them, the
 *     slices take the span's 32-key sub-chunks round-robin;
 *   - inside a wave, groups of G = head_dim/4 lanes own one key each per
 *     16-byte load: one load instruction of the wave covers 64/G consecutive
 *     keys and every byte of the fetched lines is used; the next sub-chunk is
 *     requested before the current one is consumed;
 *   - dot products are reduced across the G lanes with wavefront shuffles;
 *     each lane group keeps an online-softmax state (max, sum, output) over
 *     its keys, the groups of a wave merge with shuffles once at the end;
 *   - slices merge through LDS; with more than one split the per-split
 *     states go to a small scratch buffer and the last workgroup of the
 *     sequence to finish (device-scope ticket) merges them, writes the output
 *     rows and advances the sequence's length when the step commits.
 */
#include "blt_hip.h"
#include "blt_fatal.h"
#include "hip_check.h"
#include "attn_device.h"
#include "kv_step.h"
#include "launch.h"

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

namespace {

template <int G>
__device__ __forceinline__ float group_sum(float x) {
#pragma unroll
    for (int o = 1; o < G; o <<= 1) x += __shfl_xor(x, o, 64);
    return x;
}

__device__ __forceinline__ float dot4(float4 a, float4 b) { return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w; }

/* G lanes per key (head_dim = 4*G), NQ query rows per launch, at most WAVES
 * waves per workgroup. */
template <int G, int NQ, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void kv_step_kernel(StepArgs a) {
    constexpr int KPL = 64 / G;                    /* keys per load instruction of a wave */
    /* loads per lane and sub-chunk: at most four 16-byte loads each for K and V */
    constexpr int LOADS = SUB / KPL < 1 ? 1 : (SUB / KPL > 4 ? 4 : SUB / KPL);
    constexpr int STEP = LOADS * KPL;              /* keys a wave consumes per sub-chunk  */
    constexpr int HD = 4 * G;

    extern __shared__ float sm[];                  /* [waves][NQ][HD + 2] */
    __shared__ uint32_t sm_ticket;

    const uint32_t b = blockIdx.y;
    const uint32_t split = blockIdx.x;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t slice = wave / a.hpb;
    const uint32_t head = blockIdx.z * a.hpb + wave % a.hpb;
    const uint32_t g = lane % G;
    const uint32_t grp = lane / G;
    const bool head_ok = head < a.num_heads;

    const uint32_t len = a.self_len[b] + a.len_bias;
    const uint32_t nk = len + a.n;
    if (kv_over_capacity(a, nk)) return; /* uniform over the sequence's workgroups */
    const size_t slab = (size_t)b * a.max_seq_len;
    const uint32_t col = (head_ok ? head : 0u) * HD + 4u * g;
    const uint32_t span = kv_span_of(a, nk);
    const uint32_t k_begin = split * span;
    const uint32_t k_end = min(k_begin + span, nk);

    float4 q[NQ], o[NQ];
    float m[NQ], l[NQ];
#pragma unroll
    for (int r = 0; r < NQ; r++) {
        const uint32_t qi = min(a.q0 + r, a.n - 1u);
        q[r] = *reinterpret_cast<const float4 *>(a.q_rows + ((size_t)b * a.n_seq + qi) * a.q_stride + col);
        if (a.rope_cos) { /* the query sits at position len + qi */
            const size_t at = (size_t)(len + qi) * (HD / 2) + 2u * g;
            q[r] = rope_rotate4(q[r], a.rope_cos + at, a.rope_sin + at);
        }
        o[r] = make_float4(0.f, 0.f, 0.f, 0.f);
        m[r] = neg_inf();
        l[r] = 0.f;
    }

    auto fetch = [&](uint32_t c0, float4 (&kf)[LOADS], float4 (&vf)[LOADS]) {
#pragma unroll
        for (int t = 0; t < LOADS; t++) {
            const uint32_t j = min(c0 + grp + KPL * t, nk - 1u);
            if (j < len) {
                kf[t] = *reinterpret_cast<const float4 *>(a.cache_k + (slab + j) * a.embed_dim + col);
                vf[t] = *reinterpret_cast<const float4 *>(a.cache_v + (slab + j) * a.embed_dim + col);
            } else {
                const size_t r = (size_t)b * a.n_seq + (j - len);
                kf[t] = *reinterpret_cast<const float4 *>(a.k_rows + r * a.k_stride + col);
                vf[t] = *reinterpret_cast<const float4 *>(a.v_rows + r * a.v_stride + col);
                if (a.rope_cos) { /* a new key row is rotated at its own position j */
                    const size_t at = (size_t)j * (HD / 2) + 2u * g;
                    kf[t] = rope_rotate4(kf[t], a.rope_cos + at, a.rope_sin + at);
                }
            }
        }
    };

    /* the same for a sub-chunk that lies entirely in the cached prefix: no branch, one address form */
    auto fetch_cached = [&](uint32_t c0, float4 (&kf)[LOADS], float4 (&vf)[LOADS]) __attribute__((always_inline)) {
        const float *kb = a.cache_k + (slab + c0 + grp) * a.embed_dim + col;
        const float *vb = a.cache_v + (slab + c0 + grp) * a.embed_dim + col;
#pragma unroll
        for (int t = 0; t < LOADS; t++) {
            kf[t] = *reinterpret_cast<const float4 *>(kb + (size_t)(KPL * t) * a.embed_dim);
            vf[t] = *reinterpret_cast<const float4 *>(vb + (size_t)(KPL * t) * a.embed_dim);
        }
    };

    /* scores, online softmax and weighted sum of one sub-chunk for every query row of the launch */
    auto attend = [&](uint32_t c0, const float4 (&kf)[LOADS], const float4 (&vf)[LOADS]) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < NQ; r++) {
            const uint32_t qi = a.q0 + r;
            const uint32_t p = len + qi; /* absolute position of the query */
            /* the keys this row sees within the span, [vlo, vlo + vlen): everything up to the span's
             * end for block rows, up to its own position and inside the window for causal rows
             * (kv_cache.c:229-236), nothing for padding rows; one unsigned compare per key */
            uint32_t vhi = k_end, vlo = 0u;
            if (!a.block_kind) {
                vhi = min(vhi, p + 1u);
                if (a.window > 0u && p + 1u > a.window) vlo = p + 1u - a.window;
            }
            if (qi >= a.n) vhi = 0u;
            const uint32_t vlen = vhi > vlo ? vhi - vlo : 0u;
            float x[LOADS];
            float mt = neg_inf();
#pragma unroll
            for (int t = 0; t < LOADS; t++) {
                const uint32_t j = c0 + grp + KPL * t;
                const float s = group_sum<G>(dot4(q[r], kf[t])) * a.scale;
                const bool vis = ((j - vlo) < vlen) & isfinite(s);
                x[t] = vis ? s : neg_inf();
                mt = fmaxf(mt, x[t]);
            }
            const float mn = fmaxf(m[r], mt);
            const float alpha = m[r] == neg_inf() ? 0.f : softmax_exp(m[r] - mn);
            float ls = 0.f;
            float4 acc = make_float4(o[r].x * alpha, o[r].y * alpha, o[r].z * alpha, o[r].w * alpha);
#pragma unroll
            for (int t = 0; t < LOADS; t++) {
                const float w = x[t] == neg_inf() ? 0.f : softmax_exp(x[t] - mn);
                ls += w;
                acc.x += w * vf[t].x;
                acc.y += w * vf[t].y;
                acc.z += w * vf[t].z;
                acc.w += w * vf[t].w;
            }
            o[r] = acc;
            l[r] = l[r] * alpha + ls;
            m[r] = mn;
        }
    };

    const uint32_t stride = a.slices * STEP;
    uint32_t c0 = k_begin + slice * STEP;
    float4 kf[LOADS], vf[LOADS];
    if (c0 < k_end) fetch(c0, kf, vf);
    /* Cached sub-chunks first, in a loop whose body has no branch around a
     * load or a store: the rows of the next sub-chunk are requested, then
     * this one is worked on, and the wait before the work counts exactly the
     * requests issued after its own rows.  (With branches around the loads
     * the wait falls back to "everything", next sub-chunk included.) */
    while (c0 + stride + STEP <= len && c0 + stride < k_end) {
        float4 kn[LOADS], vn[LOADS];
        fetch_cached(c0 + stride, kn, vn);
        __builtin_amdgcn_sched_barrier(0); /* requests stay ahead of the work */
        attend(c0, kf, vf);
#pragma unroll
        for (int t = 0; t < LOADS; t++) {
            kf[t] = kn[t];
            vf[t] = vn[t];
        }
        c0 += stride;
    }
    /* the last sub-chunks of the slice: may hold the new rows (rotation, write-through) */
    while (c0 < k_end) {
        const uint32_t cn = c0 + stride;
        float4 kn[LOADS], vn[LOADS];
        if (cn < k_end) fetch(cn, kn, vn);

        /* write-through of the new rows this sub-chunk holds */
        if (a.write_through && head_ok) {
#pragma unroll
            for (int t = 0; t < LOADS; t++) {
                const uint32_t j = c0 + grp + KPL * t;
                if (j >= len && j < k_end) {
                    *reinterpret_cast<float4 *>(a.cache_k + (slab + j) * a.embed_dim + col) = kf[t];
                    *reinterpret_cast<float4 *>(a.cache_v + (slab + j) * a.embed_dim + col) = vf[t];
                }
            }
        }
        attend(c0, kf, vf);
#pragma unroll
        for (int t = 0; t < LOADS; t++) {
            kf[t] = kn[t];
            vf[t] = vn[t];
        }
        c0 = cn;
    }

    /* ---- merge the lane groups of the wave, park the wave's state in LDS ---- */
    float *mine = sm + (size_t)wave * NQ * (HD + 2);
#pragma unroll
    for (int r = 0; r < NQ; r++) {
#pragma unroll
        for (int off = G; off < 64; off <<= 1) {
            const float m2 = __shfl_xor(m[r], off, 64);
            const float l2 = __shfl_xor(l[r], off, 64);
            float4 o2;
            o2.x = __shfl_xor(o[r].x, off, 64);
            o2.y = __shfl_xor(o[r].y, off, 64);
            o2.z = __shfl_xor(o[r].z, off, 64);
            o2.w = __shfl_xor(o[r].w, off, 64);
            const float mn = fmaxf(m[r], m2);
            const float fa = m[r] == neg_inf() ? 0.f : softmax_exp(m[r] - mn);
            const float fb = m2 == neg_inf() ? 0.f : softmax_exp(m2 - mn);
            l[r] = l[r] * fa + l2 * fb;
            o[r].x = o[r].x * fa + o2.x * fb;
            o[r].y = o[r].y * fa + o2.y * fb;
            o[r].z = o[r].z * fa + o2.z * fb;
            o[r].w = o[r].w * fa + o2.w * fb;
            m[r] = mn;
        }
        if (grp == 0) {
            float *dst = mine + r * (HD + 2) + 4u * g;
            dst[0] = o[r].x;
            dst[1] = o[r].y;
            dst[2] = o[r].z;
            dst[3] = o[r].w;
            if (g == 0) {
                mine[r * (HD + 2) + HD + 0] = m[r];
                mine[r * (HD + 2) + HD + 1] = l[r];
            }
        }
    }
    __syncthreads();
    /* every wave of the workgroup has long read the old length: draw the ticket now, look at it last */
    const uint32_t early_ticket = kv_draw_early_ticket(a, b);

    /* ---- merge the slices, in two steps so that the exponentials are spread over all waves:
     * every wave rescales its own parked state to the common maximum of its head's slices
     * (nobody's maximum is overwritten), then thread t owns (local head, query, column) and adds
     * the slices up ---- */
    {
        const uint32_t hl = wave % a.hpb;
#pragma unroll
        for (int r = 0; r < NQ; r++) {
            float M = neg_inf();
            for (uint32_t s = 0; s < a.slices; s++)
                M = fmaxf(M, sm[((size_t)(s * a.hpb + hl) * NQ + r) * (HD + 2) + HD]);
            const float own = mine[r * (HD + 2) + HD];
            const float f = own == neg_inf() ? 0.f : softmax_exp(own - M);
            for (uint32_t d = lane; d < (uint32_t)HD + 2u; d += 64u)
                if (d != (uint32_t)HD) mine[r * (HD + 2) + d] *= f;
        }
    }
    __syncthreads();
    const uint32_t cells = a.hpb * NQ * HD;
    for (uint32_t t = threadIdx.x; t < cells; t += blockDim.x) {
        const uint32_t d = t % HD;
        const uint32_t r = (t / HD) % NQ;
        const uint32_t hl = t / (HD * NQ);
        const uint32_t hh = blockIdx.z * a.hpb + hl;
        const uint32_t qi = a.q0 + r;
        if (hh >= a.num_heads || qi >= a.n) continue;
        float L = 0.f, acc = 0.f;
        for (uint32_t s = 0; s < a.slices; s++) {
            const float *ps = sm + ((size_t)(s * a.hpb + hl) * NQ + r) * (HD + 2);
            L += ps[HD + 1];
            acc += ps[d];
        }
        if (a.splits == 1u) {
            a.combined[((size_t)b * a.n_seq + qi) * a.out_stride + hh * HD + d] = L > 0.f ? acc / L : 0.f;
        } else {
            float *dst = a.partial + ((((size_t)b * a.splits + split) * a.num_heads + hh) * NQ + r) * (HD + 2);
            publish(dst + d, acc);
            if (d == 0) {
                float M = neg_inf();
                for (uint32_t s = 0; s < a.slices; s++)
                    M = fmaxf(M, sm[((size_t)(s * a.hpb + hl) * NQ + r) * (HD + 2) + HD]);
                publish(dst + HD + 0, M);
                publish(dst + HD + 1, L);
            }
        }
    }

    kv_finish_sequence<HD>(a, (uint32_t)NQ, b, nk, &sm_ticket, early_ticket);
}

/* ---- device memory the family owns beyond inputs and outputs ----
 * per-split softmax records [batch][splits][heads][slots][hd + 2], per-sequence tickets [batch]
 * and one sticky error word.
 *
 * Growing entry points (blt_kv_attend_step_hip and everything built on it): one set per (host
 * thread, stream), so that steps issued on two streams never share tickets or records.  The
 * buffers only grow, and a buffer that is replaced by a larger one is kept until the process
 * ends: a graph captured earlier holds the old addresses in its kernel arguments and must stay
 * replayable.
 *
 * blt_kv_attend_step_noalloc_hip: the same records and tickets in a file-scope device array of
 * fixed size (`scratch`), one copy per GPU, whose address is looked up once per device. */
struct Scratch {
    float *partial = nullptr;
    size_t partial_floats = 0;
    uint32_t *tickets = nullptr;
    size_t ticket_count = 0;
};

constexpr size_t STATIC_PARTIAL_FLOATS = (size_t)1 << 20; /* 4 MiB of per-split records            */
constexpr size_t STATIC_TICKETS = 4096;                   /* sequences per call                     */
constexpr size_t STATIC_WORDS = 64;                       /* error word + padding to 256 bytes      */
constexpr size_t STATIC_BYTES = STATIC_PARTIAL_FLOATS * sizeof(float) + STATIC_TICKETS * sizeof(uint32_t) +
                                STATIC_WORDS * sizeof(uint32_t);
static __device__ __align__(256) unsigned char scratch[STATIC_BYTES];

constexpr int MAX_DEVICES = 64;
struct DeviceStatics {
    unsigned char *base = nullptr; /* device address of `scratch` on this GPU */
    float *partial() const { return reinterpret_cast<float *>(base); }
    uint32_t *tickets() const { return reinterpret_cast<uint32_t *>(base + STATIC_PARTIAL_FLOATS * sizeof(float)); }
    uint32_t *error() const { return tickets() + STATIC_TICKETS; }
};
DeviceStatics g_statics[MAX_DEVICES];
std::mutex g_statics_lock;
std::atomic<uint32_t> g_unchecked_steps{0}; /* device-length steps issued since the error word was last read */

/* The current device's copy of `scratch`: looked up on the first call on that device (each GPU
 * holds its own copy at its own address).  The array is zero when the code object is loaded and
 * every launch leaves tickets and error word as it found them, so nothing has to be cleared. */
const DeviceStatics &statics() {
    int dev = 0;
    HIP_CHECK(hipGetDevice(&dev));
    BLT_REQUIRE(dev >= 0 && dev < MAX_DEVICES, "device index %d out of range", dev);
    std::lock_guard<std::mutex> hold(g_statics_lock);
    if (!g_statics[dev].base) {
        void *ptr = nullptr;
        HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        BLT_REQUIRE(ptr != nullptr, "hipGetSymbolAddress returned no address for the KV step scratch");
        g_statics[dev].base = static_cast<unsigned char *>(ptr);
    }
    return g_statics[dev];
}

struct GrowingScratch {
    std::map<hipStream_t, Scratch> by_stream;
    std::map<hipStream_t, std::pair<uint32_t *, size_t>> lens_by_stream; /* staged host lengths */
    std::vector<void *> retired; /* replaced by larger buffers; live graphs may still name them */
};

GrowingScratch &growing() {
    static thread_local GrowingScratch g;
    return g;
}

/* Device copy of the caller's host lengths for this step (grow-only, per stream; ordered on the
 * stream like every launch, so the next step's copy cannot overtake this step's kernels). */
uint32_t *staged_lengths(const uint32_t *host_lens, size_t batch) {
    GrowingScratch &g = growing();
    auto &slot = g.lens_by_stream[blt_stream_key()];
    BLT_REQUIRE(!blt_stream_capturing(), "blt_kv_attend_step_lens: host lengths cannot be staged while a graph capture is open");
    if (batch > slot.second) {
        if (slot.first) g.retired.push_back(slot.first);
        slot.second = std::max<size_t>(2 * batch, 1024);
        HIP_CHECK(hipMalloc((void **)&slot.first, slot.second * sizeof(uint32_t)));
    }
    blt_upload_staged(slot.first, host_lens, batch * sizeof(uint32_t));
    return slot.first;
}

/* tickets must start at zero; a fill kernel, not a memset node, so that a capture could hold it */
__global__ void kv_clear_words_kernel(uint32_t *p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

template <int G, int NQ, int WAVES>
void launch_step(StepArgs a, uint32_t batch, hipStream_t s) {
    constexpr int HD = 4 * G;
    /* a.hpb == 0: as many heads per workgroup as there are waves */
    a.hpb = std::min<uint32_t>(a.num_heads, a.hpb ? std::min<uint32_t>(a.hpb, (uint32_t)WAVES) : (uint32_t)WAVES);
    a.slices = std::max<uint32_t>(1u, (uint32_t)WAVES / a.hpb);
    /* no more slices than a span has sub-chunks */
    const uint32_t subs = (a.span + SUB - 1) / SUB;
    a.slices = std::min(a.slices, std::max(1u, subs));
    const uint32_t waves = a.hpb * a.slices;
    dim3 grid(a.splits, batch, (a.num_heads + a.hpb - 1) / a.hpb);
    const size_t lds = (size_t)waves * NQ * (HD + 2) * sizeof(float);
    blt_launch("kv_step", kv_step_kernel<G, NQ, WAVES>, grid, dim3(64 * waves), lds, s, a);
}

template <int G>
void dispatch_nq(const StepArgs &a, uint32_t nq, uint32_t batch, hipStream_t s) {
    /* single rows: one wave per head, and a second slice of waves once a split
     * holds enough keys to keep both busy */
    const int waves = a.hpb == 1u ? 16 : a.span >= 256u ? 8 : 4;
    if (nq <= 1) {
        if (waves >= 16) launch_step<G, 1, 16>(a, batch, s);
        else if (waves >= 8) launch_step<G, 1, 8>(a, batch, s);
        else launch_step<G, 1, 4>(a, batch, s);
    } else if (nq <= 2) launch_step<G, 2, 8>(a, batch, s);
    else if (nq <= 4) launch_step<G, 4, 4>(a, batch, s);
    else if (nq <= 8) launch_step<G, 8, 4>(a, batch, s);
    else launch_step<G, 16, 4>(a, batch, s);
}

} // namespace

namespace {

/* One launch set for at most 32 new rows per sequence: rows [row0, row0 + n) of a step of
 * n_seq rows per sequence, the row pointers already advanced to row0. */
void kv_step_slice(const blt_kv_attn_cache *cache, const float *q_rows, size_t q_stride, const float *k_rows,
                   size_t k_stride, const float *v_rows, size_t v_stride, const float *rope_cos,
                   const float *rope_sin, size_t rope_positions, float *combined, size_t combined_stride, size_t n,
                   size_t n_seq, size_t row0, int step_kind, int commit, size_t max_len_hint, bool static_scratch,
                   const uint32_t *host_lens);

void kv_step_run(const blt_kv_attn_cache *cache, const float *q_rows, size_t q_stride, const float *k_rows,
                 size_t k_stride, const float *v_rows, size_t v_stride, const float *rope_cos, const float *rope_sin,
                 size_t rope_positions, float *combined, size_t combined_stride, size_t n, int step_kind, int commit,
                 size_t max_len_hint, bool static_scratch, const uint32_t *host_lens = nullptr) {
    BLT_REQUIRE(q_rows != NULL && k_rows != NULL && v_rows != NULL && combined != NULL,
                "blt_kv_attend_step: row buffers must not be NULL");
    BLT_REQUIRE(n >= 1, "blt_kv_attend_step: need at least one row");
    BLT_REQUIRE(step_kind == BLT_KV_STEP_CAUSAL || step_kind == BLT_KV_STEP_BLOCK,
                "blt_kv_attend_step: unknown step_kind");
    BLT_REQUIRE(n <= 32 || step_kind == BLT_KV_STEP_CAUSAL,
                "blt_kv_attend_step: a block step takes at most 32 rows per sequence (every row sees every "
                "new row, so the block cannot be cut)");
    BLT_REQUIRE(max_len_hint >= n, "blt_kv_attend_step: exceeds cache capacity");
    /* Host lengths and a shape none of the kernel-argument kernels takes (several rows per sequence
     * at a head width the matrix-core block kernels do not have): the lengths go to a device array
     * of the library's through the pinned ring and the step runs as a non-committing device-length
     * step. */
    blt_kv_attn_cache staged_cache;
    if (host_lens && cache != NULL) {
        const size_t hd = cache->num_heads ? cache->embed_dim / cache->num_heads : 0;
        /* ... and single rows of a few long sequences, which the split kernel spreads over more
         * compute units than one workgroup per (sequence, head) reaches */
        const bool few_long = n == 1 && cache->batch * cache->num_heads < 64 && max_len_hint > 4096;
        if ((n > 1 && hd != 32 && hd != 64) || few_long) {
            staged_cache = *cache;
            staged_cache.self_len = staged_lengths(host_lens, cache->batch);
            cache = &staged_cache;
            host_lens = nullptr;
            commit = 0;
        }
    }
    /* A causal chunk longer than 32 rows (a prompt prefill) runs as consecutive 32-row slices: a
     * slice's rows see the cache, the earlier slices' rows (written through by then) and their
     * own; only the last slice advances the lengths. */
    for (size_t row0 = 0; row0 < n; row0 += 32) {
        const size_t rows = std::min<size_t>(32, n - row0);
        const bool last = row0 + rows == n;
        kv_step_slice(cache, q_rows + row0 * q_stride, q_stride, k_rows + row0 * k_stride, k_stride,
                      v_rows + row0 * v_stride, v_stride, rope_cos, rope_sin, rope_positions,
                      combined + row0 * combined_stride, combined_stride, rows, n, row0, step_kind, last ? commit : 0,
                      max_len_hint - (n - row0 - rows), static_scratch, host_lens);
    }
    if (!host_lens) {
        g_unchecked_steps.fetch_add(1, std::memory_order_relaxed);
        blt_stream_note_device_length_step(); /* replays of a graph that holds this step arm the check themselves */
    }
}

/* Query capacity of the per-split record layout a launch of `nq` rows uses: the VALU kernel's
 * row template, 32 for the matrix-core kernels. */
uint32_t valu_slots(uint32_t nq) { return nq <= 1 ? 1u : nq <= 2 ? 2u : nq <= 4 ? 4u : nq <= 8 ? 8u : 16u; }

/* Records and tickets for a launch set that needs `floats` floats of per-split records and
 * `batch` tickets, from the fixed device array or from the growing per-stream buffers. */
void acquire_scratch(StepArgs &a, size_t floats, size_t batch, bool static_scratch) {
    const DeviceStatics &st = statics();
    a.error = st.error();
    if (static_scratch) {
        BLT_REQUIRE(floats <= STATIC_PARTIAL_FLOATS && batch <= STATIC_TICKETS,
                    "blt_kv_attend_step_noalloc: this step needs %zu bytes of per-split records for %zu sequences; "
                    "the fixed scratch holds %zu bytes and %zu sequences (use blt_kv_attend_step_hip, which "
                    "allocates, or a smaller batch)",
                    floats * sizeof(float), batch, STATIC_PARTIAL_FLOATS * sizeof(float), STATIC_TICKETS);
        a.partial = st.partial();
        a.tickets = st.tickets();
        return;
    }
    GrowingScratch &g = growing();
    Scratch &sc = g.by_stream[blt_stream_key()];
    BLT_REQUIRE(!blt_stream_capturing() || (floats <= sc.partial_floats && batch <= sc.ticket_count),
                "blt_kv_attend_step: the step would allocate its scratch while a graph capture is open; run it once "
                "eagerly with this batch size on this stream first");
    if (floats > sc.partial_floats) {
        if (sc.partial) g.retired.push_back(sc.partial);
        sc.partial_floats = std::max(floats, 2 * sc.partial_floats);
        HIP_CHECK(hipMalloc((void **)&sc.partial, sc.partial_floats * sizeof(float)));
    }
    if (batch > sc.ticket_count) {
        if (sc.tickets) g.retired.push_back(sc.tickets);
        sc.ticket_count = std::max<size_t>(2 * batch, 1024);
        HIP_CHECK(hipMalloc((void **)&sc.tickets, sc.ticket_count * sizeof(uint32_t)));
        hipLaunchKernelGGL(kv_clear_words_kernel, dim3((unsigned)((sc.ticket_count + 255) / 256)), dim3(256), 0,
                           blt_stream(), sc.tickets, sc.ticket_count);
    }
    a.partial = sc.partial;
    a.tickets = sc.tickets;
}

void kv_step_slice(const blt_kv_attn_cache *cache, const float *q_rows, size_t q_stride, const float *k_rows,
                   size_t k_stride, const float *v_rows, size_t v_stride, const float *rope_cos,
                   const float *rope_sin, size_t rope_positions, float *combined, size_t combined_stride, size_t n,
                   size_t n_seq, size_t row0, int step_kind, int commit, size_t max_len_hint, bool static_scratch,
                   const uint32_t *host_lens) {
    BLT_REQUIRE(cache != NULL && cache->self_k != NULL && cache->self_v != NULL &&
                    (cache->self_len != NULL || host_lens != NULL),
                "blt_kv_attend_step: cache buffers must not be NULL");
    const size_t E = cache->embed_dim, H = cache->num_heads;
    BLT_REQUIRE(H >= 1 && E % H == 0, "blt_kv_attend_step: embed_dim must be divisible by num_heads");
    const size_t hd = E / H;
    BLT_REQUIRE(hd == 4 || hd == 8 || hd == 16 || hd == 32 || hd == 64 || hd == 128,
                "blt_kv_attend_step: head_dim must be a power of two in [4, 128]");
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
    a.by_length = 0; /* the block launcher decides */
    a.cache_k = cache->self_k;
    a.cache_v = cache->self_v;
    a.self_len = cache->self_len;
    a.q_rows = q_rows;
    a.k_rows = k_rows;
    a.v_rows = v_rows;
    a.combined = combined;
    a.rope_cos = rope_cos;
    a.rope_sin = rope_sin;
    a.q_stride = (uint32_t)q_stride;
    a.k_stride = (uint32_t)k_stride;
    a.v_stride = (uint32_t)v_stride;
    a.out_stride = (uint32_t)combined_stride;
    a.max_seq_len = (uint32_t)cache->max_seq_len;
    a.embed_dim = (uint32_t)E;
    a.num_heads = (uint32_t)H;
    a.window = (uint32_t)cache->window;
    a.n = (uint32_t)n;
    a.n_seq = (uint32_t)n_seq;
    a.len_bias = (uint32_t)row0;
    a.scale = 1.0f / sqrtf((float)hd);
    a.block_kind = step_kind == BLT_KV_STEP_BLOCK;
    a.hpb = 0, a.slices = 1;

    const size_t subs = (max_len_hint + SUB - 1) / SUB;

    /* Lengths on the host (the reference keeps self_len there, csrc/infer/kv_cache.h:56-60): they
     * travel in the kernel arguments, KARG_SEQS sequences per launch; the capacity check was made
     * by the entry point.  Sequences [b0, b0 + nb) of the step as a launch of their own: */
    auto chunk_of = [&](const StepArgs &all, size_t b0) {
        StepArgs c = all;
        c.cache_k += b0 * cache->max_seq_len * E, c.cache_v += b0 * cache->max_seq_len * E;
        c.q_rows += b0 * n_seq * q_stride, c.k_rows += b0 * n_seq * k_stride, c.v_rows += b0 * n_seq * v_stride;
        c.combined += b0 * n_seq * combined_stride;
        return c;
    };
    if (host_lens && n_seq == 1) {
        a.self_len = nullptr, a.partial = nullptr, a.tickets = nullptr, a.error = nullptr;
        a.splits = 1, a.span = 0, a.cap = (uint32_t)cache->max_seq_len, a.q0 = 0, a.write_through = 1, a.commit = 0;
        for (size_t b0 = 0; b0 < cache->batch; b0 += KARG_SEQS) {
            const size_t nb = std::min<size_t>(KARG_SEQS, cache->batch - b0);
            uint32_t longest = 0;
            for (size_t b = 0; b < nb; b++) longest = std::max(longest, host_lens[b0 + b] + 1u);
            BLT_REQUIRE(kv_row_launch(chunk_of(a, b0), (uint32_t)nb, (uint32_t)hd, host_lens + b0, longest, 0),
                        "blt_kv_attend_step_lens: internal: head_dim %zu not taken by the row kernel", hd);
        }
        HIP_CHECK_LAUNCH("blt_kv_attend_step_lens");
        return;
    }
    /* Single rows of a batch that one workgroup per (sequence, head) spreads over the chip: the
     * waves of a workgroup slice one head's keys and meet once in LDS, nothing crosses workgroups
     * but the length ticket.
     * Measured against the split layout at 32 / 64 / 128 sequences of 4 heads: ahead or level up to
     * 8192 cached keys with up to 256 (sequence, head) pairs (21.2 against 24.2 us at 32 x 2048..4096,
     * 35.5 against 39.4 at 64), with 512 pairs ahead at 2048 keys (33.2 against 39.2) and behind at
     * 4096 (86.1 against 81.8) */
    const size_t pairs = cache->batch * H;
    if (n_seq == 1 && subs >= 4 && pairs >= 128 && pairs <= 512 && subs <= (pairs <= 256 ? 256u : 96u)) {
        a.splits = 1, a.span = 0, a.q0 = 0, a.write_through = 1, a.commit = commit;
        a.cap = (uint32_t)std::min<size_t>((size_t)cache->max_seq_len, rope_cos ? rope_positions : (size_t)UINT32_MAX);
        acquire_scratch(a, 0, cache->batch, static_scratch);
        BLT_REQUIRE(kv_row_launch(a, (uint32_t)cache->batch, (uint32_t)hd, nullptr, (uint32_t)max_len_hint, 0),
                    "blt_kv_attend_step: internal: head_dim %zu not taken by the row kernel", hd);
        HIP_CHECK_LAUNCH("blt_kv_attend_step");
        return;
    }

    /* enough workgroups to fill 256 compute units a few times over (sequences
     * shorter than the hint leave theirs idle), but no span shorter than two
     * sub-chunks */
    size_t splits = (1024 + cache->batch - 1) / cache->batch;
    splits = std::min<size_t>(splits, (subs + 1) / 2);
    splits = std::max<size_t>(1, std::min<size_t>(splits, MAX_SPLITS));
    const size_t span_subs = (subs + splits - 1) / splits;
    splits = (subs + span_subs - 1) / span_subs;
    a.splits = (uint32_t)splits;
    a.span = (uint32_t)(span_subs * SUB);
    a.hpb = 0;
    /* Single rows of a batch that one workgroup per (sequence, head) already
     * spreads over the chip: all 16 waves of a workgroup slice one head's keys
     * and merge through LDS, so nothing crosses workgroups but the ticket. */
    if (a.n == 1u && subs >= 4 && subs <= 64 && cache->batch * H >= 128 &&
        cache->batch * H <= 512) {
        a.hpb = 1;
        a.splits = 1;
        a.span = (uint32_t)(subs * SUB);
    }

    /* Blocks of two or more rows go to the matrix-core kernels (one launch for
     * up to 32 rows; the cost does not depend on the row count: measured 9.5 us
     * at 64 sequences for 2 ... 16 rows against 9.9 / 14.6 us for 2 / 3 rows on
     * the VALU kernel) where they take the head_dim; single rows and the shapes
     * they do not take go to the VALU kernel in slices of at most 16 rows.
     * Every launch reads the new rows from the inputs, so only the first one
     * stores them and only the last one may advance the lengths.
     * BLT_HIP_BLOCK_KERNEL=valu|mfma pins the choice (tuning and test hook). */
    static const int pinned = [] {
        const char *e = getenv("BLT_HIP_BLOCK_KERNEL");
        return e && strcmp(e, "valu") == 0 ? 1 : e && strcmp(e, "mfma") == 0 ? 2 : 0;
    }();
    const bool want_mfma = pinned == 2 || (pinned == 0 && a.n >= 2u) || host_lens != nullptr;
    const bool mfma = want_mfma && (hd == 32 || hd == 64);
    BLT_REQUIRE(mfma || !host_lens, "blt_kv_attend_step_lens: internal: host lengths reached a kernel without them");
    if (mfma) {
        /* the block kernel merges slices inside the workgroup, so it wants few,
         * long spans: just enough workgroups to cover the compute units */
        a.hpb = kv_block_heads_per_group((uint32_t)cache->batch, (uint32_t)subs, (uint32_t)H);
        const size_t zblocks = (H + a.hpb - 1) / a.hpb;
        /* Splitting a sequence's keys over workgroups pays only for long prefixes: the split states
         * meet in global memory and the last workgroup merges them, which costs more than the
         * eight slices of one workgroup walking up to 64 sub-chunks (2048 keys) themselves
         * (measured at 1..16 sequences: 10.4 against 17.8 us at 500 keys, 13.6 against 18.1 at
         * 1000, even at 2000; 16.7 against 30 us at 4000 keys with 16 sub-chunks per split). */
        size_t bs = 1;
        if (subs > 64) bs = std::min<size_t>((256 + cache->batch * zblocks - 1) / (cache->batch * zblocks), (subs + 15) / 16);
        bs = std::max<size_t>(1, std::min<size_t>(bs, MAX_SPLITS));
        const size_t bspan = (subs + bs - 1) / bs;
        a.splits = (uint32_t)((subs + bspan - 1) / bspan);
        a.span = (uint32_t)(bspan * SUB);
    }
    /* what a sequence may attend at most: beyond it the kernels leave the sequence alone and raise
     * the error word (lengths are device data; the hint is all the host knows) */
    a.cap = (uint32_t)std::min<size_t>({(size_t)a.splits * a.span, (size_t)cache->max_seq_len,
                                        rope_cos ? rope_positions : (size_t)UINT32_MAX});
    const uint32_t slots = mfma ? 32u : valu_slots((uint32_t)std::min<size_t>(16, n));
    acquire_scratch(a, a.splits > 1u ? cache->batch * (size_t)a.splits * H * slots * (hd + 2) : 0, cache->batch,
                    static_scratch);

    if (mfma) {
        a.q0 = 0;
        a.write_through = 1;
        a.commit = host_lens ? 0 : commit;
        if (host_lens) {
            a.self_len = nullptr;
            for (size_t b0 = 0; b0 < cache->batch; b0 += KARG_SEQS) {
                const size_t nb = std::min<size_t>(KARG_SEQS, cache->batch - b0);
                BLT_REQUIRE(kv_block_mfma_launch(chunk_of(a, b0), (uint32_t)nb, (uint32_t)hd, host_lens + b0, 0),
                            "blt_kv_attend_step_lens: internal: head_dim %zu not taken by the block kernels", hd);
            }
        } else {
            BLT_REQUIRE(kv_block_mfma_launch(a, (uint32_t)cache->batch, (uint32_t)hd, nullptr, 0),
                        "blt_kv_attend_step: internal: head_dim %zu not taken by the block kernels", hd);
        }
        HIP_CHECK_LAUNCH("blt_kv_attend_step");
        return;
    }
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
        default: dispatch_nq<32>(a, nq, (uint32_t)cache->batch, 0); break;
        }
    }
    HIP_CHECK_LAUNCH("blt_kv_attend_step");
}

} // namespace

/* Reads the sticky device error word when a device-length step was issued since the last look;
 * called by the library's synchronising entry points after their wait. */
void blt_kv_arm_device_error_check() { g_unchecked_steps.fetch_add(1, std::memory_order_relaxed); }

void blt_kv_check_device_errors() {
    if (g_unchecked_steps.exchange(0, std::memory_order_relaxed) == 0) return;
    uint32_t word = 0;
    HIP_CHECK(hipMemcpy(&word, statics().error(), sizeof(word), hipMemcpyDeviceToHost));
    if (word & KV_ERR_CAPACITY)
        BLT_FATAL("blt_kv_attend_step: exceeds cache capacity (on the device a sequence's length plus its new rows "
                  "went past max_len_hint, max_seq_len or the rotation tables; that sequence was left untouched)");
}

extern "C" void blt_kv_attend_step_hip(const blt_kv_attn_cache *cache, const float *q_rows, size_t q_stride,
                                       const float *k_rows, size_t k_stride, const float *v_rows, size_t v_stride,
                                       float *combined, size_t combined_stride, size_t n, int step_kind, int commit,
                                       size_t max_len_hint) {
    kv_step_run(cache, q_rows, q_stride, k_rows, k_stride, v_rows, v_stride, nullptr, nullptr, 0, combined,
                combined_stride, n, step_kind, commit, max_len_hint, false);
}

extern "C" void blt_kv_attend_step_noalloc_hip(const blt_kv_attn_cache *cache, const float *q_rows, size_t q_stride,
                                               const float *k_rows, size_t k_stride, const float *v_rows,
                                               size_t v_stride, float *combined, size_t combined_stride, size_t n,
                                               int step_kind, int commit, size_t max_len_hint) {
    kv_step_run(cache, q_rows, q_stride, k_rows, k_stride, v_rows, v_stride, nullptr, nullptr, 0, combined,
                combined_stride, n, step_kind, commit, max_len_hint, true);
}

extern "C" void blt_kv_rope_attend_step_hip(const blt_kv_attn_cache *cache, const float *q_rows, size_t q_stride,
                                            const float *k_rows, size_t k_stride, const float *v_rows,
                                            size_t v_stride, const float *rope_cos, const float *rope_sin,
                                            size_t rope_positions, float *combined, size_t combined_stride, size_t n,
                                            int step_kind, int commit, size_t max_len_hint) {
    BLT_REQUIRE(rope_cos != NULL && rope_sin != NULL, "blt_kv_rope_attend_step: rotation tables must not be NULL");
    BLT_REQUIRE(((reinterpret_cast<uintptr_t>(rope_cos) | reinterpret_cast<uintptr_t>(rope_sin)) & 7u) == 0,
                "blt_kv_rope_attend_step: rotation tables must be 8-byte aligned");
    BLT_REQUIRE(max_len_hint <= rope_positions,
                "blt_kv_rope_attend_step: positions up to %zu exceed the rotation tables (%zu rows)", max_len_hint,
                rope_positions);
    kv_step_run(cache, q_rows, q_stride, k_rows, k_stride, v_rows, v_stride, rope_cos, rope_sin, rope_positions,
                combined, combined_stride, n, step_kind, commit, max_len_hint, false);
}

extern "C" void blt_kv_attend_step_lens_hip(const blt_kv_attn_cache *cache, const uint32_t *self_len_host,
                                            const float *q_rows, size_t q_stride, const float *k_rows, size_t k_stride,
                                            const float *v_rows, size_t v_stride, const float *rope_cos,
                                            const float *rope_sin, size_t rope_positions, float *combined,
                                            size_t combined_stride, size_t n, int step_kind) {
    BLT_REQUIRE(self_len_host != NULL, "blt_kv_attend_step_lens: the host lengths must not be NULL");
    BLT_REQUIRE((rope_cos == NULL) == (rope_sin == NULL), "blt_kv_attend_step_lens: both rotation tables or none");
    BLT_REQUIRE(((reinterpret_cast<uintptr_t>(rope_cos) | reinterpret_cast<uintptr_t>(rope_sin)) & 7u) == 0,
                "blt_kv_attend_step_lens: rotation tables must be 8-byte aligned");
    BLT_REQUIRE(cache != NULL, "blt_kv_attend_step_lens: cache must not be NULL");
    /* the reference's check (csrc/infer/kv_cache.c:191), made where the lengths live */
    const size_t limit = std::min<size_t>(cache->max_seq_len, rope_cos ? rope_positions : SIZE_MAX);
    size_t longest = 0;
    for (size_t b = 0; b < cache->batch; b++) longest = std::max<size_t>(longest, self_len_host[b]);
    BLT_REQUIRE(longest + n <= limit, "blt_kv_attend_step_lens: exceeds cache capacity");
    kv_step_run(cache, q_rows, q_stride, k_rows, k_stride, v_rows, v_stride, rope_cos, rope_sin, rope_positions,
                combined, combined_stride, n, step_kind, 0, longest + n, false, self_len_host);
}
