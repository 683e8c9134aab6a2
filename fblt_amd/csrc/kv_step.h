/*
 * Shared by the two kernels behind blt_kv_attend_step_hip (the VALU decode
 * kernel and the MFMA block kernel): the launch arguments, the device-scope
 * publish/observe accessors for data that crosses workgroups inside one
 * launch, and the ticket + merge that finishes a sequence.
 */
#ifndef FBLT_AMD_KV_STEP_H
#define FBLT_AMD_KV_STEP_H

#include "attn_device.h"
#include "hip_check.h"
#include "rope_device.h"

constexpr int SUB = 32;        /* keys per sub-chunk (one wave, one head)       */
constexpr int MAX_SPLITS = 16; /* workgroups per sequence                        */

struct StepArgs {
    float *cache_k;
    float *cache_v;
    uint32_t *self_len;
    const float *q_rows;
    const float *k_rows;
    const float *v_rows;
    float *combined;
    const float *rope_cos; /* [positions][hd/2] rotation tables, or NULL: rows arrive rotated */
    const float *rope_sin;
    float *partial;    /* [batch][splits][heads][NQ][hd + 2] */
    uint32_t *tickets; /* [batch] */
    uint32_t *error;   /* sticky device word: KV_ERR_* bits, read back by the host at its next synchronisation */
    uint32_t q_stride, k_stride, v_stride, out_stride;
    uint32_t max_seq_len, embed_dim, num_heads;
    uint32_t window;
    uint32_t n;        /* new rows per sequence this launch works on */
    uint32_t n_seq;    /* rows per sequence in the row arrays: sequence b's rows start at row b * n_seq
                          (the row pointers are already advanced to this launch's first row) */
    uint32_t len_bias; /* rows of the same step already written through by earlier launches:
                          the sequence's length for this launch is self_len[b] + len_bias */
    uint32_t q0;       /* first query row this launch handles */
    uint32_t splits;   /* gridDim.x */
    uint32_t span;     /* keys per split, a multiple of SUB */
    uint32_t cap;      /* most keys (cached + new) a sequence may attend in this launch: what the slab, the
                          launch's splits * span and the rotation tables all hold */
    uint32_t hpb;      /* heads per workgroup */
    uint32_t slices;   /* waves per head in a workgroup */
    float scale;
    int block_kind;    /* every new row sees all keys */
    int write_through; /* this launch stores the new rows into the cache */
    int commit;        /* advance self_len when the sequence is done */
    int by_length;     /* block step with the lengths in the arguments: workgroups take the (sequence, head
                          group) pairs in the order of KargLens::order, longest sequences first */
};


/* Asks for every member of the launch's argument block at once, at kernel entry: left to itself the
 * compiler fetches them group by group where they are first needed, and each group is a round
 * trip through a scalar cache that is cold at the start of a launch. */
__device__ __forceinline__ void kv_fetch_arguments(const StepArgs &a) {
    asm volatile("" ::"s"(a.cache_k), "s"(a.cache_v), "s"(a.self_len), "s"(a.q_rows), "s"(a.k_rows), "s"(a.v_rows),
                 "s"(a.combined), "s"(a.rope_cos), "s"(a.rope_sin));
    asm volatile("" ::"s"(a.partial), "s"(a.tickets), "s"(a.error), "s"(a.q_stride), "s"(a.k_stride), "s"(a.v_stride),
                 "s"(a.out_stride), "s"(a.max_seq_len), "s"(a.embed_dim), "s"(a.num_heads), "s"(a.window));
    asm volatile("" ::"s"(a.n), "s"(a.n_seq), "s"(a.len_bias), "s"(a.q0), "s"(a.splits), "s"(a.span), "s"(a.cap),
                 "s"(a.hpb), "s"(a.slices), "s"(a.scale), "s"(a.block_kind), "s"(a.write_through), "s"(a.commit));
}

/* Where a launch takes the sequences' lengths from: a.self_len in device memory, or -- when the
 * caller keeps the lengths on the host, as the reference does (csrc/infer/kv_cache.h:56-60) -- the
 * kernel arguments themselves, KARG_SEQS sequences per launch.  With the lengths in the argument
 * block the first K/V requests of a workgroup depend on nothing but that block: one dependent
 * trip to memory less.  Such a launch checks nothing and commits nothing on the device (the host
 * did the capacity check and owns the lengths). */
constexpr int KARG_SEQS = 256;
struct KargLens {
    uint32_t v[KARG_SEQS];
    uint8_t order[KARG_SEQS]; /* by_length launches: the sequences of the launch, longest first */
};
struct DeviceLens {
    uint32_t unused;
};
template <bool KARG>
struct LensArgOf {
    typedef DeviceLens type;
};
template <>
struct LensArgOf<true> {
    typedef KargLens type;
};
template <bool KARG>
using LensArg = typename LensArgOf<KARG>::type;

__device__ __forceinline__ uint32_t kv_len_of(const StepArgs &, const KargLens &lens, uint32_t b) { return lens.v[b]; }
__device__ __forceinline__ uint32_t kv_len_of(const StepArgs &a, const DeviceLens &, uint32_t b) { return a.self_len[b]; }

/* The lengths live in device memory and the launch was sized from a host-side hint.  A sequence
 * whose length + new rows went past what the launch, its slab or the rotation tables hold must
 * neither drop keys silently nor store past its slab: every workgroup of such a sequence leaves
 * before its first load -- no write-through, no output rows, no ticket, no commit -- and one of them
 * raises a sticky error bit that the host turns into the reference's "exceeds cache capacity" fatal
 * error (csrc/infer/kv_cache.c:191) at its next synchronisation.  The condition depends on the
 * sequence only, so all workgroups of the sequence agree and the ticket stays armed. */
constexpr uint32_t KV_ERR_CAPACITY = 1u;
__device__ __forceinline__ bool kv_over_capacity(const StepArgs &a, uint32_t nk) {
    if (nk <= a.cap) return false;
    if (threadIdx.x == 0 && blockIdx.x == 0 && blockIdx.z == 0)
        __hip_atomic_fetch_or(a.error, KV_ERR_CAPACITY, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return true;
}

/* Keys per split for a sequence that attends nk keys: the sequence's own
 * sub-chunks divided evenly over the launch's splits, so that every workgroup
 * of a sequence gets the same share whatever the sequence's length (a.span,
 * sized for the longest sequence, is the upper bound). */
__device__ __forceinline__ uint32_t kv_span_of(const StepArgs &a, uint32_t nk) {
    const uint32_t subs = (nk + SUB - 1u) / SUB;
    return min(a.span, ((subs + a.splits - 1u) / a.splits) * SUB);
}

/* Device-scope store / load of data another workgroup (possibly on another
 * die of the package) reads within the same launch. */
__device__ __forceinline__ void publish(float *p, float x) {
    __hip_atomic_store(p, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float observe(const float *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* Called by every thread of every workgroup of sequence b once its per-split
 * state is published (splits > 1) or its output rows are written (splits ==
 * 1).  The last workgroup of the sequence to arrive merges the splits into
 * the output rows, re-arms the ticket and advances the sequence's length when
 * the step commits.  `slots` is the query capacity of the partial layout
 * [batch][splits][heads][slots][HD + 2] (max, sum in the two extra floats).
 *
 * The per-split states were stored with device-scope write-through stores and
 * are read back with device-scope loads, so they never sit dirty or stale in
 * one die's L2 and no cache write-back or invalidate is needed; each wave waits
 * for its own stores to complete before the barrier that precedes the
 * workgroup's ticket. */
/* The step commits, has one split per sequence but several workgroups (head
 * groups): all that has to be known is when every workgroup of the sequence
 * has read the old length.  Thread 0 of each workgroup draws its ticket at a
 * point where all its waves have done that read (after the barrier that ends
 * the key loop) -- the reply travels while the workgroup merges and stores --
 * and the one that drew the last ticket writes the new length when it is done.  Returns
 * the ticket (thread 0 only; KV_NO_TICKET when this scheme does not apply). */
constexpr uint32_t KV_NO_TICKET = 0xFFFFFFFFu;
__device__ __forceinline__ bool kv_early_ticket_applies(const StepArgs &a) {
    return a.splits == 1u && gridDim.z > 1u && a.commit;
}
__device__ __forceinline__ uint32_t kv_draw_early_ticket(const StepArgs &a, uint32_t b) {
    if (!kv_early_ticket_applies(a) || threadIdx.x != 0) return KV_NO_TICKET;
    return __hip_atomic_fetch_add(&a.tickets[b], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int HD>
__device__ __forceinline__ void kv_finish_sequence(const StepArgs &a, uint32_t slots, uint32_t b, uint32_t nk,
                                                   uint32_t *sm_ticket, uint32_t early_ticket) {
    if (a.splits == 1u && (gridDim.z == 1u || !a.commit)) {
        /* the output rows are written; the ticket is only needed to tell when the
         * last workgroup of the sequence has read the old length */
        if (a.commit && threadIdx.x == 0) a.self_len[b] = nk;
        return;
    }
    if (kv_early_ticket_applies(a)) {
        if (threadIdx.x == 0 && early_ticket == gridDim.z - 1u) {
            a.tickets[b] = 0u; /* re-armed for the next launch */
            a.self_len[b] = nk;
        }
        return;
    }
    blt_vector_memory_done(); /* every wave's published records are out before thread 0 draws the ticket */
    __syncthreads();
    if (threadIdx.x == 0)
        *sm_ticket = __hip_atomic_fetch_add(&a.tickets[b], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*sm_ticket != gridDim.x * gridDim.z - 1u) return;

    if (a.splits > 1u) {
        const uint32_t all = a.num_heads * slots * HD;
        const size_t sstride = (size_t)a.num_heads * slots * (HD + 2);
        for (uint32_t t = threadIdx.x; t < all; t += blockDim.x) {
            const uint32_t d = t % HD;
            const uint32_t r = (t / HD) % slots;
            const uint32_t hh = t / (HD * slots);
            const uint32_t qi = a.q0 + r;
            if (qi >= a.n) continue;
            const float *base = a.partial + (((size_t)b * a.splits * a.num_heads + hh) * slots + r) * (HD + 2);
            float pm[MAX_SPLITS], pl[MAX_SPLITS], po[MAX_SPLITS];
#pragma unroll
            for (int s = 0; s < MAX_SPLITS; s++) {
                const bool on = (uint32_t)s < a.splits;
                const float *ps = base + (on ? s : 0) * sstride;
                pm[s] = on ? observe(ps + HD) : neg_inf();
                pl[s] = on ? observe(ps + HD + 1) : 0.f;
                po[s] = on ? observe(ps + d) : 0.f;
            }
            float M = neg_inf();
#pragma unroll
            for (int s = 0; s < MAX_SPLITS; s++) M = fmaxf(M, pm[s]);
            float L = 0.f, acc = 0.f;
#pragma unroll
            for (int s = 0; s < MAX_SPLITS; s++) {
                const float f = pm[s] == neg_inf() ? 0.f : softmax_exp(pm[s] - M);
                L += pl[s] * f;
                acc += po[s] * f;
            }
            a.combined[((size_t)b * a.n_seq + qi) * a.out_stride + hh * HD + d] = L > 0.f ? acc / L : 0.f;
        }
    }
    if (threadIdx.x == 0) {
        a.tickets[b] = 0u;
        if (a.commit) a.self_len[b] = nk;
    }
}

/* heads per workgroup the MFMA block kernel should be launched with (set StepArgs.hpb to it) */
uint32_t kv_block_heads_per_group(uint32_t batch, uint32_t subs, uint32_t num_heads);
/* launch of the MFMA block kernel (attn_verify.hip); false when it does not take the shape.
 * host_lens: NULL (device lengths) or `batch` <= KARG_SEQS lengths for the argument block */
bool kv_block_mfma_launch(const StepArgs &a, uint32_t batch, uint32_t head_dim, const uint32_t *host_lens,
                          hipStream_t s);

/* block steps of at most 16 rows over a prefix short enough to be requested all at once
 * (attn_verify_once.hip); false when it does not take the shape */
bool kv_block_once_launch(const StepArgs &a, uint32_t batch, uint32_t head_dim, const uint32_t *host_lens,
                          hipStream_t s);

/* single-row steps with one workgroup per (sequence, head) (attn_decode_row.hip): lengths from
 * `host_lens` (at most KARG_SEQS sequences, carried in the kernel arguments; nothing is
 * committed) or, when NULL, from a.self_len with the commit through a.tickets; max_keys sizes
 * the workgroups; false when the head width is not taken */
bool kv_row_launch(const StepArgs &a, uint32_t batch, uint32_t head_dim, const uint32_t *host_lens, uint32_t max_keys,
                   hipStream_t s);

#endif
