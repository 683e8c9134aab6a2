/*
 * Dense additive masks built in device memory, bit-for-bit what the
 * reference's CPU builders write (csrc/ops/mask_builder_cpu.c:21-154): 0.0f
 * where a (query, key) pair may attend, -INFINITY where it may not.
 *
 * One thread per cell, threads of a block along the key axis so stores are
 * coalesced; pure integer predicate work bounded by the store stream (HBM).
 * Document ids are resolved on the host (O(nq + nk)) and shipped as arrays,
 * so the kernel never searches the boundary list.
 */
#include "blt_hip.h"
#include "blt_fatal.h"
#include "hip_check.h"
#include "launch.h"

#include <stdint.h>
#include <stdlib.h>
#include <vector>

namespace {

struct MaskRecipe {
    uint64_t nq, nk;
    uint64_t window;
    uint64_t causal_offset;
    const uint64_t *doc_q;  /* device, or null */
    const uint64_t *doc_kv; /* device, or null */
    const uint64_t *grp_q;  /* device, or null */
    const uint64_t *grp_kv; /* device, or null */
    int is_causal;
    int bidirectional;
};

__device__ __forceinline__ bool pair_allowed(const MaskRecipe &r, uint64_t i, uint64_t j) {
    bool ok = true;
    const uint64_t diag = i + r.causal_offset;
    if (r.is_causal && j > diag) ok = false;
    if (r.window > 0) {
        const uint64_t ref = r.is_causal ? diag : i;
        const uint64_t dist = ref >= j ? ref - j : j - ref;
        if (dist >= r.window) ok = false;
    }
    if (r.doc_q && r.doc_q[i] != r.doc_kv[j]) ok = false;
    if (r.grp_q) {
        if (r.grp_q[i] != r.grp_kv[j]) ok = false;
        else if (!r.bidirectional && j > i) ok = false;
    }
    return ok;
}

/* grid.x covers the key axis in chunks of 256 * W cells (lane = W consecutive keys, stored as one
 * 4*W-byte piece; W = 4 needs seq_len_kv % 4 == 0 so that every row starts 16-byte aligned),
 * grid.y strides over rows.  row_ok[i] ends up non-zero when row i has at least one allowed key:
 * a plain store of 1 by every wave that saw one (the same value from all of them, no atomic). */
template <int W>
__global__ __launch_bounds__(256) void attention_mask_kernel(float *__restrict__ out, MaskRecipe r,
                                                             uint32_t *__restrict__ row_ok) {
    const uint64_t j0 = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * W;
    for (uint64_t i = blockIdx.y; i < r.nq; i += gridDim.y) {
        bool any_ok = false;
        if (j0 < r.nk) { /* nk % W == 0: all W cells are inside */
            float v[W];
#pragma unroll
            for (int t = 0; t < W; t++) {
                const bool ok = pair_allowed(r, i, j0 + t);
                any_ok |= ok;
                v[t] = ok ? 0.0f : -__builtin_huge_valf();
            }
            if (W == 4) *reinterpret_cast<float4 *>(out + i * r.nk + j0) = make_float4(v[0], v[1], v[2], v[3]);
            else out[i * r.nk + j0] = v[0];
        }
        if (row_ok && __ballot(any_ok) != 0ull && (threadIdx.x & 63u) == 0u) row_ok[i] = 1u;
    }
}

__global__ __launch_bounds__(256) void count_dead_rows_kernel(const uint32_t *__restrict__ row_ok, uint64_t nq,
                                                              uint32_t *__restrict__ dead) {
    uint32_t mine = 0;
    for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < nq; i += (uint64_t)gridDim.x * 256u)
        mine += row_ok[i] == 0u;
    if (mine) atomicAdd(dead, mine);
}

struct BlockRecipe {
    uint64_t S, N, B;
    const uint64_t *starts; /* device, TRAIN only */
    int infer;
};

template <int W>
__global__ __launch_bounds__(256) void block_diffusion_mask_kernel(float *__restrict__ out, BlockRecipe r) {
    const uint64_t j0 = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * W;
    if (j0 >= r.S) return;
    for (uint64_t i = blockIdx.y; i < r.S; i += gridDim.y) {
        float v[W];
#pragma unroll
        for (int t = 0; t < W; t++) {
            const uint64_t j = j0 + t;
            bool ok;
            if (i < r.N) {
                ok = j < r.N && j <= i;
            } else if (r.infer) {
                ok = true;
            } else {
                const uint64_t blk = (i - r.N) / r.B;
                const bool own = j >= r.N && (j - r.N) / r.B == blk;
                ok = j < r.starts[blk] || own;
            }
            v[t] = ok ? 0.0f : -__builtin_huge_valf();
        }
        if (W == 4) *reinterpret_cast<float4 *>(out + i * r.S + j0) = make_float4(v[0], v[1], v[2], v[3]);
        else out[i * r.S + j0] = v[0];
    }
}

/* Host array -> 16-byte aligned arena memory, copied on the null stream. */
const uint64_t *stage_u64(const size_t *host, size_t n, blt_arena *arena) {
    if (n == 0) return nullptr;
    void *dev = blt_arena_alloc(arena, n * sizeof(uint64_t), 16);
    blt_hip_memcpy_h2d(dev, host, n * sizeof(uint64_t));
    return static_cast<const uint64_t *>(dev);
}

void doc_ids_from_boundaries(const size_t *bounds, size_t num_docs, size_t len, std::vector<size_t> &ids) {
    ids.resize(len);
    size_t d = 0;
    for (size_t p = 0; p < len; p++) {
        while (d + 1 < num_docs && p >= bounds[d]) d++;
        ids[p] = d;
    }
}

dim3 mask_grid(uint64_t rows, uint64_t cols, uint64_t per_lane) {
    const uint64_t gx = (cols + 256u * per_lane - 1u) / (256u * per_lane);
    const uint64_t gy = rows < 4096u ? (rows ? rows : 1u) : 4096u;
    return dim3((unsigned)gx, (unsigned)gy, 1u);
}

} // namespace

extern "C" void blt_build_attention_mask_hip(const blt_mask_config *config, blt_tensor *out_mask, blt_arena *arena) {
    BLT_REQUIRE(arena != NULL, "blt_build_attention_mask: arena is NULL");
    BLT_REQUIRE(arena->backend == BLT_BACKEND_HIP, "blt_build_attention_mask: HIP implementation called with non-HIP arena");
    BLT_REQUIRE(config != NULL, "blt_build_attention_mask: config is NULL");
    BLT_REQUIRE(out_mask != NULL, "blt_build_attention_mask: out_mask is NULL");
    const size_t nq = config->seq_len_q, nk = config->seq_len_kv;
    BLT_REQUIRE(nq > 0 && nk > 0, "blt_build_attention_mask: seq_len_q/seq_len_kv must be > 0");
    BLT_REQUIRE((nk + 255u) / 256u <= 0x7FFFFFFFu, "blt_build_attention_mask: seq_len_kv too large");

    const bool docs = config->doc_boundaries != NULL && config->num_docs > 0;
    const bool groups = config->query_group_ids != NULL && config->kv_group_ids != NULL;

    /* every cell is written by the kernel, so the tensor needs no clearing */
    const size_t shape[2] = {nq, nk};
    *out_mask = blt_tensor_create_uninit(arena, shape, 2, BLT_DTYPE_FP32);

    MaskRecipe r;
    r.nq = nq;
    r.nk = nk;
    r.window = config->sliding_window;
    r.causal_offset = config->causal_offset;
    r.is_causal = config->is_causal ? 1 : 0;
    r.bidirectional = config->bidirectional_within_group ? 1 : 0;
    r.doc_q = r.doc_kv = r.grp_q = r.grp_kv = nullptr;
    std::vector<size_t> dq, dk;
    if (docs) {
        doc_ids_from_boundaries(config->doc_boundaries, config->num_docs, nq, dq);
        doc_ids_from_boundaries(config->doc_boundaries, config->num_docs, nk, dk);
        r.doc_q = stage_u64(dq.data(), nq, arena);
        r.doc_kv = stage_u64(dk.data(), nk, arena);
    }
    if (groups) {
        r.grp_q = stage_u64(config->query_group_ids, nq, arena);
        r.grp_kv = stage_u64(config->kv_group_ids, nk, arena);
    }

    /* "query position has no valid key" (mask_builder_cpu.c:93).  Whenever every row's allowed keys
     * form one range -- causal, window, document and sorted-group recipes, i.e. every mask the
     * callers build -- the host knows the answer in O(nq + nk) and the call stays asynchronous;
     * otherwise the kernel flags the rows that have a key and one blocking read-back counts the rest. */
    bool host_checked = false;
    if (nq <= 0xFFFFFFFFu && nk <= 0xFFFFFFFFu) {
        std::vector<uint32_t> lo(nq), hi(nq);
        if (blt_mask_config_row_ranges(config, lo.data(), hi.data())) {
            for (size_t i = 0; i < nq; i++)
                BLT_REQUIRE(lo[i] < hi[i], "blt_build_attention_mask: query position has no valid key");
            host_checked = true;
        }
    }
    uint32_t *row_ok = nullptr, *dead = nullptr;
    if (!host_checked) {
        row_ok = static_cast<uint32_t *>(blt_arena_alloc(arena, (nq + 1) * sizeof(uint32_t), 16));
        dead = row_ok + nq;
        blt_hip_memset(row_ok, 0, (nq + 1) * sizeof(uint32_t));
    }

    if (nk % 4u == 0u)
        blt_launch("mask_attention", attention_mask_kernel<4>, mask_grid(nq, nk, 4), dim3(256), 0, 0,
                   static_cast<float *>(out_mask->data), r, row_ok);
    else
        blt_launch("mask_attention", attention_mask_kernel<1>, mask_grid(nq, nk, 1), dim3(256), 0, 0,
                   static_cast<float *>(out_mask->data), r, row_ok);
    HIP_CHECK_LAUNCH("blt_build_attention_mask");
    if (host_checked) return; /* the id vectors staged above were consumed when their uploads returned */
    const unsigned cblocks = (unsigned)((nq + 255u) / 256u < 1024u ? (nq + 255u) / 256u : 1024u);
    blt_launch("mask_row_check", count_dead_rows_kernel, dim3(cblocks), dim3(256), 0, 0, row_ok, (uint64_t)nq, dead);
    HIP_CHECK_LAUNCH("blt_build_attention_mask row check");
    uint32_t dead_rows = 0;
    blt_hip_memcpy_d2h(&dead_rows, dead, sizeof(dead_rows));
    BLT_REQUIRE(dead_rows == 0, "blt_build_attention_mask: query position has no valid key");
}

extern "C" void blt_build_block_diffusion_mask_hip(const blt_block_diffusion_config *config, blt_tensor *out_mask,
                                                   blt_arena *arena) {
    BLT_REQUIRE(config != NULL && out_mask != NULL && arena != NULL,
                "blt_build_block_diffusion_mask: config, out_mask and arena cannot be NULL");
    BLT_REQUIRE(arena->backend == BLT_BACKEND_HIP,
                "blt_build_block_diffusion_mask: HIP implementation called with non-HIP arena");
    const size_t S = config->seq_len, N = config->num_clean;
    BLT_REQUIRE(S >= 1 && N >= 1 && N <= S, "blt_build_block_diffusion_mask: need 1 <= num_clean <= seq_len");
    const bool train = config->mode == BLT_BDM_TRAIN;
    if (train) {
        BLT_REQUIRE(config->block_size >= 1, "blt_build_block_diffusion_mask: TRAIN mode needs block_size >= 1");
        BLT_REQUIRE((S - N) % config->block_size == 0,
                    "blt_build_block_diffusion_mask: block section must tile exactly (B * (M-1))");
        BLT_REQUIRE(config->block_starts != NULL, "blt_build_block_diffusion_mask: TRAIN mode needs block_starts");
        BLT_REQUIRE(config->num_blocks == (S - N) / config->block_size,
                    "blt_build_block_diffusion_mask: num_blocks must equal (S - N) / block_size");
        for (size_t b = 0; b < config->num_blocks; b++)
            BLT_REQUIRE(config->block_starts[b] < N,
                        "blt_build_block_diffusion_mask: block start must lie inside the clean prefix");
    }

    const size_t shape[2] = {S, S};
    *out_mask = blt_tensor_create_uninit(arena, shape, 2, BLT_DTYPE_FP32);

    BlockRecipe r;
    r.S = S;
    r.N = N;
    r.B = train ? config->block_size : 1;
    r.infer = train ? 0 : 1;
    r.starts = train ? stage_u64(config->block_starts, config->num_blocks, arena) : nullptr;

    if (S % 4u == 0u)
        blt_launch("mask_block_diffusion", block_diffusion_mask_kernel<4>, mask_grid(S, S, 4), dim3(256), 0, 0,
                   static_cast<float *>(out_mask->data), r);
    else
        blt_launch("mask_block_diffusion", block_diffusion_mask_kernel<1>, mask_grid(S, S, 1), dim3(256), 0, 0,
                   static_cast<float *>(out_mask->data), r);
    HIP_CHECK_LAUNCH("blt_build_block_diffusion_mask");
    /* Row i always sees column min(i, N-1) or itself, so no row can be empty
     * once the checks above hold; block_starts is caller memory and the copy
     * from it is staged before hipMemcpyAsync returns. */
}
