/*
 * C-ABI of the MI355X (gfx950) attention backend for fBLT.
 *
 * Part 1 are the device twins the reference's dispatcher binds: same
 * parameter lists as its `_cpu` / `_cuda` functions, `_hip` suffix.  Part 2 is
 * the device-memory shim the reference's core calls.  Part 3 is the host-side
 * mirror of the reference's own public API for this path (arena, dispatch,
 * patch index helpers) so that C callers written against the reference headers
 * link unchanged.  Part 4 are additive entry points that have no counterpart
 * in the reference: whole-batch launches and the batched KV-cache step.
 *
 * Errors: there are no return codes.  A violated precondition or a HIP error
 * prints "BLT Fatal Error [file:line]: ..." to stderr and calls
 * exit(EXIT_FAILURE), as the reference does (csrc/core/backend.h:13-31).
 *
 * Streams: everything is issued on the HIP default (null) stream of the
 * current device, in order, without host synchronisation unless stated.
 */
#ifndef FBLT_AMD_BLT_HIP_H
#define FBLT_AMD_BLT_HIP_H

#include "blt_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ===================================================================== */
/* Part 1 -- device twins of the reference ops                            */
/* ===================================================================== */

/* Replaces blt_attention_head_core_cuda (csrc/ops/attn_core.cu:288-311;
 * contract csrc/ops/attn_core.h:12-46).  All pointers are device pointers.
 * Needs at least one of weights_out / scores_scratch / lse_out.  Writes
 * combined[i, col_offset .. col_offset+head_dim); weights_out (post-softmax
 * weights, zeros where masked) when given; lse_out (row max, row sum) when
 * given.  scores_scratch is neither read nor written. */
void blt_attention_head_core_hip(blt_backend backend, const blt_attention_head_args *args);

/* Replaces blt_build_attention_mask_cuda (csrc/ops/mask_builder.cu:100-158).
 * Creates out_mask [seq_len_q, seq_len_kv] fp32 in the device arena (0 where
 * allowed, -INFINITY where not); index arrays in `config` are host pointers.
 * Blocks until the row-validity flags are back; aborts when a query row has
 * no allowed key. */
void blt_build_attention_mask_hip(const blt_mask_config *config, blt_tensor *out_mask, blt_arena *arena);

/* Replaces blt_build_block_diffusion_mask_cuda (csrc/ops/mask_builder.cu:187-216). */
void blt_build_block_diffusion_mask_hip(const blt_block_diffusion_config *config, blt_tensor *out_mask,
                                        blt_arena *arena);

/* Replaces blt_strided_copy_cuda (csrc/ops/vecmath.cu:144-163): rows x cols
 * fp32 tile between strided device buffers (head-slice gather, KV write-through). */
void blt_strided_copy_hip(blt_backend backend, float *dst, size_t dst_stride, const float *src,
                          size_t src_stride, size_t rows, size_t cols);

/* Replaces blt_rows_gather_cuda (csrc/ops/gather_scatter.cu:272-287; contract
 * csrc/ops/gather_scatter.h:41-42): dst[i, :] = src[pos_host[i], :] with whole-row
 * copies; pos_host is a HOST array (the rotary-table gather of the KV step,
 * csrc/infer/rope_gather.c:33-34).  No allocation, no synchronisation. */
void blt_rows_gather_hip(const blt_tensor *src, const size_t *pos_host, blt_tensor *dst);
/* csrc/ops/gather_scatter.h:21 (gather_scatter_cpu.c:7-21): out[i, :] = table[ids_host[i], :]; the
 * diffusion forward's learned D_0 rows (csrc/models/block_diffusion.c:140-146) */
void blt_embedding_lookup_hip(const blt_tensor *table, const uint32_t *ids_host, blt_tensor *out);
/* Replaces blt_indexed_row_accumulate_cuda (csrc/core/backend.c:515-518; contract
 * csrc/ops/gather_scatter.h:23-28, gather_scatter_cpu.c:41-61): io[i, :] += table[idx_host[i], :]
 * for every i whose index is not BLT_IDX_SENTINEL; idx_host is a HOST array [io rows].  The
 * hashed n-gram tables of the local encoder (csrc/models/hash_ngram.c:176-194).  Bit-identical. */
void blt_indexed_row_accumulate_hip(const blt_tensor *table, const uint32_t *idx_host, blt_tensor *io);
/* Replaces blt_scale_cuda (csrc/core/backend.c:262; csrc/ops/elementwise.h:10,
 * elementwise_cpu.c:31-40): t *= scalar in place.  Bit-identical. */
void blt_scale_hip(blt_tensor *t, float scalar);
/* Replaces blt_patch_pool_forward_cuda (contract csrc/ops/patch_pool.h:18-21, patch_pool_cpu.c:3-48):
 * out[j, :] = mean, or per-column maximum, of byte_hidden rows [start_j, start_j + len_j); patches
 * is a HOST array; empty or out-of-range patches are fatal as in the reference.  The rows of a
 * patch are added first to last and scaled by 1 / len: bit-identical. */
void blt_patch_pool_forward_hip(const blt_tensor *byte_hidden, const blt_patch_info *patches, size_t num_patches,
                                blt_patch_pool_type pool_type, blt_tensor *out);

/* Replaces blt_softmax_masked_row_inplace_cuda (csrc/ops/vecmath.cu:71-114):
 * the row softmax of csrc/ops/vecmath.h:20-31 on one device row. */
void blt_softmax_masked_row_inplace_hip(blt_backend backend, float *row, size_t row_len, size_t row_idx,
                                        bool is_causal, const float *mask_row, float scale);

/* Replaces blt_vec_dot_cuda (csrc/ops/vecmath.cu:20-69): device dot product,
 * result returned to the host (blocking). */
float blt_vec_dot_hip(blt_backend backend, const float *a, const float *b, size_t n);

/* Replaces blt_matmul_cuda (csrc/ops/linalg.cu:48-134): out[M,N] = a[M,K] *
 * b[K,N], row-major fp32 device tensors.  Up to 32 rows the result is
 * bit-identical to blt_matmul_cpu (csrc/ops/linalg_cpu.c:8-18); above that it
 * is accumulated on the matrix cores in another order.  BF16 operands, which
 * the reference converts first, are rejected. */
void blt_matmul_hip(const blt_tensor *a, const blt_tensor *b, blt_tensor *out);

/* Replaces blt_rope_apply_cuda (csrc/ops/reductions.cu:253-319): x, out are
 * [seq_len, num_heads, head_dim], cos / sin [seq_len, head_dim/2]; row t is
 * rotated by table row t.  Bit-identical to blt_rope_apply_cpu. */
void blt_rope_apply_hip(const blt_tensor *x, const blt_tensor *cos, const blt_tensor *sin, blt_tensor *out);

/* Replaces blt_rope_apply_packed_cuda (csrc/ops/reductions.cu:321-340): the
 * same rotation in place on one head's column block of packed rows. */
void blt_rope_apply_packed_hip(float *qkv_data, size_t qkv_stride, size_t head_offset, size_t seq_len,
                               size_t head_dim, const float *cos, const float *sin);

/* blt_cross_attention_forward for device tensors (csrc/models/
 * cross_attention.c:101-157): Q projection, K and V projections in one launch
 * (they share the input), all heads in one attention launch with the patch
 * mask reduced to per-row key ranges on the host (blt_mask_config_row_ranges;
 * dense device-built mask when a configuration does not reduce), output
 * projection.  No positional embedding, no residual, as in the reference. */
void blt_cross_attention_forward_hip(const blt_tensor *query_in, const blt_tensor *kv_in,
                                     const blt_cross_attention_weights *weights, blt_tensor *output,
                                     const blt_cross_attention_config *config, blt_arena *arena);

/* Device twins of the cache-aware decoder step (csrc/infer/kv_cache.c:
 * 112-159 and 161-416) with the reference's signatures, for a cache, decoder
 * weights and rows that live in device memory.  refresh_cross: one launch per
 * firing layer computes K and V of the new sub-tokens straight into the
 * tier-2 slabs.  decode_step: per layer the cross block (RMSNorm + Q
 * projection with the rows' few sub-tokens attended in its epilogue where the
 * shape allows, projection + residual: 2-3 launches) and the self-attention /
 * feed-forward layer (5 launches), then the LM head; the dense masks, strided
 * copies and per-head calls of the reference are gone, the row groups follow
 * the same latent rule (kv_cache.c:199-213).  A prompt chunk of more than 32
 * rows is staged once (rotation, write-through) and attended by the prefill
 * kernels with the causal diagonal moved by the cached length.  Up to 32 new
 * rows every projection is bit-identical to the CPU reference; attention is
 * within fp32 tolerance. */
void blt_kv_cache_refresh_cross_hip(blt_kv_cache *cache, const blt_tensor *patch_in, const blt_patch_info *patches,
                                    size_t num_patches, size_t from_patch, blt_arena *arena);
void blt_kv_decode_step_hip(blt_kv_cache *cache, const blt_tensor *patch_in, const blt_patch_info *patches,
                            size_t num_patches, const blt_tensor *d0_rows, int trailing_closed,
                            blt_tensor *logits_out, blt_arena *arena);

/* Replace blt_rmsnorm_forward_cuda (csrc/ops/reductions.cu:390-396; CPU loop
 * reductions_cpu.c:327-352, bit-identical here), blt_add_cuda and
 * blt_swiglu_forward_cuda (csrc/ops/elementwise.cu:102-134; CPU loops
 * elementwise_cpu.c:9-18 exact, 86-99 within fp32 tolerance). */
void blt_rmsnorm_forward_hip(const blt_tensor *x, const blt_tensor *weight, blt_tensor *out);
void blt_add_hip(const blt_tensor *a, const blt_tensor *b, blt_tensor *out);
void blt_swiglu_forward_hip(const blt_tensor *gate, const blt_tensor *up, blt_tensor *out);

/* blt_multihead_attention for device tensors (csrc/models/attention.c:
 * 130-207): QKV projection (+ rotation), all heads in one attention launch,
 * output projection.  Work buffers come from `arena` (a device arena); when
 * use_rope is set without caches the tables are computed on the host by
 * blt_rope_precompute and uploaded. */
void blt_multihead_attention_hip(const blt_tensor *input, const blt_tensor *weight_qkv,
                                 const blt_tensor *weight_proj, blt_tensor *output,
                                 const blt_attention_config *config, blt_arena *arena);

/* csrc/models/transformer.h (transformer.c:97-128): the pre-norm block every BLT transformer is
 * made of -- RMSNorm, attention block, residual, RMSNorm, SwiGLU feed-forward, residual; called
 * once per layer by the patch transformer (csrc/models/transformer_stack.c:228-248 under
 * global_transformer.c:69-97) and by the local encoder (csrc/models/local_encoder.c:243-248).
 * RMSNorm + SwiGLU with FP32 weights only. */
void blt_transformer_forward_hip(const blt_tensor *input, const blt_transformer_weights *weights, blt_tensor *output,
                                 const blt_transformer_config *config, blt_arena *arena);

/* csrc/models/local_encoder.h:71-73 (local_encoder.c:193-281): bytes -> byte embedding + hashed
 * n-gram embeddings -> P_0 = pooled patches (repeated over the k sub-token column blocks) -> per
 * layer the byte transformer block and, where it fires, P += cross_attention(RMSNorm(P), h).
 * bytes_in [seq_len] UINT8 on either side (the ids are hashed on the host, as in the reference);
 * weights, outputs and the arena are device memory; patches, doc_boundaries are HOST arrays.
 * Unlike the reference's body on a device arena, sub-token splits (patch_dim = k * embed_dim,
 * k > 1) work: the expanded group ids are host memory here. */
/* csrc/models/local_decoder.c:233-351 on the device: per layer the cross block (when it fires)
 * in three launches and the byte block in five, then the LM head. */
void blt_local_decoder_forward_ext_hip(const blt_local_decoder *model, const blt_tensor *byte_hidden_in,
                                       const blt_tensor *patch_in, const blt_patch_info *patches, size_t num_patches,
                                       const size_t *doc_boundaries, size_t num_docs, int trailing_closed,
                                       blt_tensor *logits_out, blt_arena *arena);
void blt_local_encoder_forward_hip(const blt_local_encoder *model, const blt_tensor *bytes_in,
                                   const blt_patch_info *patches, size_t num_patches, const size_t *doc_boundaries,
                                   size_t num_docs, blt_tensor *patch_out, blt_tensor *byte_hidden_out,
                                   blt_arena *arena);

/* ===================================================================== */
/* Part 2 -- device memory shim (csrc/core/cuda_shim.h:18-31,             */
/*           csrc/ops/memory.cu:19-77)                                    */
/* ===================================================================== */
void *blt_hip_malloc(size_t bytes);
void blt_hip_free(void *ptr);
void blt_hip_memset(void *dst, int value, size_t bytes);                 /* async, default stream */
void blt_hip_memcpy_h2d(void *dst, const void *src, size_t bytes);       /* src is consumed on return; the copy itself is ordered on the library's stream */
void blt_hip_memcpy_d2h(void *dst, const void *src, size_t bytes);       /* blocking */
void blt_backend_pass_sync_hip(void);                                    /* device sync + error check */

/* ===================================================================== */
/* Part 3 -- host mirror of the reference's public API for this path      */
/* ===================================================================== */

/* csrc/core/allocator.h:18-23 (allocator.c:36-160).  backend selects host or
 * device memory for the arena's buffer. */
blt_arena *blt_arena_create(size_t capacity_bytes, blt_backend backend);
void blt_arena_destroy(blt_arena *arena);
void blt_arena_reset(blt_arena *arena);
void *blt_arena_alloc(blt_arena *arena, size_t bytes, size_t alignment);
/* csrc/core/allocator.h:33 (tensor.c:154-162, backend.c:494-501).  Memory the caller fills and
 * reads on the host (group-id arrays, weight-view and model structs): arena memory on the CPU
 * backend, zeroed host memory for a device arena, plus a 64-byte token of the arena that marks the
 * block's place in it.  A device arena's blocks are released with blt_arena_reset /
 * blt_arena_destroy, or once the arena's offset has been rewound to or below their token. */
void *blt_container_alloc(blt_arena *arena, size_t bytes);
blt_tensor blt_tensor_create(blt_arena *arena, const size_t *shape, size_t ndim, blt_dtype dtype);
blt_tensor blt_tensor_create_uninit(blt_arena *arena, const size_t *shape, size_t ndim, blt_dtype dtype);
/* csrc/core/allocator.h:35-41 */
void blt_tensor_upload(blt_tensor *dst, const void *host_src, size_t bytes);
void blt_tensor_download(const blt_tensor *src, void *host_dst, size_t bytes);
/* csrc/core/backend.h:61-63 */
void blt_backend_pass_sync(blt_backend backend);

/* Run-time dispatch with the reference's signatures (csrc/core/backend.c:
 * 455-492).  This library holds no CPU compute path: a call tagged
 * BLT_BACKEND_CPU is a fatal error, never a silent fallback. */
void blt_attention_head_core(blt_backend backend, const blt_attention_head_args *args);
void blt_build_attention_mask(const blt_mask_config *config, blt_tensor *out_mask, blt_arena *arena);
void blt_build_block_diffusion_mask(const blt_block_diffusion_config *config, blt_tensor *out_mask,
                                    blt_arena *arena);
void blt_strided_copy(blt_backend backend, float *dst, size_t dst_stride, const float *src, size_t src_stride,
                      size_t rows, size_t cols);
void blt_softmax_masked_row_inplace(blt_backend backend, float *row, size_t row_len, size_t row_idx,
                                    bool is_causal, const float *mask_row, float scale);
float blt_vec_dot(blt_backend backend, const float *a, const float *b, size_t n);
/* csrc/core/backend.c:532-534: the backend comes from src. */
void blt_rows_gather(const blt_tensor *src, const size_t *pos_host, blt_tensor *dst);
void blt_embedding_lookup(const blt_tensor *table, const uint32_t *ids_host, blt_tensor *out);
/* csrc/core/backend.c:515-518, 262; csrc/ops/patch_pool.h:20: the backend comes from the first tensor. */
void blt_indexed_row_accumulate(const blt_tensor *table, const uint32_t *idx_host, blt_tensor *io);
void blt_scale(blt_tensor *t, float scalar);
void blt_patch_pool_forward(const blt_tensor *byte_hidden, const blt_patch_info *patches, size_t num_patches,
                            blt_patch_pool_type pool_type, blt_tensor *out);
/* csrc/infer/rope_gather.h / rope_gather.c:5-35: rows positions[0..n) of the two rotary
 * tables into new [n, half] tensors of the arena. */
void blt_rope_position_gather(const blt_tensor *cos_cache, const blt_tensor *sin_cache, const size_t *positions,
                              size_t n, blt_tensor *cos_out, blt_tensor *sin_out, blt_arena *arena);
/* csrc/core/backend.c:397-399, 307-345; csrc/models/attention.h:24-26.  The
 * backend comes from the first tensor (matmul, rope_apply), the output
 * tensors (precompute), the explicit argument (packed) or the input tensor
 * (attention block). */
void blt_matmul(const blt_tensor *a, const blt_tensor *b, blt_tensor *out);
/* Tables for device tensors are computed on the host with the reference's
 * own formula and libm calls (csrc/ops/reductions_cpu.c:179-197), so they are
 * bit-identical to the CPU reference, then uploaded (blocking). */
void blt_rope_precompute(size_t max_seq_len, const blt_rope_config *config, blt_tensor *cos_out, blt_tensor *sin_out);
void blt_rope_apply(const blt_tensor *x, const blt_tensor *cos, const blt_tensor *sin, blt_tensor *out);
void blt_rope_apply_packed(float *qkv_data, size_t qkv_stride, size_t head_offset, size_t seq_len, size_t head_dim,
                           const float *cos, const float *sin, blt_backend backend);
void blt_multihead_attention(const blt_tensor *input, const blt_tensor *weight_qkv, const blt_tensor *weight_proj,
                             blt_tensor *output, const blt_attention_config *config, blt_arena *arena);
/* csrc/models/cross_attention.h:49-51 */
void blt_cross_attention_forward(const blt_tensor *query_in, const blt_tensor *kv_in,
                                 const blt_cross_attention_weights *weights, blt_tensor *output,
                                 const blt_cross_attention_config *config, blt_arena *arena);
/* csrc/core/backend.c:254-256, 276-278, 380-382 */
void blt_transformer_forward(const blt_tensor *input, const blt_transformer_weights *weights, blt_tensor *output,
                             const blt_transformer_config *config, blt_arena *arena);
/* csrc/models/local_encoder.h:71-73 */
/* csrc/models/local_decoder.h:112-125 (local_decoder.c:233-361), the inference form: loss_out
 * must be NULL (the loss is a training op) and d0_opts NULL or BLT_D0_HFINAL (block rows with
 * their own D_0 go through blt_local_decoder_forward_diffusion_infer). */
void blt_local_decoder_forward_ext(const blt_local_decoder *model, const blt_tensor *byte_hidden_in,
                                   const blt_tensor *patch_in, const blt_patch_info *patches, size_t num_patches,
                                   const blt_tensor *bytes_in, const blt_tensor *targets, const size_t *doc_boundaries,
                                   size_t num_docs, const blt_local_decoder_d0_opts *d0_opts, int trailing_closed,
                                   blt_tensor *logits_out, blt_tensor *loss_out, blt_arena *arena);
void blt_local_encoder_forward(const blt_local_encoder *model, const blt_tensor *bytes_in, const blt_patch_info *patches,
                               size_t num_patches, const size_t *doc_boundaries, size_t num_docs, blt_tensor *patch_out,
                               blt_tensor *byte_hidden_out, blt_arena *arena);
void blt_add(const blt_tensor *a, const blt_tensor *b, blt_tensor *out);
void blt_swiglu_forward(const blt_tensor *gate, const blt_tensor *up, blt_tensor *out);
void blt_rmsnorm_forward(const blt_tensor *x, const blt_tensor *weight, blt_tensor *out);

/* csrc/infer/kv_cache.h:70-117 and csrc/models/local_common.h:68-69.  The
 * cache container and its handle arrays live on the host heap, the K/V
 * payloads come zero-filled from `arena` (kv_cache.c:27-75); reset, truncate
 * and common_patches are host bookkeeping (kv_cache.c:77-110). */
blt_kv_cache *blt_kv_cache_create(blt_arena *arena, const blt_local_decoder *decoder, size_t max_seq_len);
blt_kv_cache *blt_kv_cache_create_batched(blt_arena *arena, const blt_local_decoder *decoder, size_t max_seq_len,
                                          size_t batch_size);
void blt_kv_cache_destroy(blt_kv_cache *cache);
void blt_kv_cache_reset(blt_kv_cache *cache);
void blt_kv_cache_truncate(blt_kv_cache *cache, size_t self_len, size_t num_patches);
size_t blt_kv_cache_common_patches(const blt_kv_cache *cache, const blt_patch_info *patches, size_t num_patches);
void blt_kv_cache_refresh_cross(blt_kv_cache *cache, const blt_tensor *patch_in, const blt_patch_info *patches,
                                size_t num_patches, size_t from_patch, blt_arena *arena);
void blt_kv_decode_step(blt_kv_cache *cache, const blt_tensor *patch_in, const blt_patch_info *patches,
                        size_t num_patches, const blt_tensor *d0_rows, int trailing_closed, blt_tensor *logits_out,
                        blt_arena *arena);
void blt_local_decoder_forward_diffusion_infer(const blt_local_decoder *model, const blt_tensor *byte_hidden_in,
                                               const blt_tensor *patch_in, const blt_patch_info *patches,
                                               size_t num_patches, const blt_block_batch *batch, blt_d0_mode d0_mode,
                                               blt_tensor *logits_out, blt_arena *arena);
bool blt_local_cross_attn_fires(blt_xattn_placement placement, bool cross_attn_all_layers, size_t num_layers,
                                size_t layer);

/* Byte<->patch index helpers; host integer code in the reference as well
 * (csrc/ops/patch_pool.h:29-41, patch_pool_cpu.c:98-142). */
void blt_patch_build_group_ids(const blt_patch_info *patches, size_t num_patches, size_t seq_len,
                               size_t *query_group_ids_out, size_t *kv_group_ids_out);
size_t blt_patch_decoder_latent_at(const blt_patch_info *patches, size_t num_patches, size_t pos);
void blt_patch_expand_group_ids(const size_t *group_ids_in, size_t n, size_t k, size_t *group_ids_out);

/* ===================================================================== */
/* Part 4 -- additive entry points (no counterpart in the reference)      */
/* ===================================================================== */

/* How a problem says which (query, key) pairs are visible without a dense
 * [nq, nk] matrix in memory. */
typedef enum {
    BLT_ATTN_MASK_FROM_HEAD = 0, /* use head.mask / head.is_causal as the per-head call does */
    BLT_ATTN_MASK_CAUSAL = 1,    /* j <= i + causal_offset, and i + causal_offset - j < window if window > 0 */
    BLT_ATTN_MASK_ROW_RANGE = 2  /* row i sees keys row_lo[i] <= j < row_hi[i] (device uint32 arrays) */
} blt_attn_mask_kind;

/* One (sequence, head) problem of a batch: the reference's argument block
 * plus an optional mask descriptor.  With a descriptor, head.mask must be
 * NULL; none of the three score buffers is required. */
typedef struct {
    blt_attention_head_args head;
    uint32_t mask_kind; /* blt_attn_mask_kind */
    uint32_t row_span;  /* BLT_ATTN_MASK_ROW_RANGE: the longest range of any row when the caller knows it (it built
                           the ranges on the host); 0 = unknown, taken as short.  Short ranges (a patch's bytes) run
                           one row per wave; long ones (document-causal self-attention) on the matrix cores. */
    size_t causal_offset;
    size_t window;
    const uint32_t *row_lo; /* device, [nq] */
    const uint32_t *row_hi; /* device, [nq] */
} blt_attention_problem;

/* All problems of a forward pass in one go: what the reference issues as a
 * caller loop of count per-head calls (csrc/models/attention.c:199-202,
 * cross_attention.c:147-150).  `problems` is a HOST array; it is staged to the
 * device on the default stream before the kernels that read it. */
void blt_attention_batch_hip(const blt_attention_problem *problems, size_t count);

/* A batch whose descriptors stay resident on the device, for callers that
 * run the same set of problems repeatedly (same pointers, new contents). */
typedef struct blt_attention_plan blt_attention_plan;
blt_attention_plan *blt_attention_plan_create_hip(const blt_attention_problem *problems, size_t count);
void blt_attention_plan_run_hip(const blt_attention_plan *plan);
void blt_attention_plan_destroy_hip(blt_attention_plan *plan);
/* Name of the kernel family the plan selected ("rows", "mfma32", ...), for logs. */
const char *blt_attention_plan_kernel_hip(const blt_attention_plan *plan);

/* Row ranges equivalent to a blt_mask_config, computed on the host in
 * O(nq + nk): returns 1 and fills lo/hi (host arrays [seq_len_q]) when every
 * row's allowed set is one contiguous key range (true for causal, window,
 * document and sorted-group masks), 0 when it is not (then use the dense
 * mask).  Rows with no allowed key get lo == hi. */
int blt_mask_config_row_ranges(const blt_mask_config *config, uint32_t *lo, uint32_t *hi);

/* Batched tier-1 KV cache in the layout blt_kv_cache_create_batched reserves
 * (csrc/infer/kv_cache.c:27-71): self_k / self_v are [batch*max_seq_len,
 * embed_dim] fp32 row-major, row b*max_seq_len + pos holds absolute position
 * pos of sequence b.  self_len is a DEVICE array [batch] of valid rows. */
typedef struct {
    float *self_k;
    float *self_v;
    uint32_t *self_len;
    size_t batch;
    size_t max_seq_len;
    size_t embed_dim;
    size_t num_heads;
    size_t window; /* local_window of the decoder, 0 = none */
} blt_kv_attn_cache;

enum {
    BLT_KV_STEP_CAUSAL = 0, /* new row r sees keys j <= self_len + r (kv_cache.c:229-236) */
    BLT_KV_STEP_BLOCK = 1   /* every new row sees all self_len + n keys (INFER block rows,
                               mask_builder_cpu.c:133-135) */
};

/* The attention statements of blt_kv_decode_step (csrc/infer/kv_cache.c:
 * 343-390) for every sequence of the batch in one launch: write the n new
 * K/V rows of each sequence through to rows [len_b, len_b+n) FIRST, then
 * attend over rows [0, len_b+n) for every head, write combined[b*n + r, :]
 * and, when `commit` is non-zero, advance self_len[b] by n.  q_rows, k_rows,
 * v_rows and combined are [batch*n, *] with the given row strides (elements);
 * K rows are already rotated.  max_len_hint >= max_b(self_len[b]) + n sizes
 * the launch (the host knows it, as the reference's host-side self_len does);
 * sequences shorter than the hint simply leave blocks idle.  A sequence whose
 * device-side length + n exceeds the hint (rounded up to the launch's span),
 * max_seq_len or the rotation tables is left untouched -- no write-through, no
 * output rows, no commit -- and the next synchronising call of the library
 * (blt_backend_pass_sync_hip, blt_hip_memcpy_d2h, blt_tensor_download) ends
 * with "exceeds cache capacity", the reference's check of csrc/infer/
 * kv_cache.c:191 made where the lengths live.  A causal step
 * of more than 32 rows per sequence (a prompt prefill) is run as consecutive
 * 32-row slices; a block step takes at most 32 rows (the reference's
 * BLT_BLOCKGEN_MAX_B, csrc/infer/block_generation.c:154). */
void blt_kv_attend_step_hip(const blt_kv_attn_cache *cache, const float *q_rows, size_t q_stride,
                            const float *k_rows, size_t k_stride, const float *v_rows, size_t v_stride,
                            float *combined, size_t combined_stride, size_t n, int step_kind, int commit,
                            size_t max_len_hint);

/* blt_kv_attend_step_hip for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid it).  No counterpart in the reference.  Same
 * arguments, same kernels, same results; the per-split softmax records, the per-sequence tickets
 * and the error word come from a fixed device array inside the library (4 MiB of records, 4096
 * sequences; one copy per GPU, held until the process ends) instead of buffers that grow on demand,
 * and the call issues no hipMalloc / hipFree.  A step that needs more (batch * splits * heads *
 * row slots * (head_dim + 2) floats of records with splits > 1, or more than 4096 sequences) ends
 * with a message naming both figures.  All calls on one GPU share the array: calls that overlap
 * on that GPU (two streams, two threads) race; issue them in order on one stream. */
void blt_kv_attend_step_noalloc_hip(const blt_kv_attn_cache *cache, const float *q_rows, size_t q_stride,
                                    const float *k_rows, size_t k_stride, const float *v_rows, size_t v_stride,
                                    float *combined, size_t combined_stride, size_t n, int step_kind, int commit,
                                    size_t max_len_hint);

/* blt_kv_attend_step_hip with the rotation of the new rows fused in: the step
 * of blt_kv_decode_step from the QKV projection's output to `combined`
 * (csrc/infer/kv_cache.c:262-271 position gather, 343-366 per-head copy-out,
 * blt_rope_apply of Q and K, copy-back and write-through, 368-390 attention).
 * q_rows / k_rows / v_rows are the UN-rotated new rows, typically the three
 * column blocks of the packed [batch*n, 3E] projection output (stride 3E).
 * Row r of sequence b sits at position self_len[b] + r; Q and K pairs
 * (2i, 2i+1) of every head are rotated by rope_cos / rope_sin
 * [rope_positions, head_dim/2] (DEVICE copies of the tables
 * blt_rope_precompute fills, csrc/ops/reductions_cpu.c:179-197) exactly as
 * blt_rope_apply_cpu does (reductions_cpu.c:199-229), so the K rows stored in
 * the cache are bit-identical to the reference's.  Requires max_len_hint <=
 * rope_positions.  One launch replaces the reference's 6 strided copies + 2
 * rotations + 1 attention call per head. */
void blt_kv_rope_attend_step_hip(const blt_kv_attn_cache *cache, const float *q_rows, size_t q_stride,
                                 const float *k_rows, size_t k_stride, const float *v_rows, size_t v_stride,
                                 const float *rope_cos, const float *rope_sin, size_t rope_positions,
                                 float *combined, size_t combined_stride, size_t n, int step_kind, int commit,
                                 size_t max_len_hint);

/* The single-row step with the lengths where the reference keeps them: on the
 * host (blt_kv_cache.self_len, csrc/infer/kv_cache.h:56-60; advanced by the
 * caller after the step, kv_cache.c:416).  self_len_host[b] is the number of
 * valid rows of sequence b; cache->self_len (the device array) is neither read
 * nor written and may be NULL.  The lengths travel in the kernel arguments, so
 * the first K/V requests of a workgroup depend on nothing but the argument
 * block -- one memory round trip less than the device-length step -- and the
 * capacity check of kv_cache.c:191 is made on the host before anything is
 * launched ("exceeds cache capacity").  rope_cos / rope_sin as in
 * blt_kv_rope_attend_step_hip, or both NULL for rows that arrive rotated.
 * n and step_kind as in blt_kv_attend_step_hip (single rows, causal chunks,
 * blocks of at most 32 rows); nothing is committed on the device.  Head
 * widths the matrix-core block kernels do not take (anything but 32 and 64)
 * with n > 1 stage the lengths to a device array of the library's and run the
 * device-length kernels.  Not for replay from a graph: the lengths are frozen
 * into the launch. */
void blt_kv_attend_step_lens_hip(const blt_kv_attn_cache *cache, const uint32_t *self_len_host,
                                 const float *q_rows, size_t q_stride, const float *k_rows, size_t k_stride,
                                 const float *v_rows, size_t v_stride, const float *rope_cos, const float *rope_sin,
                                 size_t rope_positions, float *combined, size_t combined_stride, size_t n,
                                 int step_kind);

/* One decoder layer of blt_kv_decode_step (csrc/infer/kv_cache.c:326-414
 * without the optional cross-attention: RMSNorm, QKV projection, rotation +
 * write-through + attention of the new rows, output projection, residual;
 * RMSNorm, up / gate projections, SwiGLU, down projection, residual) for ALL
 * sequences of a batched cache at once: rows_in / rows_out are [batch*n,
 * embed_dim] device rows (rows_out may alias rows_in), sequence b's rows sit
 * at positions self_len[b] .. self_len[b]+n-1.  The reference runs this for
 * one sequence at a time; batching leaves every sequence's arithmetic
 * untouched apart from the projections' summation order above 32 rows.  Work
 * buffers come from `arena` (device).  Blocks with RMSNorm and SwiGLU only.
 * No counterpart in the reference (its batched decode is reserved storage,
 * csrc/infer/kv_cache.h:71-75). */
void blt_kv_decode_layer_hip(const blt_kv_attn_cache *cache, const blt_transformer_weights *weights,
                             const float *rows_in, float *rows_out, const float *rope_cos, const float *rope_sin,
                             size_t rope_positions, size_t n, int step_kind, int commit, size_t max_len_hint,
                             blt_arena *arena);

/* The decoder step for every sequence of a batched cache at once -- the
 * decode indexing the reference reserves storage for but does not implement
 * (csrc/infer/kv_cache.h:71-75).  Sequence b has self_len[b] valid byte rows
 * (HOST array [batch_size], advanced by n on return; the cache's own scalar
 * self_len / cross_num_patches are not used), its own patch table patches[b]
 * of num_patches[b] entries whose sub-tokens refresh_cross_seq has written,
 * and n = d0_rows->shape[0] / batch_size new rows at d0_rows[b*n .. b*n+n);
 * trailing_closed may be NULL (all 0).  logits_out is [batch_size*n,
 * vocab_size].  Every sequence's arithmetic is that of blt_kv_decode_step_hip
 * on that sequence alone, apart from the projections' summation order once
 * batch_size*n exceeds 32 rows.  Lengths and row groups are staged through
 * host memory: not capturable into a graph. */
void blt_kv_cache_refresh_cross_seq_hip(blt_kv_cache *cache, size_t seq, const blt_tensor *patch_in,
                                        const blt_patch_info *patches, size_t num_patches, size_t from_patch,
                                        blt_arena *arena);
void blt_kv_decode_step_batched_hip(blt_kv_cache *cache, size_t *self_len, const blt_patch_info *const *patches,
                                    const size_t *num_patches, const int *trailing_closed, const blt_tensor *d0_rows,
                                    blt_tensor *logits_out, blt_arena *arena);

/* csrc/models/block_diffusion.h:131-134 (block_diffusion.c:776-795): the inference-mode diffusion
 * forward over [clean prefix ; block rows] -- the call blt_draft_block makes once per denoising
 * pass (csrc/infer/block_generation.c:156-266).  Same parameter list; every tensor and the arena
 * in device memory; logits_out is [num_clean + n_block_rows, vocab_size].  The reference runs all
 * S rows through S x S attention against the dense INFER mask; here the clean rows are the
 * incremental decoder step over an empty cache (a clean row never sees a block row,
 * csrc/ops/mask_builder_cpu.c:128-131) and the block rows one block step over what it cached
 * (133-135) -- the same arithmetic per row, projections in their summation order above 32 rows
 * apart.  At most 32 block rows (the reference's BLT_BLOCKGEN_MAX_B).  As in the reference the
 * decoder's local_window plays no part. */
void blt_local_decoder_forward_diffusion_infer_hip(const blt_local_decoder *model, const blt_tensor *byte_hidden_in,
                                                   const blt_tensor *patch_in, const blt_patch_info *patches,
                                                   size_t num_patches, const blt_block_batch *batch,
                                                   blt_d0_mode d0_mode, blt_tensor *logits_out, blt_arena *arena);

/* The block rows of that forward over a cache that already holds the clean prefix (sequence 0:
 * cache->self_len == batch->num_clean rows, tier 2 refreshed for num_patches patches): what a
 * denoising pass needs when the prefix was decoded through blt_kv_decode_step, without
 * recomputing it -- the cost of a pass no longer depends on the prefix length beyond reading its
 * K and V once.  logits_out is [n_block_rows, vocab_size]; row r cross-attends latent
 * batch->groups[r], sits at rotary position batch->positions[r] and starts from zeros or from
 * d0_embed_weight[batch->tokens[r]].  Nothing is committed: the cache's lengths stay, rows past
 * self_len are scratch.  No counterpart in the reference, whose draft loop recomputes the prefix
 * on every pass. */
void blt_kv_block_step_hip(blt_kv_cache *cache, size_t num_patches, const blt_block_batch *batch, blt_d0_mode d0_mode,
                           blt_tensor *logits_out, blt_arena *arena);

/* The stream every launch, asynchronous copy and memset of the library goes
 * to, per calling thread: the null stream (the reference's behaviour) unless
 * set otherwise.  `stream` is a hipStream_t. */
void blt_hip_set_stream(void *stream);
void *blt_hip_get_stream(void);

/* Record the library calls issued between begin and end into a HIP graph
 * instead of running them (the calls go to a library-owned stream under
 * hipStreamBeginCapture), and replay them with one graph launch on the
 * current stream: for launch-bound loops such as a decode step of several
 * small kernels.  Calls that would allocate device memory or stage
 * descriptors through host memory during a capture end with a message: run
 * each call once eagerly first; use resident plans or strided batches for
 * attention.  A replay repeats the recorded launches with the recorded
 * arguments (pointers, lengths hints); data behind the pointers is read anew. */
typedef struct blt_hip_graph blt_hip_graph;
void blt_hip_capture_begin(void);
blt_hip_graph *blt_hip_capture_end(void);
void blt_hip_graph_launch(const blt_hip_graph *graph);
void blt_hip_graph_destroy(blt_hip_graph *graph);

/* Per-kernel device time of every launch the library issues between begin and
 * end, from HIP events attached to each dispatch (the kernel's own begin/end
 * timestamps, without launch gaps).  `end` synchronises the device, fills up to
 * `capacity` rows (one per kernel tag) and returns the number of tags seen. */
typedef struct {
    char name[48];
    uint64_t launches;
    double total_ms;
    double min_ms;
    double max_ms;
} blt_hip_kernel_time;
void blt_hip_profile_begin(void);
size_t blt_hip_profile_end(blt_hip_kernel_time *out, size_t capacity);
/* The same close, launch by launch: the duration in milliseconds of every launch since `begin`, in
 * the order they were issued (up to `capacity` of them); returns the number of launches seen.
 * For medians and percentiles of a kernel's duration. */
size_t blt_hip_profile_end_list(float *ms_out, size_t capacity);

/* Library build tag and the architecture its kernels were compiled for. */
const char *blt_hip_build_info(void);

#ifdef __cplusplus
}
#endif

#endif /* FBLT_AMD_BLT_HIP_H */
