/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * Single-threaded CPU restatement of the reference's attention path, used as
 * the checker for the HIP backend and as the timed CPU baseline.  Nothing in
 * the shipped library links, loads or calls this file.
 *
 * Every function names the reference lines it restates.  Build flags follow
 * the reference (CMakeLists.txt:10-12,43,120): -std=c99 -O2, no -march, no
 * fast-math, plus -ffp-contract=off so no fused multiply-add can appear.
 *
 * How each function is pinned (none is "parity unpinned"):
 *   orc_vec_dot, orc_softmax_masked_row_inplace, orc_attention_head_core
 *       bit-for-bit against the reference compiled from its own sources
 *       (oracle/_ref), the reference's inline vectors
 *       (tests/unit/models/unit_attention.c:82-88,167-171,
 *       unit_cross_attention.c:111-117), closed forms (two-key sigmoid,
 *       uniform weights, single visible key, all-masked row) and a float64
 *       brute force on tiny shapes.
 *   orc_build_attention_mask, orc_build_block_diffusion_mask
 *       bit-for-bit against oracle/_ref over the reference's variant matrix
 *       (tests/parity/parity_cuda_composites.c:66-150), the hard-coded 14x14
 *       TRAIN matrix and INFER rule (tests/unit/models/unit_block_diffusion.c:
 *       123-172), the causal/window/doc/group cases of
 *       tests/unit/backend/unit_mask.c:14-192.
 *   orc_patch_build_group_ids, orc_patch_decoder_latent_at,
 *   orc_patch_expand_group_ids
 *       the expected arrays of tests/unit/models/unit_local_decoder.c:94-113
 *       and tests/unit/backend/unit_mask.c:116-127, plus oracle/_ref.
 *   orc_strided_copy, orc_kv_* (slab indexing, step masks, write-through,
 *   attend)
 *       against oracle/_ref op calls issued in the order of
 *       csrc/infer/kv_cache.c:343-390, and against the dense causal attention
 *       over the same rows (the reference's cached == dense invariant,
 *       tests/unit/infer/unit_kv_cache.c:136-151).
 *   orc_rope_precompute, orc_rope_apply, orc_rope_position_gather,
 *   orc_kv_rope_attend_step
 *       bit-for-bit against oracle/_ref (blt_rope_precompute_cpu,
 *       blt_rope_apply_cpu over the same rows); closed forms: position 0 is
 *       the identity, (cos, sin) = (0, 1) maps (x0, x1) to (-x1, x0) -- the
 *       forward twin of the reference's backward vector
 *       (tests/unit/backend/unit_reductions_cpu.c:133-157) --, pair norms are
 *       preserved, q.k after rotation depends only on the position
 *       difference; the step against rotating by hand and calling
 *       orc_kv_attend_step.
 *   orc_kv_cache_refresh_cross, orc_kv_cross_block, orc_kv_decode_step
 *       bit-for-bit (logits and all four cache tiers) against oracle/_ref's
 *       blt_kv_cache_refresh_cross and blt_kv_decode_step (csrc/infer/
 *       kv_cache.c) over prefill chunks and single-row steps, with and
 *       without window, sub-token split and trailing_closed; and through the
 *       reference's own invariant that the cached steps reproduce the dense
 *       decoder forward (tests/unit/infer/unit_kv_cache.c:136-151), here
 *       blt_local_decoder_forward of oracle/_ref.
 *   orc_matmul, orc_rope_apply_packed, orc_multihead_attention,
 *   orc_cross_attention_forward
 *       bit-for-bit against oracle/_ref (blt_matmul, blt_rope_apply_packed,
 *       blt_multihead_attention and blt_cross_attention_forward compiled from
 *       csrc/models/attention.c and cross_attention.c; the cross block also
 *       against the numbers and the group isolation of
 *       tests/unit/models/unit_cross_attention.c:111-117, 229-246); the
 *       reference's vectors: [[1,2],[3,4]] x [[5,6],[7,8]] = [[19,22],[43,50]]
 *       (tests/unit/backend/unit_linalg_cpu.c:10-48) and the identity-weight
 *       two-token block -> {0.6697615, 0.3302385, ...}, causal row 0 one-hot
 *       (tests/unit/models/unit_attention.c:82-88, 160-171); a float64 numpy
 *       product; the block against its parts called by hand.
 *   orc_rmsnorm_forward, orc_add, orc_swiglu_forward, orc_kv_decode_layer, orc_transformer_forward
 *       bit-for-bit against oracle/_ref (blt_rmsnorm_forward, blt_add, blt_swiglu_forward,
 *       blt_transformer_forward); RMSNorm of a constant row = +-weight, silu(0) = 0, float64.
 *   orc_local_decoder_forward
 *       bit-for-bit against oracle/_ref's blt_local_decoder_forward_ext (window, documents,
 *       sub-token split, trailing_closed) and against the incremental decoder step over the same
 *       rows; with the encoder and the block restatement, the whole blt_model_forward.
 *   orc_local_decoder_forward_diffusion_infer, orc_kv_block_step, orc_kv_*_step_kind
 *       bit-for-bit against oracle/_ref's blt_local_decoder_forward_diffusion_infer over D_0
 *       modes, sub-token split, window, placements and block geometry; the cached form (prefix as
 *       an incremental step, block rows as one block step) bit-for-bit against the dense one.
 *   orc_indexed_row_accumulate, orc_scale, orc_patch_pool_forward, orc_ngram_indices,
 *   orc_embed_bytes, orc_local_encoder_forward
 *       bit-for-bit against oracle/_ref: the three ops on random inputs with sentinel entries and
 *       patches of 1..30 rows, the index lists of n = 1..8 against the reference's own
 *       blt_rolling_hash_init / _update state machine (three prime / modulus pairs, a run of equal
 *       bytes), the whole forward (patch_out and byte_hidden_out) over sub-token splits, window,
 *       documents, every cross placement, both pools and 0..6 tables.
 */
#ifndef FBLT_AMD_ORACLE_H
#define FBLT_AMD_ORACLE_H

#include "blt_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Return codes: 0 = done; a positive value = the reference would have aborted
 * (BLT_REQUIRE) at this point; the value says which requirement. */
enum {
    ORC_OK = 0,
    ORC_ERR_NULL_BUFFER = 1,     /* attn_core_cpu.c:18-19 */
    ORC_ERR_NO_SCORE_BUFFER = 2, /* attn_core_cpu.c:20-21 */
    ORC_ERR_EMPTY_SHAPE = 3,     /* mask_builder_cpu.c:30 */
    ORC_ERR_ROW_WITHOUT_KEY = 4, /* mask_builder_cpu.c:93, 152 */
    ORC_ERR_BAD_BLOCK_CONFIG = 5,/* mask_builder_cpu.c:105-119 */
    ORC_ERR_PATCH_TILING = 6,    /* patch_pool_cpu.c:107-111 */
    ORC_ERR_CAPACITY = 7,        /* kv_cache.c:191 */
    ORC_ERR_ARG = 8              /* reductions_cpu.c:181, rope_gather.c:21-25 */
};

/* csrc/ops/vecmath_cpu.c:6-14 */
float orc_vec_dot(const float *a, const float *b, size_t n);

/* csrc/ops/vecmath_cpu.c:16-53 */
void orc_softmax_masked_row_inplace(float *row, size_t row_len, size_t row_idx, bool is_causal,
                                    const float *mask_row, float scale);

/* csrc/ops/vecmath_cpu.c:55-63 */
void orc_strided_copy(float *dst, size_t dst_stride, const float *src, size_t src_stride, size_t rows,
                      size_t cols);

/* csrc/ops/attn_core_cpu.c:16-57.  Weights land in weights_out, else in
 * scores_scratch, as the reference does. */
int orc_attention_head_core(const blt_attention_head_args *a);

/* The reference's caller loop: one core call per (sequence, head), in array
 * order (csrc/models/attention.c:199-202).  Stops at the first failure. */
int orc_attention_head_core_many(const blt_attention_head_args *a, size_t count);

/* csrc/ops/mask_builder_cpu.c:11-95.  `out` is [seq_len_q * seq_len_kv]. */
int orc_build_attention_mask(const blt_mask_config *config, float *out);

/* csrc/ops/mask_builder_cpu.c:97-154.  `out` is [seq_len * seq_len]. */
int orc_build_block_diffusion_mask(const blt_block_diffusion_config *config, float *out);

/* csrc/ops/patch_pool_cpu.c:98-112 */
int orc_patch_build_group_ids(const blt_patch_info *patches, size_t num_patches, size_t seq_len,
                              size_t *query_group_ids_out, size_t *kv_group_ids_out);

/* csrc/ops/patch_pool_cpu.c:114-131 */
size_t orc_patch_decoder_latent_at(const blt_patch_info *patches, size_t num_patches, size_t pos);

/* csrc/ops/patch_pool_cpu.c:133-142 */
void orc_patch_expand_group_ids(const size_t *group_ids_in, size_t n, size_t k, size_t *group_ids_out);

/* ---- KV cache: layout, step masks, write-through, attend --------------- */

/* Row of the tier-1 slab that holds absolute byte position `pos` of sequence
 * `b`: tensors are [batch*max_seq_len, E] row-major (kv_cache.c:56-60), row
 * index == absolute position (kv_cache.h:17-18). */
size_t orc_kv_row(size_t b, size_t pos, size_t max_seq_len);

/* Element offset of (b, pos, head, d) in a tier-1 tensor. */
size_t orc_kv_slot(size_t b, size_t pos, size_t head, size_t d, size_t max_seq_len, size_t embed_dim,
                   size_t head_dim);

/* Self-attention step mask, kv_cache.c:224-238: n rows, total = base + n
 * columns; allowed = j <= base+r and (window == 0 or base+r-j < window). */
void orc_kv_self_mask(float *out, size_t n, size_t base, size_t window);

/* The attention part of one decode step for one sequence, kv_cache.c:343-390
 * without the projections and RoPE: `q_rows`, `k_rows`, `v_rows` are the n new
 * rows [n, E] (K already rotated).  K/V rows are written through to slab rows
 * [base, base+n) of sequence `b` FIRST, then every head attends over rows
 * [0, base+n) with the dense step mask, weights_out == NULL and a scratch
 * score buffer.  `combined` [n, E] is zeroed and then filled head by head.
 * Scratch buffers are allocated inside.  Returns ORC_ERR_CAPACITY when
 * base + n exceeds max_seq_len. */
int orc_kv_attend_step(float *self_k, float *self_v, size_t max_seq_len, size_t embed_dim, size_t num_heads,
                       size_t b, size_t base, size_t n, size_t window, const float *q_rows,
                       const float *k_rows, const float *v_rows, float *combined);

/* RoPE tables, reductions_cpu.c:179-197: cos_out / sin_out are [max_seq_len, head_dim/2]. */
int orc_rope_precompute(size_t max_seq_len, float theta, size_t head_dim, float *cos_out, float *sin_out);

/* reductions_cpu.c:199-229: rotate pairs (2i, 2i+1) of every head of row t by
 * the angle in cos/sin row t.  x and out are [seq_len, num_heads, head_dim]. */
void orc_rope_apply(const float *x, size_t seq_len, size_t num_heads, size_t head_dim, const float *cos_rows,
                    const float *sin_rows, float *out);

/* rope_gather.c:5-35: out row i = cache row positions[i]; ORC_ERR_ARG when a position is past the cache. */
int orc_rope_position_gather(const float *cos_cache, const float *sin_cache, size_t cache_rows, size_t half,
                             const size_t *positions, size_t n, float *cos_out, float *sin_out);

/* One decode step for one sequence including the rotation, kv_cache.c:262-271
 * and 343-390: the n new Q/K/V rows arrive un-rotated with their own row
 * strides (slices of the packed QKV rows); Q and K are rotated per head at
 * positions base..base+n-1, rotated K and V are written through, then the
 * heads attend as in orc_kv_attend_step. */
int orc_kv_rope_attend_step(float *self_k, float *self_v, size_t max_seq_len, size_t embed_dim, size_t num_heads,
                            size_t b, size_t base, size_t n, size_t window, const float *q_rows, size_t q_stride,
                            const float *k_rows, size_t k_stride, const float *v_rows, size_t v_stride,
                            const float *cos_cache, const float *sin_cache, size_t cache_rows, float *combined);

/* linalg_cpu.c:8-18: out[m,n] = a[m,k] * b[k,n], k ascending, product and sum rounded separately. */
void orc_matmul(const float *a, const float *b, float *out, size_t m, size_t k, size_t n);

/* backend.c:331-344: rotation in place of one head's column block of packed rows. */
void orc_rope_apply_packed(float *qkv, size_t qkv_stride, size_t head_offset, size_t seq_len, size_t head_dim,
                           const float *cos_rows, const float *sin_rows);

/* models/attention.c:130-207 with host buffers: input [T,E], weight_qkv
 * [E,3E], weight_proj [E,E], output [T,E].  Tables are computed inside when
 * use_rope is set and no caches are given.  mask_config (or NULL) as in
 * blt_attention_config. */
int orc_multihead_attention(const float *input, const float *weight_qkv, const float *weight_proj, float *output,
                            size_t seq_len, size_t embed_dim, size_t num_heads, int is_causal, int use_rope,
                            float rope_theta, const float *rope_cos_cache, const float *rope_sin_cache,
                            const blt_mask_config *mask_config);

/* models/cross_attention.c:101-157 with host buffers: query_in [P,E], kv_in
 * [T,E], four [E,E] weights, output [P,E]; mask_config is required. */
int orc_cross_attention_forward(const float *query_in, const float *kv_in, const float *wq, const float *wk,
                                const float *wv, const float *wproj, float *output, size_t num_patches,
                                size_t seq_len, size_t embed_dim, size_t num_heads,
                                const blt_mask_config *mask_config);

/* reductions_cpu.c:325-352 (eps 1e-6), elementwise_cpu.c:9-18 and 86-99. */
void orc_rmsnorm_forward(const float *x, const float *weight, float *out, size_t rows, size_t dim);
void orc_add(const float *a, const float *b, float *out, size_t n);
void orc_swiglu_forward(const float *gate, const float *up, float *out, size_t n);

/* One decoder layer of kv_cache.c:326-414 for the n new rows of sequence b
 * (self-attention block with rotation and write-through, feed-forward block;
 * no cross-attention).  Weights are row-major [in, out]. */
int orc_kv_decode_layer(float *self_k, float *self_v, size_t max_seq_len, size_t embed_dim, size_t num_heads,
                        size_t b, size_t base, size_t n, size_t window, const float *norm1_w, const float *qkv_w,
                        const float *proj_w, const float *norm2_w, const float *up_w, const float *gate_w,
                        const float *down_w, size_t hidden, const float *cos_cache, const float *sin_cache,
                        size_t cache_rows, const float *rows_in, float *rows_out);

/* models/local_common.c:49-64 */
int orc_local_cross_attn_fires(int placement, int cross_attn_all_layers, size_t num_layers, size_t layer);

/* infer/kv_cache.c:112-159 for sequence b of a host cache: K / V of the
 * sub-tokens of patches [from_patch, num_patches) into the tier-2 slabs of
 * every layer whose cross block fires.  patch_in is [num_patches*k, E]. */
int orc_kv_cache_refresh_cross(blt_kv_cache *cache, size_t b, const float *patch_in, size_t num_patches,
                               size_t from_patch);

/* infer/kv_cache.c:303-341 (mask 240-251): the cross block of a decoder layer
 * for the n new rows of sequence b; q_group[r] is the latent patch of row r,
 * sub-token j belongs to patch j / k_split. */
int orc_kv_cross_block(const float *cross_k, const float *cross_v, size_t max_subtokens, size_t E, size_t heads,
                       size_t b, size_t total_sub, size_t k_split, const size_t *q_group, size_t n,
                       const float *norm_w, const float *wq, const float *wproj, const float *rows_in,
                       float *rows_out);

/* infer/kv_cache.c:161-416: the whole incremental decoder step for the n new
 * rows of sequence b (valid length `base`) of a host cache, LM head included.
 * Does not advance any length. */
int orc_kv_decode_step(blt_kv_cache *cache, size_t b, size_t base, const blt_patch_info *patches,
                       size_t num_patches, const float *d0_rows, size_t n, int trailing_closed,
                       float *logits_out);

/* The KV step statements with the step kind (block_kind != 0: every new row sees all keys, the
 * INFER rule of ops/mask_builder_cpu.c:133-135) and optional rotary positions of the new rows. */
int orc_kv_attend_step_kind(float *self_k, float *self_v, size_t max_seq_len, size_t E, size_t H, size_t b,
                            size_t base, size_t n, size_t window, int block_kind, const float *q_rows,
                            const float *k_rows, const float *v_rows, float *combined);
int orc_kv_rope_attend_step_kind(float *self_k, float *self_v, size_t max_seq_len, size_t E, size_t H, size_t b,
                                 size_t base, size_t n, size_t window, int block_kind, const size_t *row_positions,
                                 const float *q_rows, size_t q_stride, const float *k_rows, size_t k_stride,
                                 const float *v_rows, size_t v_stride, const float *cos_cache,
                                 const float *sin_cache, size_t cache_rows, float *combined);
int orc_kv_decode_layer_kind(float *self_k, float *self_v, size_t max_seq_len, size_t E, size_t H, size_t b,
                             size_t base, size_t n, size_t window, int block_kind, const size_t *row_positions,
                             const float *norm1_w, const float *qkv_w, const float *proj_w, const float *norm2_w,
                             const float *up_w, const float *gate_w, const float *down_w, size_t hidden,
                             const float *cos_cache, const float *sin_cache, size_t cache_rows, const float *rows_in,
                             float *rows_out);

/* models/block_diffusion.c:776-795 (context 110-204, self-attention 246-323, layers 336-398): the
 * inference-mode diffusion forward over [clean prefix ; block rows], all rows densely.
 * byte_hidden [num_clean, E], patch_in [num_patches, patch_dim], logits_out [S, vocab]. */
int orc_local_decoder_forward_diffusion_infer(const blt_local_decoder *dec, const float *byte_hidden,
                                              const float *patch_in, const blt_patch_info *patches,
                                              size_t num_patches, const blt_block_batch *batch, int d0_mode,
                                              float *logits_out);

/* The block rows of that forward over a host cache holding the clean prefix of sequence b (`base`
 * = num_clean rows, tier 2 refreshed); logits_out [n_block_rows, vocab]; nothing is committed. */
int orc_kv_block_step(blt_kv_cache *cache, size_t b, size_t base, size_t num_patches, const blt_block_batch *batch,
                      int d0_mode, float *logits_out);

/* models/local_decoder.c:233-351 without D_0 options and without the loss: logits [seq_len, vocab]. */
int orc_local_decoder_forward(const blt_local_decoder *dec, const float *byte_hidden, size_t seq_len,
                              const float *patch_in, const blt_patch_info *patches, size_t num_patches,
                              const size_t *doc_boundaries, size_t num_docs, int trailing_closed, float *logits_out);

/* models/transformer.c:97-128, RMSNorm + SwiGLU block */
int orc_transformer_forward(const float *input, const float *norm1_w, const float *qkv_w, const float *proj_w,
                            const float *norm2_w, const float *up_w, const float *gate_w, const float *down_w,
                            float *output, size_t seq_len, size_t embed_dim, size_t hidden_dim, size_t num_heads,
                            int is_causal, int use_rope, float rope_theta, const float *rope_cos_cache,
                            const float *rope_sin_cache, const blt_mask_config *mask_config);

/* ops/gather_scatter_cpu.c:41-61: io[i, :] += table[idx[i], :], BLT_IDX_SENTINEL entries skipped. */
int orc_indexed_row_accumulate(const float *table, size_t vocab, const uint32_t *idx, float *io, size_t rows,
                               size_t embed_dim);
/* ops/elementwise_cpu.c:31-40 */
void orc_scale(float *x, size_t n, float scalar);
/* ops/patch_pool_cpu.c:3-48: pool_type 0 = mean, 1 = per-column maximum. */
int orc_patch_pool_forward(const float *byte_hidden, size_t seq_len, size_t embed_dim, const blt_patch_info *patches,
                           size_t num_patches, int pool_type, float *out);
/* models/hash_ngram.c:16-79, 176-191: the bucket index of every position for n-gram size n (rolling
 * polynomial hash with the circular window); BLT_IDX_SENTINEL before the first full window. */
int orc_ngram_indices(const uint8_t *bytes, size_t seq_len, size_t n, uint64_t prime, uint64_t modulus,
                      uint32_t *idx);
/* models/hash_ngram.c:142-207 on top of models/byte_embedding.c:16-53: out = byte_table[bytes] +
 * sum of the hashed tables (in order), scaled by 1 / (num_ngram_sizes + 1) when normalize is set. */
int orc_embed_bytes(const float *byte_table, const blt_hash_ngram_config *config,
                    const blt_hash_ngram_weights *weights, const uint8_t *bytes, size_t seq_len, float *out);
/* models/local_encoder.c:193-281 with host tensors in `enc` (context 52-113): patch_out
 * [num_patches, patch_dim], byte_hidden_out [seq_len, embed_dim]. */
int orc_local_encoder_forward(const blt_local_encoder *enc, const uint8_t *bytes, size_t seq_len,
                              const blt_patch_info *patches, size_t num_patches, const size_t *doc_boundaries,
                              size_t num_docs, float *patch_out, float *byte_hidden_out);

#ifdef __cplusplus
}
#endif

#endif /* FBLT_AMD_ORACLE_H */
