/*
 * Boundary types of the fBLT tensor-op C API, restated for the HIP attention
 * backend.  Each struct is laid out exactly as the reference's own header lays
 * it out (LP64), so a pointer handed over by the reference's C inference code
 * can be read here without a copy or a conversion.  The static assertions at
 * the end of this file are the contract: they hold for the reference compiled
 * with gcc on x86-64 Linux.
 *
 * Reference definitions mirrored here:
 *   blt_backend, blt_tensor            csrc/core/tensor.h:13-32
 *   blt_dtype                          csrc/core/dtype.h:11-17
 *   blt_arena                          csrc/core/allocator.h:11-16
 *   blt_attention_head_args            csrc/ops/attn_core.h:25-44
 *   blt_mask_config                    csrc/ops/mask_builder.h:12-32
 *   blt_block_diffusion_mode/_config   csrc/ops/mask_builder.h:43-68
 *   blt_patch_info                     csrc/models/patcher.h:16-20
 */
#ifndef FBLT_AMD_BLT_ABI_H
#define FBLT_AMD_BLT_ABI_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- backend selector ------------------------------------------------- */
/* The reference enumerates CPU=0 and one device slot (=1).  This backend
 * owns the device slot: every pointer tagged BLT_BACKEND_HIP is HIP device
 * memory of the current device. */
typedef enum {
    BLT_BACKEND_CPU = 0,
    BLT_BACKEND_HIP = 1
} blt_backend;

typedef enum {
    BLT_DTYPE_FP32 = 0,
    BLT_DTYPE_BF16 = 1,
    BLT_DTYPE_INT32 = 2,
    BLT_DTYPE_UINT8 = 3,
    BLT_DTYPE_FP8_E4M3 = 4
} blt_dtype;

#define BLT_MAX_NDIM 4

/* ---- tensor descriptor (104 bytes) ------------------------------------ */
typedef struct {
    void *data;
    size_t shape[BLT_MAX_NDIM];
    size_t strides[BLT_MAX_NDIM]; /* in elements, row-major */
    size_t ndim;
    size_t numel;
    blt_dtype dtype;
    blt_backend backend;
    bool is_view;
} blt_tensor;

/* ---- bump arena (32 bytes) -------------------------------------------- */
/* The caller owns the arena and rewinds it by assigning `offset`. */
typedef struct {
    void *buffer;
    size_t capacity;
    size_t offset;
    blt_backend backend;
} blt_arena;

/* ---- one (sequence, head) attention problem (136 bytes) ---------------- */
/* Row strides are in float elements.  `combined` receives head_dim columns
 * starting at combined_col_offset of every query row; all other columns are
 * left alone.  `mask`, when given, is a dense additive [nq, nk] matrix with
 * row stride nk and wins over is_causal. */
typedef struct {
    const float *q;
    size_t q_stride;
    const float *k;
    size_t k_stride;
    const float *v;
    size_t v_stride;
    float *combined;
    size_t combined_stride;
    size_t combined_col_offset;
    float *weights_out;    /* optional [nq*nk]: post-softmax weights            */
    float *lse_out;        /* optional [nq*2]:  (row max, sum of exponentials)  */
    float *scores_scratch; /* optional [nq*nk] workspace; never read or written */
    const float *mask;     /* optional [nq*nk] additive mask                    */
    size_t nq;
    size_t nk;
    size_t head_dim;
    bool is_causal;
    float scale;
} blt_attention_head_args;

/* ---- dense mask recipe (72 bytes) -------------------------------------- */
/* All index arrays are HOST pointers, also when the mask itself is built in
 * device memory. */
typedef struct {
    size_t seq_len_q;
    size_t seq_len_kv;
    size_t sliding_window;        /* 0 = no window                              */
    const size_t *doc_boundaries; /* entry d = first position of document d+1   */
    size_t num_docs;              /* array holds num_docs-1 entries             */
    const size_t *query_group_ids;
    const size_t *kv_group_ids;
    bool bidirectional_within_group;
    bool is_causal;
    size_t causal_offset;         /* causal rows may see keys j <= i + offset   */
} blt_mask_config;

typedef enum {
    BLT_BDM_TRAIN = 0,
    BLT_BDM_INFER = 1
} blt_block_diffusion_mode;

/* ---- BLT-D block mask recipe (48 bytes) -------------------------------- */
typedef struct {
    blt_block_diffusion_mode mode;
    size_t seq_len;   /* S: square mask                                         */
    size_t num_clean; /* N: rows/cols [0, N) are the clean prefix               */
    size_t block_size;
    const size_t *block_starts; /* TRAIN only, HOST pointer, num_blocks entries */
    size_t num_blocks;
} blt_block_diffusion_config;

/* ---- patch boundary record (24 bytes) ---------------------------------- */
typedef struct {
    size_t start_idx;
    size_t length;
    float peak_entropy;
} blt_patch_info;

/* ---- rotary embedding recipe (16 bytes), csrc/ops/rope.h:10-13 ---------- */
typedef struct {
    float theta;     /* 500000.0f in BLT */
    size_t head_dim; /* even */
} blt_rope_config;

/* ---- multi-head attention block (56 bytes), csrc/models/attention.h:12-22 */
typedef struct {
    size_t embed_dim;
    size_t num_heads;
    size_t head_dim; /* 0 = embed_dim / num_heads */
    bool is_causal;
    bool use_rope;
    float rope_theta;
    const blt_tensor *rope_cos_cache;   /* optional [seq_len, head_dim/2] */
    const blt_tensor *rope_sin_cache;
    const blt_mask_config *mask_config; /* overrides is_causal when non-NULL */
} blt_attention_config;

/* ---- cross-attention block (48 + 32 bytes), csrc/models/cross_attention.h:21-41 */
typedef enum {
    BLT_CROSS_ATTN_NO_SPLIT = 0,
    BLT_CROSS_ATTN_SPLIT_QUERY,
    BLT_CROSS_ATTN_SPLIT_KV
} blt_cross_attention_split_mode;

typedef struct {
    size_t embed_dim;
    size_t patch_dim;                          /* carried for the callers; the forward pass does not read it */
    blt_cross_attention_split_mode split_mode; /* likewise */
    size_t num_heads;
    size_t head_dim;                           /* 0 = embed_dim / num_heads */
    const blt_mask_config *mask_config;        /* required: block-diagonal patch mask */
} blt_cross_attention_config;

typedef struct {
    const blt_tensor *weight_q;    /* [embed_dim, embed_dim] each */
    const blt_tensor *weight_k;
    const blt_tensor *weight_v;
    const blt_tensor *weight_proj;
} blt_cross_attention_weights;

/* ---- learned weights of one transformer block (72 bytes), ------------- */
/* csrc/models/transformer.h:42-52                                          */
typedef struct {
    const blt_tensor *norm1_weight;
    const blt_tensor *norm1_bias; /* NULL for RMSNorm blocks */
    const blt_tensor *attn_qkv_w;
    const blt_tensor *attn_proj_w;
    const blt_tensor *norm2_weight;
    const blt_tensor *norm2_bias; /* NULL for RMSNorm blocks */
    const blt_tensor *ffn_up_w;
    const blt_tensor *ffn_gate_w; /* SwiGLU blocks */
    const blt_tensor *ffn_down_w;
} blt_transformer_weights;

/* ---- local decoder and its two-tier KV cache ---------------------------- */
/* csrc/models/local_common.h:21-35, 58-64; csrc/models/local_decoder.h:17-30,
 * 60-72; csrc/infer/kv_cache.h:45-65.  Only the inference-side members are
 * listed by name in comments; the layouts are complete.                     */
typedef enum {
    BLT_XATTN_DEFAULT = 0, /* cross_attn_all_layers decides: all layers, or the last one only */
    BLT_XATTN_NONE,
    BLT_XATTN_LAST,
    BLT_XATTN_ALL,
    BLT_XATTN_FIRST
} blt_xattn_placement;

typedef struct {
    blt_tensor norm1_weight;      /* [E]        */
    blt_tensor attn_qkv_w;        /* [E, 3E]    */
    blt_tensor attn_proj_w;       /* [E, E]     */
    blt_tensor norm2_weight;      /* [E]        */
    blt_tensor ffn_up_w;          /* [E, hidden]*/
    blt_tensor ffn_gate_w;        /* [E, hidden]*/
    blt_tensor ffn_down_w;        /* [hidden, E]*/
    blt_tensor cross_norm_weight; /* [E]; the cross block comes first in a decoder layer */
    blt_tensor cross_weight_q;    /* [E, E]     */
    blt_tensor cross_weight_k;
    blt_tensor cross_weight_v;
    blt_tensor cross_weight_proj;
} blt_local_layer_storage;

typedef struct {
    size_t embed_dim;
    size_t patch_dim; /* 0 = embed_dim; a multiple k of embed_dim splits every patch into k sub-tokens */
    size_t num_layers;
    size_t hidden_dim;
    size_t num_heads;
    size_t cross_attn_heads;
    size_t local_window; /* 0 = full causal */
    bool cross_attn_all_layers;
    blt_xattn_placement cross_attn_placement;
    float rope_theta;
    size_t max_seq_len;
    size_t vocab_size;
} blt_local_decoder_config;

typedef struct {
    blt_local_decoder_config config;
    blt_tensor rope_cos_cache, rope_sin_cache; /* [max_seq_len, head_dim/2] */
    blt_local_layer_storage *layers;           /* [num_layers] */
    blt_tensor lm_head_weight;                 /* [embed_dim, vocab_size] */
    blt_tensor d0_embed_weight;                /* [257, embed_dim]; not read by the decode step */
} blt_local_decoder;

typedef struct {
    const blt_local_decoder *decoder;
    size_t max_seq_len;
    size_t batch_size;
    size_t max_subtokens; /* = max_seq_len */
    size_t embed_dim;
    size_t k;             /* patch_dim / embed_dim */
    size_t patch_dim;
    blt_tensor *self_k;   /* [num_layers] x [batch_size*max_seq_len, embed_dim]: row b*max_seq_len + pos */
    blt_tensor *self_v;
    size_t self_len;      /* valid byte positions of the single-sequence cache */
    blt_tensor *cross_k;  /* [num_layers] x [batch_size*max_subtokens, embed_dim] */
    blt_tensor *cross_v;
    size_t cross_num_patches;
    blt_patch_info *cached_patches; /* [batch_size*max_seq_len] boundary snapshot */
} blt_kv_cache;

/* csrc/models/transformer.h:15-38 */
typedef enum {
    BLT_NORM_LAYERNORM = 0,
    BLT_NORM_RMSNORM = 1
} blt_norm_type;

typedef enum {
    BLT_ACTIVATION_GELU = 0,
    BLT_ACTIVATION_SWIGLU = 1
} blt_activation_type;

typedef struct {
    blt_attention_config attn_config;
    size_t hidden_dim;
    float layer_norm_eps;
    blt_norm_type norm_type;
    blt_activation_type activation_type;
    int use_bf16;
} blt_transformer_config;

/* csrc/models/local_decoder.h:42-46 */
typedef enum {
    BLT_D0_HFINAL = 0, /* every row of byte_hidden_in is a real encoder state */
    BLT_D0_ZEROS,      /* block rows start from zero vectors */
    BLT_D0_LEARNED     /* block rows read d0_embed_weight[token] */
} blt_d0_mode;

/* csrc/models/local_decoder.h:48-54 */
typedef struct {
    blt_d0_mode d0_mode;
    size_t num_hfinal_rows;
    const uint32_t *d0_extra_tokens;
} blt_local_decoder_d0_opts;

#define BLT_MASK_TOKEN_ID 256u /* csrc/models/block_diffusion.h:32 */

/* csrc/models/block_diffusion.h:37-86: the block section behind a clean prefix.  The inference
 * forward reads num_clean, n_block_rows, block_size, num_blocks, tokens, positions, groups and
 * trailing_closed; the rest belongs to the training loss. */
typedef struct {
    size_t num_clean;
    size_t block_size;
    size_t num_blocks;
    size_t n_block_rows;
    float t;
    uint32_t *tokens;     /* [n_block_rows] byte value or BLT_MASK_TOKEN_ID */
    size_t *positions;    /* [n_block_rows] byte position of every block row (rotary tables) */
    uint8_t *targets;
    uint8_t *cell_valid;
    uint8_t *cell_masked;
    size_t *groups;       /* [n_block_rows] latent patch the row cross-attends */
    float loss_scale;
    float last_row_scale;
    int clean_sum;
    int mask_norm;
    int trailing_closed;  /* the last clean byte closes its patch and reads the last latent */
} blt_block_batch;

/* csrc/ops/patch_pool.h:13-16 */
typedef enum {
    BLT_POOL_MEAN = 0, /* average of the patch's byte rows       */
    BLT_POOL_MAX = 1   /* per-column maximum of the patch's rows */
} blt_patch_pool_type;

#define BLT_IDX_SENTINEL 0xFFFFFFFFu /* csrc/ops/gather_scatter.h:27: "no row" in an index list */

/* csrc/models/hash_ngram.h:13-27 */
#define BLT_MAX_NGRAM_SIZES 6
typedef struct {
    size_t ngram_sizes[BLT_MAX_NGRAM_SIZES];
    size_t num_ngram_sizes;
    size_t per_ngram_vocab; /* rows of every table = modulus of the rolling hash */
    uint64_t hash_prime;
    bool normalize;         /* divide the sum by num_ngram_sizes + 1 */
    size_t embed_dim;
} blt_hash_ngram_config;

typedef struct {
    blt_tensor tables[BLT_MAX_NGRAM_SIZES]; /* each [per_ngram_vocab, embed_dim] */
    size_t num_tables;
} blt_hash_ngram_weights;

/* csrc/models/local_encoder.h:22-48 */
typedef struct {
    size_t embed_dim;
    size_t num_layers;
    size_t patch_dim; /* 0 = embed_dim */
    size_t hidden_dim;
    size_t num_heads;
    size_t cross_attn_heads;
    size_t local_window; /* 0 = full causal */
    bool cross_attn_all_layers;
    blt_xattn_placement cross_attn_placement;
    blt_patch_pool_type pool_type;
    blt_hash_ngram_config ngram_config;
    float rope_theta;
    size_t max_seq_len;
} blt_local_encoder_config;

typedef struct {
    blt_local_encoder_config config;
    blt_tensor byte_embedding_weight; /* [256, embed_dim] */
    blt_hash_ngram_weights ngram_weights;
    blt_tensor rope_cos_cache, rope_sin_cache; /* [max_seq_len, head_dim/2] */
    blt_local_layer_storage *layers;           /* [num_layers] */
} blt_local_encoder;

#ifdef __cplusplus
}
#define BLT_ABI_ASSERT(c, m) static_assert(c, m)
#else
#define BLT_ABI_ASSERT(c, m) _Static_assert(c, m)
#endif

BLT_ABI_ASSERT(sizeof(size_t) == 8 && sizeof(void *) == 8, "LP64 only");
BLT_ABI_ASSERT(sizeof(blt_tensor) == 104, "blt_tensor layout");
BLT_ABI_ASSERT(offsetof(blt_tensor, dtype) == 88 && offsetof(blt_tensor, is_view) == 96, "blt_tensor tail");
BLT_ABI_ASSERT(sizeof(blt_arena) == 32, "blt_arena layout");
BLT_ABI_ASSERT(sizeof(blt_attention_head_args) == 136, "blt_attention_head_args layout");
BLT_ABI_ASSERT(offsetof(blt_attention_head_args, mask) == 96, "blt_attention_head_args.mask");
BLT_ABI_ASSERT(offsetof(blt_attention_head_args, is_causal) == 128 &&
                   offsetof(blt_attention_head_args, scale) == 132,
               "blt_attention_head_args tail");
BLT_ABI_ASSERT(sizeof(blt_mask_config) == 72, "blt_mask_config layout");
BLT_ABI_ASSERT(sizeof(blt_transformer_weights) == 72, "blt_transformer_weights layout");
BLT_ABI_ASSERT(sizeof(blt_cross_attention_config) == 48 && offsetof(blt_cross_attention_config, num_heads) == 24,
               "blt_cross_attention_config layout");
BLT_ABI_ASSERT(sizeof(blt_cross_attention_weights) == 32, "blt_cross_attention_weights layout");
BLT_ABI_ASSERT(sizeof(blt_rope_config) == 16 && offsetof(blt_rope_config, head_dim) == 8, "blt_rope_config layout");
BLT_ABI_ASSERT(sizeof(blt_attention_config) == 56 && offsetof(blt_attention_config, rope_theta) == 28 &&
                   offsetof(blt_attention_config, mask_config) == 48,
               "blt_attention_config layout");
BLT_ABI_ASSERT(offsetof(blt_mask_config, bidirectional_within_group) == 56 &&
                   offsetof(blt_mask_config, is_causal) == 57 && offsetof(blt_mask_config, causal_offset) == 64,
               "blt_mask_config tail");
BLT_ABI_ASSERT(sizeof(blt_block_diffusion_config) == 48, "blt_block_diffusion_config layout");
BLT_ABI_ASSERT(sizeof(blt_patch_info) == 24, "blt_patch_info layout");
BLT_ABI_ASSERT(sizeof(blt_local_layer_storage) == 12 * 104, "blt_local_layer_storage layout");
BLT_ABI_ASSERT(sizeof(blt_local_decoder_config) == 88 && offsetof(blt_local_decoder_config, cross_attn_placement) == 60 &&
                   offsetof(blt_local_decoder_config, rope_theta) == 64 &&
                   offsetof(blt_local_decoder_config, max_seq_len) == 72,
               "blt_local_decoder_config layout");
BLT_ABI_ASSERT(sizeof(blt_local_decoder) == 512 && offsetof(blt_local_decoder, layers) == 296 &&
                   offsetof(blt_local_decoder, lm_head_weight) == 304,
               "blt_local_decoder layout");
BLT_ABI_ASSERT(sizeof(blt_kv_cache) == 112 && offsetof(blt_kv_cache, self_len) == 72 &&
                   offsetof(blt_kv_cache, cached_patches) == 104,
               "blt_kv_cache layout");

BLT_ABI_ASSERT(sizeof(blt_transformer_config) == 80 && offsetof(blt_transformer_config, hidden_dim) == 56 &&
                   offsetof(blt_transformer_config, norm_type) == 68 && offsetof(blt_transformer_config, use_bf16) == 76,
               "blt_transformer_config layout");
BLT_ABI_ASSERT(sizeof(blt_hash_ngram_config) == 88 && offsetof(blt_hash_ngram_config, hash_prime) == 64 &&
                   sizeof(blt_hash_ngram_weights) == 632 && offsetof(blt_hash_ngram_weights, num_tables) == 624,
               "blt_hash_ngram_config / _weights layout");
BLT_ABI_ASSERT(sizeof(blt_local_encoder_config) == 176 && offsetof(blt_local_encoder_config, pool_type) == 64 &&
                   offsetof(blt_local_encoder_config, ngram_config) == 72 &&
                   offsetof(blt_local_encoder_config, rope_theta) == 160,
               "blt_local_encoder_config layout");
BLT_ABI_ASSERT(sizeof(blt_local_encoder) == 1128 && offsetof(blt_local_encoder, ngram_weights) == 280 &&
                   offsetof(blt_local_encoder, rope_cos_cache) == 912 && offsetof(blt_local_encoder, layers) == 1120,
               "blt_local_encoder layout");
BLT_ABI_ASSERT(sizeof(blt_block_batch) == 112 && offsetof(blt_block_batch, tokens) == 40 &&
                   offsetof(blt_block_batch, groups) == 80 && offsetof(blt_block_batch, trailing_closed) == 104,
               "blt_block_batch layout");

#endif /* FBLT_AMD_BLT_ABI_H */
