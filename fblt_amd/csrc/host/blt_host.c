/*
 * Host side of the HIP attention backend, in C99 like the reference's host
 * code.  Holds the arena/tensor helpers, the run-time dispatchers with the
 * reference's public names, the byte<->patch index helpers (host integer code
 * in the reference too) and the mask-recipe -> row-range reduction.  Every
 * device action goes through the extern "C" entry points of blt_hip.h; no HIP
 * header is included here.
 */
#include "blt_hip.h"
#include "blt_fatal.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ */
/* Arena + tensors (reference behaviour: csrc/core/allocator.c:36-160) */
/* ------------------------------------------------------------------ */

static size_t dtype_bytes(blt_dtype t) {
    switch (t) {
    case BLT_DTYPE_FP32:
    case BLT_DTYPE_INT32:
        return 4;
    case BLT_DTYPE_BF16:
        return 2;
    case BLT_DTYPE_UINT8:
    case BLT_DTYPE_FP8_E4M3:
        return 1;
    }
    return 0;
}

blt_arena *blt_arena_create(size_t capacity_bytes, blt_backend backend) {
    BLT_REQUIRE(capacity_bytes > 0, "blt_arena_create: capacity must be positive");
    blt_arena *a = (blt_arena *)calloc(1, sizeof(*a));
    BLT_REQUIRE(a != NULL, "blt_arena_create: out of host memory");
    a->capacity = capacity_bytes;
    a->backend = backend;
    if (backend == BLT_BACKEND_HIP) {
        a->buffer = blt_hip_malloc(capacity_bytes);
    } else {
        void *p = NULL;
        if (posix_memalign(&p, 64, capacity_bytes) != 0) p = NULL;
        a->buffer = p;
    }
    if (!a->buffer) BLT_FATAL("failed to allocate arena buffer");
    return a;
}

/* Host blocks handed out by blt_container_alloc() for device arenas, newest first. */
typedef struct host_block {
    struct host_block *next;
    const blt_arena *arena;
    size_t at;   /* the arena's offset when the block was handed out */
    size_t seen; /* the arena's offset after the newest allocation this library saw (kept in the newest block) */
} host_block;
#define HOST_BLOCK_HEADER 64 /* keeps the payload 64-byte aligned, as arena containers are */

static host_block *g_host_blocks = NULL;
static pthread_mutex_t g_host_blocks_lock = PTHREAD_MUTEX_INITIALIZER;

/* Frees the arena's host blocks that were handed out at or above `keep_to` (all of them with
 * `all` set).  Caller holds the lock. */
static void host_blocks_release(const blt_arena *a, size_t keep_to, int all) {
    host_block **link = &g_host_blocks;
    while (*link) {
        host_block *b = *link;
        if (b->arena == a && (all || b->at >= keep_to)) {
            *link = b->next;
            free(b);
        } else {
            link = &b->next;
        }
    }
}

/* Called before every allocation from a device arena: an offset below what the last allocation
 * left behind means the caller has rewound the arena since, and the blocks handed out at or above
 * the new offset are dead, as their arena-resident twins of the CPU backend would be.  Then notes
 * where this allocation will leave the offset.  Costs a pointer comparison while the arena has no
 * blocks. */
static void host_blocks_sweep(const blt_arena *a, size_t offset_after) {
    if (!g_host_blocks) return; /* racy peek: a block list that is empty needs no sweep */
    pthread_mutex_lock(&g_host_blocks_lock);
    host_block *newest = g_host_blocks;
    while (newest && newest->arena != a) newest = newest->next;
    if (newest) {
        if (a->offset < newest->seen) {
            host_blocks_release(a, a->offset, 0);
            newest = g_host_blocks;
            while (newest && newest->arena != a) newest = newest->next;
        }
        if (newest) newest->seen = offset_after;
    }
    pthread_mutex_unlock(&g_host_blocks_lock);
}

void blt_arena_destroy(blt_arena *a) {
    if (!a) return;
    if (a->backend == BLT_BACKEND_HIP) {
        pthread_mutex_lock(&g_host_blocks_lock);
        host_blocks_release(a, 0, 1);
        pthread_mutex_unlock(&g_host_blocks_lock);
        blt_hip_free(a->buffer);
    } else {
        free(a->buffer);
    }
    free(a);
}

void blt_arena_reset(blt_arena *a) {
    if (!a) return;
    a->offset = 0;
    if (a->backend == BLT_BACKEND_HIP) {
        pthread_mutex_lock(&g_host_blocks_lock);
        host_blocks_release(a, 0, 1);
        pthread_mutex_unlock(&g_host_blocks_lock);
    }
}

void *blt_arena_alloc(blt_arena *a, size_t bytes, size_t alignment) {
    if (!a || !a->buffer) BLT_FATAL("invalid arena");
    if (alignment == 0) alignment = 1;
    const size_t at = (a->offset + (alignment - 1)) & ~(alignment - 1);
    if (at + bytes > a->capacity)
        BLT_FATAL("arena allocation exceeded capacity: need %zu (aligned %zu), offset %zu, capacity %zu", bytes, at,
                  a->offset, a->capacity);
    if (a->backend == BLT_BACKEND_HIP) host_blocks_sweep(a, at + bytes);
    a->offset = at + bytes;
    return (char *)a->buffer + at;
}

/* Containers are what callers fill and read on the host: group-id arrays, weight-view structs,
 * model structs (csrc/models/local_decoder.c:76-80, transformer_stack.c:85).  On the CPU backend
 * they live in the arena (csrc/core/tensor.c:154); for a device arena the reference hands out
 * zeroed host memory instead (tensor.c:156-162, backend.c:494-501) and never releases it.  Here a
 * block belongs to its arena and takes ONE BYTE of it as a token, which gives the block a place
 * in the arena's order (a run of containers costs the arena at most the 63 bytes the next
 * tensor's alignment would have skipped anyway): the block is released when the arena is reset
 * or destroyed, or at the first allocation after the caller has rewound the arena's offset to or
 * below its token (csrc/infer/self_speculation.c:359-401 rewinds that way), which is when a
 * container of the CPU backend would be dead too.  Every allocation from the arena looks for
 * such a rewind, so a loop that rewinds to a marker every round holds one round's blocks at
 * most, whether its first allocation of a round is a container or a tensor. */
void *blt_container_alloc(blt_arena *a, size_t bytes) {
    if (!a || !a->buffer) BLT_FATAL("invalid arena");
    if (a->backend != BLT_BACKEND_HIP) return blt_arena_alloc(a, bytes, 64);
    BLT_REQUIRE(bytes <= (size_t)-1 - HOST_BLOCK_HEADER, "blt_container_alloc: size overflows");
    void *raw = NULL;
    if (posix_memalign(&raw, 64, HOST_BLOCK_HEADER + bytes) != 0) raw = NULL;
    BLT_REQUIRE(raw != NULL, "blt_container_alloc: host allocation failed");
    host_block *b = (host_block *)raw;
    memset(b, 0, HOST_BLOCK_HEADER + bytes);
    b->arena = a;
    (void)blt_arena_alloc(a, 1, 1); /* the token; sweeps the blocks a rewind has killed */
    b->at = a->offset - 1;
    b->seen = a->offset;
    pthread_mutex_lock(&g_host_blocks_lock);
    b->next = g_host_blocks;
    g_host_blocks = b;
    pthread_mutex_unlock(&g_host_blocks_lock);
    return (char *)b + HOST_BLOCK_HEADER;
}

static blt_tensor tensor_make(blt_arena *arena, const size_t *shape, size_t ndim, blt_dtype dtype, int clear) {
    BLT_REQUIRE(ndim <= BLT_MAX_NDIM, "blt_tensor_create: ndim exceeds BLT_MAX_NDIM");
    blt_tensor t;
    memset(&t, 0, sizeof(t));
    t.dtype = dtype;
    t.backend = arena ? arena->backend : BLT_BACKEND_CPU;
    t.ndim = ndim;
    t.numel = ndim ? 1 : 0;
    for (size_t d = 0; d < ndim; d++) {
        t.shape[d] = shape[d];
        t.numel *= shape[d];
    }
    size_t run = 1;
    for (size_t d = ndim; d-- > 0;) {
        t.strides[d] = run;
        run *= shape[d];
    }
    const size_t bytes = t.numel * dtype_bytes(dtype);
    t.data = blt_arena_alloc(arena, bytes, 64);
    if (clear && bytes) {
        if (t.backend == BLT_BACKEND_HIP) blt_hip_memset(t.data, 0, bytes);
        else memset(t.data, 0, bytes);
    }
    return t;
}

blt_tensor blt_tensor_create(blt_arena *arena, const size_t *shape, size_t ndim, blt_dtype dtype) {
    return tensor_make(arena, shape, ndim, dtype, 1);
}

blt_tensor blt_tensor_create_uninit(blt_arena *arena, const size_t *shape, size_t ndim, blt_dtype dtype) {
    return tensor_make(arena, shape, ndim, dtype, 0);
}

void blt_tensor_upload(blt_tensor *dst, const void *host_src, size_t bytes) {
    BLT_REQUIRE(dst != NULL && dst->data != NULL && host_src != NULL, "blt_tensor_upload: NULL argument");
    if (dst->backend == BLT_BACKEND_HIP) blt_hip_memcpy_h2d(dst->data, host_src, bytes);
    else memcpy(dst->data, host_src, bytes);
}

void blt_tensor_download(const blt_tensor *src, void *host_dst, size_t bytes) {
    BLT_REQUIRE(src != NULL && src->data != NULL && host_dst != NULL, "blt_tensor_download: NULL argument");
    if (src->backend == BLT_BACKEND_HIP) blt_hip_memcpy_d2h(host_dst, src->data, bytes);
    else memcpy(host_dst, src->data, bytes);
}

void blt_backend_pass_sync(blt_backend backend) {
    if (backend == BLT_BACKEND_HIP) blt_backend_pass_sync_hip();
}

/* ------------------------------------------------------------------ */
/* Dispatchers (reference: csrc/core/backend.c:104-138, 455-492).       */
/* There is no CPU compute path in this library.                        */
/* ------------------------------------------------------------------ */

#define BLT_DEVICE_ONLY(backend, what)                                                                             \
    do {                                                                                                           \
        if ((backend) != BLT_BACKEND_HIP)                                                                          \
            BLT_FATAL(what ": this library implements the HIP backend only (got backend %d)", (int)(backend));     \
    } while (0)

void blt_attention_head_core(blt_backend backend, const blt_attention_head_args *args) {
    BLT_DEVICE_ONLY(backend, "blt_attention_head_core");
    blt_attention_head_core_hip(backend, args);
}

void blt_build_attention_mask(const blt_mask_config *config, blt_tensor *out_mask, blt_arena *arena) {
    BLT_DEVICE_ONLY(arena ? arena->backend : BLT_BACKEND_CPU, "blt_build_attention_mask");
    blt_build_attention_mask_hip(config, out_mask, arena);
}

void blt_build_block_diffusion_mask(const blt_block_diffusion_config *config, blt_tensor *out_mask,
                                    blt_arena *arena) {
    BLT_DEVICE_ONLY(arena ? arena->backend : BLT_BACKEND_CPU, "blt_build_block_diffusion_mask");
    blt_build_block_diffusion_mask_hip(config, out_mask, arena);
}

void blt_strided_copy(blt_backend backend, float *dst, size_t dst_stride, const float *src, size_t src_stride,
                      size_t rows, size_t cols) {
    BLT_DEVICE_ONLY(backend, "blt_strided_copy");
    blt_strided_copy_hip(backend, dst, dst_stride, src, src_stride, rows, cols);
}

void blt_rows_gather(const blt_tensor *src, const size_t *pos_host, blt_tensor *dst) {
    BLT_REQUIRE(src != NULL, "blt_rows_gather: arguments cannot be NULL");
    BLT_DEVICE_ONLY(src->backend, "blt_rows_gather");
    blt_rows_gather_hip(src, pos_host, dst);
}

void blt_embedding_lookup(const blt_tensor *table, const uint32_t *ids_host, blt_tensor *out) {
    BLT_REQUIRE(table != NULL, "blt_embedding_lookup: arguments cannot be NULL");
    BLT_DEVICE_ONLY(table->backend, "blt_embedding_lookup");
    blt_embedding_lookup_hip(table, ids_host, out);
}

void blt_rope_position_gather(const blt_tensor *cos_cache, const blt_tensor *sin_cache, const size_t *positions,
                              size_t n, blt_tensor *cos_out, blt_tensor *sin_out, blt_arena *arena) {
    BLT_REQUIRE(cos_cache != NULL && sin_cache != NULL && positions != NULL && cos_out != NULL && sin_out != NULL &&
                    arena != NULL,
                "blt_rope_position_gather: arguments cannot be NULL");
    BLT_REQUIRE(n >= 1, "blt_rope_position_gather: n must be >= 1");
    BLT_REQUIRE(cos_cache->ndim == 2 && cos_cache->dtype == BLT_DTYPE_FP32,
                "blt_rope_position_gather: cos_cache must be a 2D FP32 tensor");
    BLT_REQUIRE(sin_cache->ndim == 2 && sin_cache->dtype == BLT_DTYPE_FP32,
                "blt_rope_position_gather: sin_cache must be a 2D FP32 tensor");
    const size_t max_seq_len = cos_cache->shape[0], half = cos_cache->shape[1];
    BLT_REQUIRE(sin_cache->shape[0] == max_seq_len && sin_cache->shape[1] == half,
                "blt_rope_position_gather: cos/sin cache shape mismatch");
    for (size_t i = 0; i < n; i++)
        BLT_REQUIRE(positions[i] < max_seq_len,
                    "blt_rope_position_gather: positions[%zu]=%zu out of cache range [0, %zu)", i, positions[i],
                    max_seq_len);
    const size_t shape[2] = {n, half};
    *cos_out = blt_tensor_create_uninit(arena, shape, 2, BLT_DTYPE_FP32);
    *sin_out = blt_tensor_create_uninit(arena, shape, 2, BLT_DTYPE_FP32);
    blt_rows_gather(cos_cache, positions, cos_out);
    blt_rows_gather(sin_cache, positions, sin_out);
}

void blt_softmax_masked_row_inplace(blt_backend backend, float *row, size_t row_len, size_t row_idx, bool is_causal,
                                    const float *mask_row, float scale) {
    BLT_DEVICE_ONLY(backend, "blt_softmax_masked_row_inplace");
    blt_softmax_masked_row_inplace_hip(backend, row, row_len, row_idx, is_causal, mask_row, scale);
}

void blt_cross_attention_forward(const blt_tensor *query_in, const blt_tensor *kv_in,
                                 const blt_cross_attention_weights *weights, blt_tensor *output,
                                 const blt_cross_attention_config *config, blt_arena *arena) {
    BLT_REQUIRE(query_in != NULL, "blt_cross_attention: query_in must be [num_patches, embed_dim] FP32");
    BLT_DEVICE_ONLY(query_in->backend, "blt_cross_attention_forward");
    blt_cross_attention_forward_hip(query_in, kv_in, weights, output, config, arena);
}

/* ------------------------------------------------------------------ */
/* two-tier KV cache container (csrc/infer/kv_cache.c:27-110)          */
/* ------------------------------------------------------------------ */
/* Geometry of a cache for a decoder, checked in one place.  The struct contract
 * (include/blt_abi.h, mirroring csrc/infer/kv_cache.h:45-65): per layer four [rows, embed]
 * fp32 tensors, tier 1 with batch * max_seq_len byte rows, tier 2 with batch * max_subtokens
 * sub-token rows; a patch of patch_dim columns splits into patch_dim / embed sub-tokens. */
typedef struct {
    size_t layers;
    size_t embed;
    size_t patch_dim;
    size_t split;      /* sub-tokens per patch */
    size_t subtokens;  /* tier-2 rows per sequence */
    size_t batch;
} kv_geometry;

static kv_geometry kv_geometry_of(const blt_local_decoder *decoder, size_t max_seq_len, size_t batch_size) {
    const blt_local_decoder_config *cfg = &decoder->config;
    kv_geometry g;
    g.layers = cfg->num_layers;
    g.embed = cfg->embed_dim;
    g.patch_dim = cfg->patch_dim != 0 ? cfg->patch_dim : cfg->embed_dim;
    BLT_REQUIRE(g.embed > 0 && g.patch_dim % g.embed == 0,
                "blt_kv_cache_create: patch_dim (%zu) must be a positive multiple of embed_dim (%zu)", g.patch_dim,
                g.embed);
    BLT_REQUIRE(max_seq_len >= 2 && max_seq_len <= cfg->max_seq_len,
                "blt_kv_cache_create: max_seq_len %zu outside [2, %zu], the decoder's own limit", max_seq_len,
                cfg->max_seq_len);
    g.split = g.patch_dim / g.embed;
    g.subtokens = max_seq_len; /* every patch covers at least one byte, so tier 2 never needs more rows */
    g.batch = batch_size != 0 ? batch_size : 1;
    return g;
}

blt_kv_cache *blt_kv_cache_create_batched(blt_arena *arena, const blt_local_decoder *decoder, size_t max_seq_len,
                                          size_t batch_size) {
    BLT_REQUIRE(arena != NULL && decoder != NULL, "blt_kv_cache_create: arena and decoder cannot be NULL");
    const kv_geometry g = kv_geometry_of(decoder, max_seq_len, batch_size);
    blt_kv_cache *cache = (blt_kv_cache *)calloc(1, sizeof(*cache));
    BLT_REQUIRE(cache != NULL, "blt_kv_cache_create: out of host memory for the container");
    cache->decoder = decoder;
    cache->batch_size = g.batch;
    cache->max_seq_len = max_seq_len;
    cache->max_subtokens = g.subtokens;
    cache->embed_dim = g.embed;
    cache->patch_dim = g.patch_dim;
    cache->k = g.split;

    /* The four tiers: where the container keeps each handle array, and the rows of one layer's
     * tensor.  Each handle array is a heap block of its own (destroy releases them one by one,
     * and so does the reference's, csrc/infer/kv_cache.c:77-87); the payloads are zero-filled
     * arena tensors, placed layer by layer. */
    const struct {
        blt_tensor **handles;
        size_t rows;
    } tiers[4] = {{&cache->self_k, g.batch * max_seq_len},
                  {&cache->self_v, g.batch * max_seq_len},
                  {&cache->cross_k, g.batch * g.subtokens},
                  {&cache->cross_v, g.batch * g.subtokens}};
    for (size_t t = 0; t < 4; t++) {
        *tiers[t].handles = (blt_tensor *)calloc(g.layers != 0 ? g.layers : 1, sizeof(blt_tensor));
        BLT_REQUIRE(*tiers[t].handles != NULL, "blt_kv_cache_create: out of host memory for %zu layer handles", g.layers);
    }
    for (size_t layer = 0; layer < g.layers; layer++) {
        for (size_t t = 0; t < 4; t++) {
            const size_t shape[2] = {tiers[t].rows, g.embed};
            (*tiers[t].handles)[layer] = blt_tensor_create(arena, shape, 2, BLT_DTYPE_FP32);
        }
    }
    cache->cached_patches = (blt_patch_info *)calloc(g.batch * max_seq_len, sizeof(blt_patch_info));
    BLT_REQUIRE(cache->cached_patches != NULL, "blt_kv_cache_create: out of host memory for the patch table");
    return cache;
}

blt_kv_cache *blt_kv_cache_create(blt_arena *arena, const blt_local_decoder *decoder, size_t max_seq_len) {
    return blt_kv_cache_create_batched(arena, decoder, max_seq_len, 1);
}

void blt_kv_cache_destroy(blt_kv_cache *cache) {
    if (cache == NULL) return;
    blt_tensor *const handle_arrays[4] = {cache->self_k, cache->self_v, cache->cross_k, cache->cross_v};
    for (size_t t = 0; t < 4; t++) free(handle_arrays[t]);
    free(cache->cached_patches);
    free(cache);
}

/* Rollback is bookkeeping only: rows past the valid counts are dead by contract
 * (csrc/infer/kv_cache.c:89-99). */
void blt_kv_cache_truncate(blt_kv_cache *cache, size_t self_len, size_t num_patches) {
    BLT_REQUIRE(cache != NULL, "blt_kv_cache_truncate: cache cannot be NULL");
    BLT_REQUIRE(self_len <= cache->max_seq_len, "blt_kv_cache_truncate: %zu byte rows exceed the cache's %zu",
                self_len, cache->max_seq_len);
    BLT_REQUIRE(num_patches <= cache->max_subtokens, "blt_kv_cache_truncate: %zu patches exceed the cache's %zu",
                num_patches, cache->max_subtokens);
    cache->self_len = self_len;
    cache->cross_num_patches = num_patches;
}

void blt_kv_cache_reset(blt_kv_cache *cache) { blt_kv_cache_truncate(cache, 0, 0); }

/* Length of the common prefix of the cached patch table and a new segmentation: patches agree
 * when start and length agree (csrc/infer/kv_cache.c:101-109). */
size_t blt_kv_cache_common_patches(const blt_kv_cache *cache, const blt_patch_info *patches, size_t num_patches) {
    const size_t limit = num_patches < cache->cross_num_patches ? num_patches : cache->cross_num_patches;
    for (size_t p = 0; p < limit; p++) {
        const blt_patch_info *old = &cache->cached_patches[p];
        if (old->start_idx != patches[p].start_idx || old->length != patches[p].length) return p;
    }
    return limit;
}

bool blt_local_cross_attn_fires(blt_xattn_placement placement, bool cross_attn_all_layers, size_t num_layers,
                                size_t layer) {
    switch (placement) {
    case BLT_XATTN_NONE: return false;
    case BLT_XATTN_LAST: return layer + 1 == num_layers;
    case BLT_XATTN_ALL: return true;
    case BLT_XATTN_FIRST: return layer == 0;
    case BLT_XATTN_DEFAULT:
    default: return cross_attn_all_layers || layer + 1 == num_layers;
    }
}

void blt_kv_cache_refresh_cross(blt_kv_cache *cache, const blt_tensor *patch_in, const blt_patch_info *patches,
                                size_t num_patches, size_t from_patch, blt_arena *arena) {
    BLT_REQUIRE(patch_in != NULL, "blt_kv_cache_refresh_cross: arguments cannot be NULL");
    BLT_DEVICE_ONLY(patch_in->backend, "blt_kv_cache_refresh_cross");
    blt_kv_cache_refresh_cross_hip(cache, patch_in, patches, num_patches, from_patch, arena);
}

void blt_kv_decode_step(blt_kv_cache *cache, const blt_tensor *patch_in, const blt_patch_info *patches,
                        size_t num_patches, const blt_tensor *d0_rows, int trailing_closed, blt_tensor *logits_out,
                        blt_arena *arena) {
    BLT_REQUIRE(d0_rows != NULL, "blt_kv_decode_step: arguments cannot be NULL");
    BLT_DEVICE_ONLY(d0_rows->backend, "blt_kv_decode_step");
    blt_kv_decode_step_hip(cache, patch_in, patches, num_patches, d0_rows, trailing_closed, logits_out, arena);
}

void blt_local_decoder_forward_diffusion_infer(const blt_local_decoder *model, const blt_tensor *byte_hidden_in,
                                               const blt_tensor *patch_in, const blt_patch_info *patches,
                                               size_t num_patches, const blt_block_batch *batch, blt_d0_mode d0_mode,
                                               blt_tensor *logits_out, blt_arena *arena) {
    BLT_REQUIRE(byte_hidden_in != NULL, "forward_diffusion_infer: arguments cannot be NULL");
    BLT_DEVICE_ONLY(byte_hidden_in->backend, "blt_local_decoder_forward_diffusion_infer");
    blt_local_decoder_forward_diffusion_infer_hip(model, byte_hidden_in, patch_in, patches, num_patches, batch, d0_mode,
                                                  logits_out, arena);
}

void blt_transformer_forward(const blt_tensor *input, const blt_transformer_weights *weights, blt_tensor *output,
                             const blt_transformer_config *config, blt_arena *arena) {
    BLT_REQUIRE(input != NULL, "Transformer: input, weights, output, and config cannot be NULL");
    BLT_DEVICE_ONLY(input->backend, "blt_transformer_forward");
    blt_transformer_forward_hip(input, weights, output, config, arena);
}

void blt_indexed_row_accumulate(const blt_tensor *table, const uint32_t *idx_host, blt_tensor *io) {
    BLT_REQUIRE(table != NULL, "blt_indexed_row_accumulate: arguments cannot be NULL");
    BLT_DEVICE_ONLY(table->backend, "blt_indexed_row_accumulate");
    blt_indexed_row_accumulate_hip(table, idx_host, io);
}

void blt_scale(blt_tensor *t, float scalar) {
    BLT_REQUIRE(t != NULL, "blt_scale: tensor must not be null");
    BLT_DEVICE_ONLY(t->backend, "blt_scale");
    blt_scale_hip(t, scalar);
}

void blt_patch_pool_forward(const blt_tensor *byte_hidden, const blt_patch_info *patches, size_t num_patches,
                            blt_patch_pool_type pool_type, blt_tensor *out) {
    BLT_REQUIRE(byte_hidden != NULL, "patch_pool: NULL tensor");
    BLT_DEVICE_ONLY(byte_hidden->backend, "blt_patch_pool_forward");
    blt_patch_pool_forward_hip(byte_hidden, patches, num_patches, pool_type, out);
}

void blt_local_encoder_forward(const blt_local_encoder *model, const blt_tensor *bytes_in, const blt_patch_info *patches,
                               size_t num_patches, const size_t *doc_boundaries, size_t num_docs, blt_tensor *patch_out,
                               blt_tensor *byte_hidden_out, blt_arena *arena) {
    BLT_REQUIRE(patch_out != NULL, "blt_local_encoder_forward: patch_out and byte_hidden_out cannot be NULL");
    BLT_DEVICE_ONLY(patch_out->backend, "blt_local_encoder_forward");
    blt_local_encoder_forward_hip(model, bytes_in, patches, num_patches, doc_boundaries, num_docs, patch_out,
                                  byte_hidden_out, arena);
}

void blt_local_decoder_forward_ext(const blt_local_decoder *model, const blt_tensor *byte_hidden_in,
                                   const blt_tensor *patch_in, const blt_patch_info *patches, size_t num_patches,
                                   const blt_tensor *bytes_in, const blt_tensor *targets, const size_t *doc_boundaries,
                                   size_t num_docs, const blt_local_decoder_d0_opts *d0_opts, int trailing_closed,
                                   blt_tensor *logits_out, blt_tensor *loss_out, blt_arena *arena) {
    (void)targets;
    BLT_REQUIRE(logits_out != NULL, "blt_local_decoder_forward_ext: logits_out cannot be NULL");
    BLT_REQUIRE(loss_out != NULL || bytes_in == NULL,
                "blt_local_decoder_forward_ext: bytes_in is only used for the loss; pass NULL when loss_out is NULL");
    BLT_DEVICE_ONLY(logits_out->backend, "blt_local_decoder_forward_ext");
    BLT_REQUIRE(loss_out == NULL,
                "blt_local_decoder_forward_ext: the HIP backend runs the inference form only (loss_out must be NULL)");
    BLT_REQUIRE(d0_opts == NULL || d0_opts->d0_mode == BLT_D0_HFINAL,
                "blt_local_decoder_forward_ext: D_0 modes other than BLT_D0_HFINAL go through "
                "blt_local_decoder_forward_diffusion_infer on the HIP backend");
    blt_local_decoder_forward_ext_hip(model, byte_hidden_in, patch_in, patches, num_patches, doc_boundaries, num_docs,
                                      trailing_closed, logits_out, arena);
}

void blt_add(const blt_tensor *a, const blt_tensor *b, blt_tensor *out) {
    BLT_REQUIRE(a != NULL, "blt_add: input tensors must be FP32 with matching element count");
    BLT_DEVICE_ONLY(a->backend, "blt_add");
    blt_add_hip(a, b, out);
}

void blt_swiglu_forward(const blt_tensor *gate, const blt_tensor *up, blt_tensor *out) {
    BLT_REQUIRE(gate != NULL, "SwiGLU: gate/up must be FP32 with matching element count");
    BLT_DEVICE_ONLY(gate->backend, "blt_swiglu_forward");
    blt_swiglu_forward_hip(gate, up, out);
}

void blt_rmsnorm_forward(const blt_tensor *x, const blt_tensor *weight, blt_tensor *out) {
    BLT_REQUIRE(x != NULL, "RMSNorm: input must be 2D FP32");
    BLT_DEVICE_ONLY(x->backend, "blt_rmsnorm_forward");
    blt_rmsnorm_forward_hip(x, weight, out);
}

void blt_matmul(const blt_tensor *a, const blt_tensor *b, blt_tensor *out) {
    BLT_REQUIRE(a != NULL, "matmul: inputs must not be NULL");
    BLT_DEVICE_ONLY(a->backend, "blt_matmul");
    blt_matmul_hip(a, b, out);
}

void blt_rope_precompute(size_t max_seq_len, const blt_rope_config *config, blt_tensor *cos_out, blt_tensor *sin_out) {
    BLT_REQUIRE(config != NULL && cos_out != NULL && sin_out != NULL, "rope: arguments must not be NULL");
    BLT_DEVICE_ONLY(cos_out->backend, "blt_rope_precompute");
    BLT_REQUIRE(config->head_dim % 2 == 0, "rope: head_dim must be even");
    const size_t half = config->head_dim / 2;
    BLT_REQUIRE(cos_out->ndim == 2 && cos_out->dtype == BLT_DTYPE_FP32 && cos_out->shape[0] == max_seq_len &&
                    cos_out->shape[1] == half,
                "rope cos_out");
    BLT_REQUIRE(sin_out->ndim == 2 && sin_out->dtype == BLT_DTYPE_FP32 && sin_out->shape[0] == max_seq_len &&
                    sin_out->shape[1] == half && sin_out->backend == cos_out->backend,
                "rope sin_out");
    if (max_seq_len * half == 0) return;
    float *c = (float *)malloc(max_seq_len * half * sizeof(float));
    float *s = (float *)malloc(max_seq_len * half * sizeof(float));
    BLT_REQUIRE(c != NULL && s != NULL, "rope: failed to allocate host staging");
    /* the reference's formula and libm calls, csrc/ops/reductions_cpu.c:188-196 */
    for (size_t pos = 0; pos < max_seq_len; pos++) {
        for (size_t i = 0; i < half; i++) {
            float freq = 1.0f / powf(config->theta, (float)(2 * i) / (float)config->head_dim);
            float angle = (float)pos * freq;
            c[pos * half + i] = cosf(angle);
            s[pos * half + i] = sinf(angle);
        }
    }
    blt_hip_memcpy_h2d(cos_out->data, c, max_seq_len * half * sizeof(float));
    blt_hip_memcpy_h2d(sin_out->data, s, max_seq_len * half * sizeof(float));
    blt_backend_pass_sync_hip(); /* the staging buffers are freed next */
    free(c);
    free(s);
}

void blt_rope_apply(const blt_tensor *x, const blt_tensor *cos, const blt_tensor *sin, blt_tensor *out) {
    BLT_REQUIRE(x != NULL, "rope: x must be 3D FP32");
    BLT_DEVICE_ONLY(x->backend, "blt_rope_apply");
    blt_rope_apply_hip(x, cos, sin, out);
}

void blt_rope_apply_packed(float *qkv_data, size_t qkv_stride, size_t head_offset, size_t seq_len, size_t head_dim,
                           const float *cos, const float *sin, blt_backend backend) {
    BLT_DEVICE_ONLY(backend, "blt_rope_apply_packed");
    blt_rope_apply_packed_hip(qkv_data, qkv_stride, head_offset, seq_len, head_dim, cos, sin);
}

void blt_multihead_attention(const blt_tensor *input, const blt_tensor *weight_qkv, const blt_tensor *weight_proj,
                             blt_tensor *output, const blt_attention_config *config, blt_arena *arena) {
    BLT_REQUIRE(input != NULL, "blt_multihead_attention: input must be [seq_len, embed_dim] FP32");
    BLT_DEVICE_ONLY(input->backend, "blt_multihead_attention");
    blt_multihead_attention_hip(input, weight_qkv, weight_proj, output, config, arena);
}

float blt_vec_dot(blt_backend backend, const float *a, const float *b, size_t n) {
    BLT_DEVICE_ONLY(backend, "blt_vec_dot");
    return blt_vec_dot_hip(backend, a, b, n);
}

/* ------------------------------------------------------------------ */
/* Byte <-> patch index (reference: csrc/ops/patch_pool_cpu.c:98-142)   */
/* ------------------------------------------------------------------ */

void blt_patch_build_group_ids(const blt_patch_info *patches, size_t num_patches, size_t seq_len,
                               size_t *query_group_ids_out, size_t *kv_group_ids_out) {
    BLT_REQUIRE(patches != NULL || num_patches == 0, "patch_group_ids: NULL patches");
    BLT_REQUIRE(query_group_ids_out != NULL && kv_group_ids_out != NULL, "patch_group_ids: NULL output array");

    size_t cursor = 0;
    for (size_t p = 0; p < num_patches; p++) {
        query_group_ids_out[p] = p;
        BLT_REQUIRE(patches[p].start_idx == cursor, "patch_group_ids: patches must tile [0, seq_len) contiguously");
        BLT_REQUIRE(patches[p].length >= 1, "patch_group_ids: empty patch");
        const size_t end = cursor + patches[p].length;
        BLT_REQUIRE(end <= seq_len, "patch_group_ids: patches do not cover [0, seq_len) exactly");
        while (cursor < end) kv_group_ids_out[cursor++] = p;
    }
    BLT_REQUIRE(cursor == seq_len, "patch_group_ids: patches do not cover [0, seq_len) exactly");
}

size_t blt_patch_decoder_latent_at(const blt_patch_info *patches, size_t num_patches, size_t pos) {
    BLT_REQUIRE(patches != NULL && num_patches >= 1, "patch_decoder_latent: need at least one patch");
    if (pos < patches[0].start_idx) return 0;
    /* Patches are ordered by start; the owner is the last one starting at or before pos. */
    size_t owner = num_patches;
    for (size_t p = 0; p < num_patches && patches[p].start_idx <= pos; p++) {
        if (pos - patches[p].start_idx < patches[p].length) {
            owner = p;
            break;
        }
    }
    if (owner == num_patches) return num_patches - 1; /* not covered by any patch */
    const int closes_patch = (pos - patches[owner].start_idx) + 1 == patches[owner].length;
    const int has_successor = owner + 1 < num_patches;
    if (closes_patch && has_successor) return owner; /* final byte: its own latent */
    return owner == 0 ? 0 : owner - 1;               /* otherwise the previous latent */
}

void blt_patch_expand_group_ids(const size_t *group_ids_in, size_t n, size_t k, size_t *group_ids_out) {
    BLT_REQUIRE(group_ids_in != NULL || n == 0, "patch_expand_group_ids: NULL group_ids_in");
    BLT_REQUIRE(group_ids_out != NULL || n * k == 0, "patch_expand_group_ids: NULL group_ids_out");
    BLT_REQUIRE(k >= 1, "patch_expand_group_ids: k must be >= 1");
    size_t w = 0;
    for (size_t i = 0; i < n; i++)
        for (size_t r = 0; r < k; r++) group_ids_out[w++] = group_ids_in[i];
}

/* ------------------------------------------------------------------ */
/* Mask recipe -> per-row key ranges                                    */
/* ------------------------------------------------------------------ */

/* Document id per position from the boundary list: entry d is the first
 * position of document d+1 (reference: csrc/ops/mask_builder_cpu.c:11-19). */
static void doc_ids(const size_t *bounds, size_t num_docs, size_t len, size_t *out) {
    size_t d = 0;
    for (size_t p = 0; p < len; p++) {
        while (d + 1 < num_docs && p >= bounds[d]) d++;
        out[p] = d;
    }
}

/* For an id array, first[j]/last[j] style lookups: returns 1 when equal ids
 * form contiguous runs (so "same id" is an interval of positions). */
static int runs_are_contiguous(const size_t *ids, size_t n) {
    /* A value may not reappear after its run ended.  O(n log n) would need a
     * sort; ids here are patch/doc indices < n in practice, so try a direct
     * table first and fall back to a quadratic scan for exotic values. */
    size_t maxv = 0;
    for (size_t i = 0; i < n; i++)
        if (ids[i] > maxv) maxv = ids[i];
    if (maxv <= 4 * n + 1024) {
        unsigned char *seen = (unsigned char *)calloc(maxv + 1, 1);
        if (!seen) return 0;
        int ok = 1;
        for (size_t i = 0; i < n && ok; i++) {
            if (i > 0 && ids[i] == ids[i - 1]) continue;
            if (seen[ids[i]]) ok = 0;
            seen[ids[i]] = 1;
        }
        free(seen);
        return ok;
    }
    for (size_t i = 1; i < n; i++) {
        if (ids[i] == ids[i - 1]) continue;
        for (size_t j = 0; j + 1 < i; j++)
            if (ids[j] == ids[i]) return 0;
    }
    return 1;
}

/* Interval [lo, hi) of positions of `ids` (length n, contiguous runs) that
 * carry value `want`; lo == hi when absent.  `hint` speeds up sorted queries. */
static void run_of(const size_t *ids, size_t n, size_t want, size_t *hint, size_t *lo, size_t *hi) {
    size_t s = *hint < n ? *hint : 0;
    size_t scanned = 0;
    while (scanned < n && ids[s] != want) {
        s = (s + 1 == n) ? 0 : s + 1;
        scanned++;
    }
    if (scanned == n) {
        *lo = *hi = 0;
        return;
    }
    size_t b = s;
    while (b > 0 && ids[b - 1] == want) b--;
    size_t e = s;
    while (e < n && ids[e] == want) e++;
    *lo = b;
    *hi = e;
    *hint = b;
}

static inline size_t zmin(size_t a, size_t b) { return a < b ? a : b; }
static inline size_t zmax(size_t a, size_t b) { return a > b ? a : b; }

int blt_mask_config_row_ranges(const blt_mask_config *c, uint32_t *lo_out, uint32_t *hi_out) {
    BLT_REQUIRE(c != NULL && lo_out != NULL && hi_out != NULL, "blt_mask_config_row_ranges: NULL argument");
    const size_t nq = c->seq_len_q, nk = c->seq_len_kv;
    BLT_REQUIRE(nq > 0 && nk > 0, "blt_mask_config_row_ranges: seq_len_q/seq_len_kv must be > 0");
    if (nk > 0xFFFFFFFFu || nq > 0xFFFFFFFFu) return 0;

    const int docs = c->doc_boundaries != NULL && c->num_docs > 0;
    const int groups = c->query_group_ids != NULL && c->kv_group_ids != NULL;
    const size_t W = c->sliding_window;

    size_t *dq = NULL, *dk = NULL;
    int ok = 1;
    if (docs) {
        dq = (size_t *)malloc(nq * sizeof(size_t));
        dk = (size_t *)malloc(nk * sizeof(size_t));
        BLT_REQUIRE(dq != NULL && dk != NULL, "blt_mask_config_row_ranges: out of host memory");
        doc_ids(c->doc_boundaries, c->num_docs, nq, dq);
        doc_ids(c->doc_boundaries, c->num_docs, nk, dk); /* non-decreasing, so runs are contiguous */
    }
    if (groups && !runs_are_contiguous(c->kv_group_ids, nk)) ok = 0;

    size_t doc_hint = 0, grp_hint = 0;
    for (size_t i = 0; i < nq && ok; i++) {
        size_t lo = 0, hi = nk; /* allowed keys: lo <= j < hi */
        if (c->is_causal) {
            /* j <= i + offset */
            const size_t diag = i + c->causal_offset;
            hi = zmin(hi, diag + 1);
            if (W > 0) {
                /* |diag - j| < W */
                lo = zmax(lo, diag + 1 >= W ? diag + 1 - W : 0);
                hi = zmin(hi, diag + W);
            }
        } else if (W > 0) {
            lo = zmax(lo, i + 1 >= W ? i + 1 - W : 0);
            hi = zmin(hi, i + W);
        }
        if (docs) {
            size_t a, b;
            run_of(dk, nk, dq[i], &doc_hint, &a, &b);
            lo = zmax(lo, a);
            hi = zmin(hi, b);
        }
        if (groups) {
            size_t a, b;
            run_of(c->kv_group_ids, nk, c->query_group_ids[i], &grp_hint, &a, &b);
            lo = zmax(lo, a);
            hi = zmin(hi, b);
            if (!c->bidirectional_within_group) hi = zmin(hi, i + 1);
        }
        if (hi < lo) hi = lo;
        lo_out[i] = (uint32_t)lo;
        hi_out[i] = (uint32_t)hi;
    }
    free(dq);
    free(dk);
    return ok;
}
