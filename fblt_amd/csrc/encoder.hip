/*
 * The local encoder's forward pass on the device, and the three tensor ops it
 * needs beyond the attention blocks (reference: csrc/models/local_encoder.c:193-281,
 * csrc/models/hash_ngram.c:142-207, csrc/models/byte_embedding.c:16-53,
 * csrc/ops/gather_scatter_cpu.c:41-61, csrc/ops/elementwise_cpu.c:31-40,
 * csrc/ops/patch_pool_cpu.c:3-48):
 *
 *   e_0 = (byte_embedding[b_i] + sum_n table_n[hash_n(b_{i-n+1..i})]) / (K + 1)
 *   P_0 = pool(e_0, patches), repeated over the k sub-token column blocks
 *   per layer: h = transformer_block(h); where the cross block fires,
 *              P = P + cross_attention(RMSNorm(P), h)
 *
 * Hashing is integer work on the host, as in the reference; everything that
 * touches floats runs on the device.  The three small kernels keep the
 * reference's order of additions, so they are bit-identical to the CPU ops:
 * the embedding sum adds the tables in their order and scales last, the mean
 * pool adds a patch's rows first to last and multiplies by 1 / len.
 */
#include "blt_hip.h"
#include "blt_fatal.h"
#include "hip_check.h"
#include "launch.h"

#include <cstdlib>
#include <cstring>
#include <vector>

/* blt_cross_attention_forward_hip with the steps either side of it in a caller's layer folded in
 * (mha.hip): norm_w, when set, is the weight of the RMSNorm that makes query_in's rows the queries
 * (taken inside the query projection), residual [rows, embed] is added to the projected output. */
void blt_cross_attention_run(const blt_tensor *query_in, const blt_tensor *kv_in,
                             const blt_cross_attention_weights *weights, blt_tensor *output,
                             const blt_cross_attention_config *config, blt_arena *arena, const float *norm_w,
                             const float *residual);

namespace {

constexpr int IDX_PER_LAUNCH = 512; /* index entries a launch carries in its arguments */
struct IndexChunk {
    uint32_t v[IDX_PER_LAUNCH];
};

/* io[row0 + i, :] += table[idx[i], :] for every i whose index is not the sentinel */
__global__ __launch_bounds__(256) void rows_accumulate_kernel(const float *__restrict__ table, float *__restrict__ io,
                                                              uint64_t row_len, IndexChunk idx) {
    const uint32_t at = idx.v[blockIdx.x];
    if (at == BLT_IDX_SENTINEL) return;
    const float *s = table + (uint64_t)at * row_len;
    float *d = io + (uint64_t)blockIdx.x * row_len;
    for (uint64_t t = threadIdx.x; t < row_len; t += 256u) d[t] += s[t];
}

__global__ __launch_bounds__(256) void scale_kernel(float *__restrict__ x, uint64_t n, float scalar) {
    for (uint64_t t = (uint64_t)blockIdx.x * 256u + threadIdx.x; t < n; t += (uint64_t)gridDim.x * 256u) x[t] *= scalar;
}

constexpr int PATCHES_PER_LAUNCH = 256;
struct PatchChunk {
    uint32_t start[PATCHES_PER_LAUNCH];
    uint32_t len[PATCHES_PER_LAUNCH];
};

/* One workgroup per patch, one thread per column: the patch's rows first to last (the reference's
 * order of additions), written into `copies` column blocks of the output row. */
__global__ __launch_bounds__(256) void patch_pool_kernel(const float *__restrict__ h, float *__restrict__ out,
                                                         uint32_t embed_dim, uint32_t out_stride, uint32_t copies,
                                                         int take_max, PatchChunk p) {
    const uint32_t start = p.start[blockIdx.x], len = p.len[blockIdx.x];
    float *dst = out + (uint64_t)blockIdx.x * out_stride;
    for (uint32_t d = threadIdx.x; d < embed_dim; d += 256u) {
        const float *src = h + (uint64_t)start * embed_dim + d;
        float acc;
        if (take_max) {
            acc = src[0];
            for (uint32_t i = 1; i < len; i++) {
                const float v = src[(uint64_t)i * embed_dim];
                if (v > acc) acc = v;
            }
        } else {
            acc = 0.0f;
            for (uint32_t i = 0; i < len; i++) acc += src[(uint64_t)i * embed_dim];
            acc *= 1.0f / (float)len;
        }
        for (uint32_t c = 0; c < copies; c++) dst[c * embed_dim + d] = acc;
    }
}

constexpr int MAX_TABLES = BLT_MAX_NGRAM_SIZES;
struct EmbedTables {
    const float *table[MAX_TABLES];
    const uint32_t *idx[MAX_TABLES]; /* device arrays [seq_len], sentinel = no contribution */
    uint32_t count;
};

/* out[i, :] = (byte_table[ids[i], :] + table_0[idx_0[i], :] + ... ) * scale, the tables in order */
__global__ __launch_bounds__(256) void embed_sum_kernel(const float *__restrict__ byte_table,
                                                        const uint32_t *__restrict__ ids, float *__restrict__ out,
                                                        uint32_t embed_dim, EmbedTables t, int scaled, float scale) {
    const uint32_t i = blockIdx.x;
    const float *base = byte_table + (uint64_t)ids[i] * embed_dim;
    for (uint32_t d = threadIdx.x; d < embed_dim; d += 256u) {
        float acc = base[d];
        for (uint32_t n = 0; n < t.count; n++) {
            const uint32_t at = t.idx[n][i];
            if (at != BLT_IDX_SENTINEL) acc += t.table[n][(uint64_t)at * embed_dim + d];
        }
        if (scaled) acc *= scale;
        out[(uint64_t)i * embed_dim + d] = acc;
    }
}

void check_2d(const blt_tensor *t, size_t rows, size_t cols, const char *msg) {
    BLT_REQUIRE(t != NULL && t->data != NULL && t->ndim == 2 && t->dtype == BLT_DTYPE_FP32 &&
                    t->backend == BLT_BACKEND_HIP && (rows == 0 || t->shape[0] == rows) &&
                    (cols == 0 || t->shape[1] == cols),
                "%s", msg);
}

blt_tensor view_2d(void *data, size_t rows, size_t cols) {
    blt_tensor t;
    std::memset(&t, 0, sizeof(t));
    t.data = data;
    t.shape[0] = rows, t.shape[1] = cols;
    t.strides[0] = cols, t.strides[1] = 1;
    t.ndim = 2;
    t.numel = rows * cols;
    t.dtype = BLT_DTYPE_FP32;
    t.backend = BLT_BACKEND_HIP;
    t.is_view = true;
    return t;
}

void pool_launch(const float *h, size_t seq_len, size_t embed_dim, const blt_patch_info *patches, size_t num_patches,
                 blt_patch_pool_type pool_type, float *out, size_t out_stride, size_t copies) {
    BLT_REQUIRE(pool_type == BLT_POOL_MEAN || pool_type == BLT_POOL_MAX, "patch_pool: unknown pool_type");
    BLT_REQUIRE(seq_len <= 0xFFFFFFFFu && embed_dim <= 0xFFFFFFFFu && out_stride <= 0xFFFFFFFFu,
                "patch_pool: sizes exceed 2^32-1");
    for (size_t j0 = 0; j0 < num_patches; j0 += PATCHES_PER_LAUNCH) {
        const size_t n = std::min<size_t>(PATCHES_PER_LAUNCH, num_patches - j0);
        PatchChunk c;
        std::memset(&c, 0, sizeof(c));
        for (size_t j = 0; j < n; j++) {
            const blt_patch_info &pi = patches[j0 + j];
            BLT_REQUIRE(pi.length >= 1, "patch_pool: empty patch");
            BLT_REQUIRE(pi.start_idx + pi.length <= seq_len, "patch_pool: patch out of range");
            c.start[j] = (uint32_t)pi.start_idx, c.len[j] = (uint32_t)pi.length;
        }
        hipLaunchKernelGGL(patch_pool_kernel, dim3((unsigned)n), dim3(256), 0, blt_stream(), h, out + j0 * out_stride,
                           (uint32_t)embed_dim, (uint32_t)out_stride, (uint32_t)copies,
                           pool_type == BLT_POOL_MAX ? 1 : 0, c);
        HIP_CHECK_LAUNCH("blt_patch_pool_forward");
    }
}

/* The reference's rolling polynomial hash (csrc/models/hash_ngram.c:16-79), restated in closed
 * form: position i >= n - 1 hashes bytes b[i-n+1..i] as sum b[j] * prime^(i-j) mod modulus;
 * earlier positions have no n-gram.  prime * modulus fits 64 bits (checked as the reference does),
 * so no product overflows. */
void ngram_indices(const uint8_t *bytes, size_t seq_len, size_t n, uint64_t prime, uint64_t modulus, uint32_t *idx) {
    BLT_REQUIRE(n > 0 && n <= 8, "blt_rolling_hash_init: n must be in [1, 8]");
    BLT_REQUIRE(modulus > 1, "blt_rolling_hash_init: modulus must be > 1");
    BLT_REQUIRE(prime > 0 && prime <= ((UINT64_MAX - 255) / modulus),
                "blt_rolling_hash_init: prime * modulus would overflow uint64");
    for (size_t i = 0; i < seq_len; i++) {
        if (i + 1 < n) {
            idx[i] = BLT_IDX_SENTINEL;
            continue;
        }
        uint64_t hash = 0;
        for (size_t j = i + 1 - n; j <= i; j++) hash = (hash * prime + bytes[j]) % modulus;
        idx[i] = (uint32_t)hash;
    }
}

} // namespace

/* Replaces blt_indexed_row_accumulate_cuda (contract csrc/ops/gather_scatter.h:23-28,
 * gather_scatter_cpu.c:41-61): io[i, :] += table[idx_host[i], :], sentinel entries skipped. */
extern "C" void blt_indexed_row_accumulate_hip(const blt_tensor *table, const uint32_t *idx_host, blt_tensor *io) {
    BLT_REQUIRE(table != NULL && idx_host != NULL && io != NULL, "blt_indexed_row_accumulate: arguments cannot be NULL");
    check_2d(table, 0, 0, "blt_indexed_row_accumulate: HIP implementation needs 2D FP32 device tensors");
    check_2d(io, 0, 0, "blt_indexed_row_accumulate: HIP implementation needs 2D FP32 device tensors");
    const size_t rows = io->shape[0], embed_dim = io->shape[1];
    BLT_REQUIRE(table->shape[1] == embed_dim, "blt_indexed_row_accumulate: embed_dim mismatch");
    if (embed_dim == 0) return;
    for (size_t r0 = 0; r0 < rows; r0 += IDX_PER_LAUNCH) {
        const size_t n = std::min<size_t>(IDX_PER_LAUNCH, rows - r0);
        IndexChunk c;
        for (size_t i = 0; i < (size_t)IDX_PER_LAUNCH; i++) {
            c.v[i] = i < n ? idx_host[r0 + i] : BLT_IDX_SENTINEL;
            BLT_REQUIRE(c.v[i] == BLT_IDX_SENTINEL || c.v[i] < table->shape[0],
                        "blt_indexed_row_accumulate: index out of range");
        }
        hipLaunchKernelGGL(rows_accumulate_kernel, dim3((unsigned)n), dim3(256), 0, blt_stream(),
                           (const float *)table->data, (float *)io->data + r0 * embed_dim, (uint64_t)embed_dim, c);
        HIP_CHECK_LAUNCH("blt_indexed_row_accumulate");
    }
}

/* Replaces blt_scale_cuda (csrc/ops/elementwise.h:10, elementwise_cpu.c:31-40): t *= scalar in place. */
extern "C" void blt_scale_hip(blt_tensor *t, float scalar) {
    BLT_REQUIRE(t != NULL, "blt_scale: tensor must not be null");
    BLT_REQUIRE(t->dtype == BLT_DTYPE_FP32, "blt_scale: only supports FP32 tensors");
    BLT_REQUIRE(t->backend == BLT_BACKEND_HIP, "blt_scale: HIP implementation called with non-HIP backend");
    if (t->numel == 0) return;
    const unsigned blocks = (unsigned)std::min<size_t>((t->numel + 255u) / 256u, 4096u);
    hipLaunchKernelGGL(scale_kernel, dim3(blocks), dim3(256), 0, blt_stream(), (float *)t->data, (uint64_t)t->numel,
                       scalar);
    HIP_CHECK_LAUNCH("blt_scale");
}

/* Replaces blt_patch_pool_forward_cuda (contract csrc/ops/patch_pool.h:18-21, patch_pool_cpu.c:3-48):
 * out[j, :] = mean or per-column maximum of byte_hidden rows [start_j, start_j + len_j); the
 * patch table is a HOST array. */
extern "C" void blt_patch_pool_forward_hip(const blt_tensor *byte_hidden, const blt_patch_info *patches,
                                           size_t num_patches, blt_patch_pool_type pool_type, blt_tensor *out) {
    BLT_REQUIRE(byte_hidden != NULL && out != NULL, "patch_pool: NULL tensor");
    BLT_REQUIRE(patches != NULL || num_patches == 0, "patch_pool: NULL patches");
    check_2d(byte_hidden, 0, 0, "patch_pool: byte_hidden must be 2D FP32");
    const size_t seq_len = byte_hidden->shape[0], embed_dim = byte_hidden->shape[1];
    check_2d(out, num_patches, embed_dim, "patch_pool: out must be [num_patches, embed_dim] FP32");
    if (num_patches == 0 || embed_dim == 0) return;
    pool_launch((const float *)byte_hidden->data, seq_len, embed_dim, patches, num_patches, pool_type,
                (float *)out->data, embed_dim, 1);
}

/* csrc/models/local_encoder.c:193-281 on device tensors.  bytes_in may live on either side (the
 * ids are consumed on the host, as in the reference); weights, outputs and the arena are device
 * memory.  Index arrays and mask metadata are host allocations of this call. */
extern "C" void blt_local_encoder_forward_hip(const blt_local_encoder *model, const blt_tensor *bytes_in,
                                              const blt_patch_info *patches, size_t num_patches,
                                              const size_t *doc_boundaries, size_t num_docs, blt_tensor *patch_out,
                                              blt_tensor *byte_hidden_out, blt_arena *arena) {
    BLT_REQUIRE(model != NULL && bytes_in != NULL && arena != NULL,
                "blt_local_encoder: model, bytes_in and arena cannot be NULL");
    BLT_REQUIRE(arena->backend == BLT_BACKEND_HIP, "blt_local_encoder: HIP implementation needs a device arena");
    BLT_REQUIRE(patches != NULL && num_patches >= 1, "blt_local_encoder: need at least one patch");
    BLT_REQUIRE(bytes_in->ndim == 1 && bytes_in->dtype == BLT_DTYPE_UINT8,
                "blt_local_encoder: bytes_in must be 1D UINT8 [seq_len]");
    const blt_local_encoder_config &cfg = model->config;
    const size_t seq_len = bytes_in->shape[0];
    BLT_REQUIRE(seq_len >= 1 && seq_len <= cfg.max_seq_len, "blt_local_encoder: seq_len must be in [1, max_seq_len]");
    BLT_REQUIRE(patch_out != NULL && byte_hidden_out != NULL,
                "blt_local_encoder_forward: patch_out and byte_hidden_out cannot be NULL");
    const size_t E = cfg.embed_dim;
    const size_t patch_dim = cfg.patch_dim == 0 ? E : cfg.patch_dim;
    BLT_REQUIRE(E > 0 && patch_dim % E == 0, "blt_local_encoder_forward: patch_dim must be a multiple of embed_dim");
    const size_t k = patch_dim / E;
    check_2d(patch_out, num_patches, patch_dim, "blt_local_encoder_forward: patch_out must be [num_patches, patch_dim] FP32");
    check_2d(byte_hidden_out, seq_len, E, "blt_local_encoder_forward: byte_hidden_out must be [seq_len, embed_dim] FP32");
    check_2d(&model->byte_embedding_weight, 256, E, "blt_local_encoder_forward: byte_embedding_weight must be [256, embed_dim]");
    BLT_REQUIRE(cfg.num_heads >= 1 && E % cfg.num_heads == 0 && (E / cfg.num_heads) % 2 == 0,
                "blt_local_encoder_forward: embed_dim must split into heads of even width");
    const size_t half = E / cfg.num_heads / 2;
    check_2d(&model->rope_cos_cache, 0, half, "blt_local_encoder_forward: rope caches must be [max_seq_len, head_dim/2]");
    check_2d(&model->rope_sin_cache, 0, half, "blt_local_encoder_forward: rope caches must be [max_seq_len, head_dim/2]");
    BLT_REQUIRE(model->rope_cos_cache.shape[0] >= seq_len && model->rope_sin_cache.shape[0] >= seq_len,
                "blt_local_encoder_forward: rope caches are shorter than the sequence");
    BLT_REQUIRE(model->layers != NULL && cfg.num_layers >= 1, "blt_local_encoder_forward: layers cannot be NULL");
    const blt_hash_ngram_config &ng = cfg.ngram_config;
    BLT_REQUIRE(ng.num_ngram_sizes <= BLT_MAX_NGRAM_SIZES && ng.embed_dim == E,
                "blt_local_encoder_forward: ngram_config does not fit the encoder");

    /* ---- ids and bucket indices: host work, one upload ---- */
    std::vector<uint8_t> bytes(seq_len);
    if (bytes_in->backend == BLT_BACKEND_HIP) blt_hip_memcpy_d2h(bytes.data(), bytes_in->data, seq_len);
    else std::memcpy(bytes.data(), bytes_in->data, seq_len);
    std::vector<uint32_t> host_idx((1 + (size_t)MAX_TABLES) * seq_len);
    for (size_t i = 0; i < seq_len; i++) host_idx[i] = bytes[i];
    EmbedTables tables;
    std::memset(&tables, 0, sizeof(tables));
    uint32_t *dev_idx = (uint32_t *)blt_arena_alloc(arena, host_idx.size() * sizeof(uint32_t), 64);
    for (size_t t = 0; t < ng.num_ngram_sizes; t++) {
        const size_t n = ng.ngram_sizes[t];
        if (n == 0 || n > seq_len) continue; /* hash_ngram.c:178-180 */
        check_2d(&model->ngram_weights.tables[t], ng.per_ngram_vocab, E, "blt_hash_ngram_forward: weights->tables");
        uint32_t *dst = host_idx.data() + (1 + (size_t)tables.count) * seq_len;
        ngram_indices(bytes.data(), seq_len, n, ng.hash_prime, ng.per_ngram_vocab, dst);
        tables.table[tables.count] = (const float *)model->ngram_weights.tables[t].data;
        tables.idx[tables.count] = dev_idx + (1 + (size_t)tables.count) * seq_len;
        tables.count++;
    }
    blt_hip_memcpy_h2d(dev_idx, host_idx.data(), (1 + (size_t)tables.count) * seq_len * sizeof(uint32_t));

    const size_t byte_shape[2] = {seq_len, E}, patch_shape[2] = {num_patches, patch_dim};
    blt_tensor h = blt_tensor_create_uninit(arena, byte_shape, 2, BLT_DTYPE_FP32);
    hipLaunchKernelGGL(embed_sum_kernel, dim3((unsigned)seq_len), dim3(256), 0, blt_stream(),
                       (const float *)model->byte_embedding_weight.data, (const uint32_t *)dev_idx, (float *)h.data,
                       (uint32_t)E, tables, ng.normalize ? 1 : 0, 1.0f / (float)(ng.num_ngram_sizes + 1));
    HIP_CHECK_LAUNCH("blt_local_encoder_forward: embedding");

    /* ---- P_0: pooled rows in every sub-token column block (local_encoder.c:237-245) ---- */
    blt_tensor p = blt_tensor_create_uninit(arena, patch_shape, 2, BLT_DTYPE_FP32);
    pool_launch((const float *)h.data, seq_len, E, patches, num_patches, cfg.pool_type, (float *)p.data, patch_dim, k);

    /* ---- masks (local_encoder.c:52-113): host metadata ---- */
    std::vector<size_t> q_groups(num_patches), kv_groups(seq_len), q_groups_split;
    blt_patch_build_group_ids(patches, num_patches, seq_len, q_groups.data(), kv_groups.data());
    blt_mask_config local_mask, cross_mask;
    std::memset(&local_mask, 0, sizeof(local_mask));
    std::memset(&cross_mask, 0, sizeof(cross_mask));
    local_mask.seq_len_q = local_mask.seq_len_kv = seq_len;
    local_mask.sliding_window = cfg.local_window;
    local_mask.doc_boundaries = doc_boundaries;
    local_mask.num_docs = num_docs;
    local_mask.is_causal = true;
    cross_mask.seq_len_q = num_patches * k;
    cross_mask.seq_len_kv = seq_len;
    cross_mask.kv_group_ids = kv_groups.data();
    cross_mask.bidirectional_within_group = true;
    if (k == 1) {
        cross_mask.query_group_ids = q_groups.data();
    } else {
        q_groups_split.resize(num_patches * k);
        blt_patch_expand_group_ids(q_groups.data(), num_patches, k, q_groups_split.data());
        cross_mask.query_group_ids = q_groups_split.data();
    }
    blt_tensor cos_view = view_2d(model->rope_cos_cache.data, seq_len, half);
    blt_tensor sin_view = view_2d(model->rope_sin_cache.data, seq_len, half);

    blt_transformer_config layer_cfg;
    std::memset(&layer_cfg, 0, sizeof(layer_cfg));
    layer_cfg.attn_config.embed_dim = E;
    layer_cfg.attn_config.num_heads = cfg.num_heads;
    layer_cfg.attn_config.is_causal = true;
    layer_cfg.attn_config.use_rope = true;
    layer_cfg.attn_config.rope_theta = cfg.rope_theta;
    layer_cfg.attn_config.rope_cos_cache = &cos_view;
    layer_cfg.attn_config.rope_sin_cache = &sin_view;
    layer_cfg.attn_config.mask_config = &local_mask;
    layer_cfg.hidden_dim = cfg.hidden_dim;
    layer_cfg.norm_type = BLT_NORM_RMSNORM;
    layer_cfg.activation_type = BLT_ACTIVATION_SWIGLU;
    blt_cross_attention_config cross_cfg;
    std::memset(&cross_cfg, 0, sizeof(cross_cfg));
    cross_cfg.embed_dim = E;
    cross_cfg.patch_dim = patch_dim;
    cross_cfg.split_mode = k == 1 ? BLT_CROSS_ATTN_NO_SPLIT : BLT_CROSS_ATTN_SPLIT_QUERY;
    cross_cfg.num_heads = cfg.cross_attn_heads;
    cross_cfg.mask_config = &cross_mask;

    /* ---- layers; the last results land in the caller's tensors ---- */
    size_t last_cross = cfg.num_layers; /* none */
    for (size_t l = 0; l < cfg.num_layers; l++)
        if (blt_local_cross_attn_fires(cfg.cross_attn_placement, cfg.cross_attn_all_layers, cfg.num_layers, l)) last_cross = l;
    for (size_t l = 0; l < cfg.num_layers; l++) {
        const blt_local_layer_storage *s = &model->layers[l];
        blt_transformer_weights w;
        std::memset(&w, 0, sizeof(w));
        w.norm1_weight = &s->norm1_weight, w.attn_qkv_w = &s->attn_qkv_w, w.attn_proj_w = &s->attn_proj_w;
        w.norm2_weight = &s->norm2_weight, w.ffn_up_w = &s->ffn_up_w, w.ffn_gate_w = &s->ffn_gate_w;
        w.ffn_down_w = &s->ffn_down_w;
        blt_tensor h_next = l + 1 == cfg.num_layers ? view_2d(byte_hidden_out->data, seq_len, E)
                                                    : blt_tensor_create_uninit(arena, byte_shape, 2, BLT_DTYPE_FP32);
        blt_transformer_forward_hip(&h, &w, &h_next, &layer_cfg, arena);
        h = h_next;
        if (!blt_local_cross_attn_fires(cfg.cross_attn_placement, cfg.cross_attn_all_layers, cfg.num_layers, l)) continue;

        /* P_{l+1} = P_l + cross(RMSNorm(P_l), h) (local_encoder.c:255-272), the norm inside the query
         * projection and the sum in the epilogue of the output projection: three launches */
        blt_tensor p_rows = view_2d(p.data, num_patches * k, E);
        blt_cross_attention_weights xw;
        xw.weight_q = &s->cross_weight_q, xw.weight_k = &s->cross_weight_k, xw.weight_v = &s->cross_weight_v;
        xw.weight_proj = &s->cross_weight_proj;
        blt_tensor p_next = l == last_cross ? view_2d(patch_out->data, num_patches, patch_dim)
                                            : blt_tensor_create_uninit(arena, patch_shape, 2, BLT_DTYPE_FP32);
        blt_tensor next_rows = view_2d(p_next.data, num_patches * k, E);
        blt_cross_attention_run(&p_rows, &h, &xw, &next_rows, &cross_cfg, arena,
                                (const float *)s->cross_norm_weight.data, (const float *)p.data);
        p = p_next;
    }
    if (last_cross == cfg.num_layers) /* no cross block fired: P_0 is the result */
        blt_strided_copy_hip(BLT_BACKEND_HIP, (float *)patch_out->data, num_patches * patch_dim, (const float *)p.data,
                             num_patches * patch_dim, 1, num_patches * patch_dim);
    /* the host index arrays of the masks are consumed by the calls above (ranges are staged, dense
     * masks are built before the attention launch is issued): nothing outlives this call */
}

/*
 * blt_local_decoder_forward_ext without D_0 options and loss (reference: csrc/models/
 * local_decoder.c:233-351).  D_0 is byte_hidden_in itself; per layer B = D + cross(RMSNorm(D),
 * patch sub-tokens) where the cross block fires (norm inside the query projection, sum in the
 * output projection's epilogue: three launches), D = byte block(B) under the causal, windowed,
 * per-document mask (five launches); logits = D_final * lm_head.  A byte reads the latent the
 * paper's rule gives it (blt_patch_decoder_latent_at, the last byte of the window its own patch's
 * when trailing_closed): one sub-token group per row, so the cross mask travels as key ranges.
 */
extern "C" void blt_local_decoder_forward_ext_hip(const blt_local_decoder *model, const blt_tensor *byte_hidden_in,
                                                  const blt_tensor *patch_in, const blt_patch_info *patches,
                                                  size_t num_patches, const size_t *doc_boundaries, size_t num_docs,
                                                  int trailing_closed, blt_tensor *logits_out, blt_arena *arena) {
    BLT_REQUIRE(model != NULL && byte_hidden_in != NULL && patch_in != NULL && patches != NULL && arena != NULL,
                "blt_local_decoder_forward_ext: model, byte_hidden_in, patch_in, patches and arena cannot be NULL");
    BLT_REQUIRE(logits_out != NULL, "blt_local_decoder_forward_ext: logits_out cannot be NULL");
    BLT_REQUIRE(arena->backend == BLT_BACKEND_HIP, "blt_local_decoder_forward_ext: HIP implementation needs a device arena");
    const blt_local_decoder_config &cfg = model->config;
    const size_t E = cfg.embed_dim, V = cfg.vocab_size;
    BLT_REQUIRE(cfg.num_heads != 0 && E % cfg.num_heads == 0 && (E / cfg.num_heads) % 2 == 0,
                "blt_local_decoder_forward_ext: embed_dim / num_heads must be an even head width");
    BLT_REQUIRE(byte_hidden_in->ndim == 2 && byte_hidden_in->dtype == BLT_DTYPE_FP32 && byte_hidden_in->shape[1] == E &&
                    byte_hidden_in->backend == BLT_BACKEND_HIP,
                "blt_local_decoder_forward_ext: byte_hidden_in must be [seq_len, embed_dim] FP32");
    const size_t seq_len = byte_hidden_in->shape[0];
    BLT_REQUIRE(seq_len >= 1 && seq_len <= cfg.max_seq_len,
                "blt_local_decoder_forward_ext: seq_len must be in [1, max_seq_len]");
    BLT_REQUIRE(num_patches >= 1, "blt_local_decoder_forward_ext: num_patches must be >= 1");
    const size_t patch_dim = cfg.patch_dim == 0 ? E : cfg.patch_dim;
    BLT_REQUIRE(patch_dim % E == 0, "blt_local_decoder_forward_ext: patch_dim must be a multiple of embed_dim");
    const size_t k = patch_dim / E, half = E / cfg.num_heads / 2;
    check_2d(patch_in, num_patches, patch_dim, "blt_local_decoder_forward_ext: patch_in must be [num_patches, patch_dim] FP32");
    check_2d(logits_out, seq_len, V, "blt_local_decoder_forward_ext: logits_out must be [seq_len, vocab_size] FP32");
    check_2d(&model->lm_head_weight, E, V, "blt_local_decoder_forward_ext: lm_head_weight must be [embed_dim, vocab_size] FP32");
    check_2d(&model->rope_cos_cache, cfg.max_seq_len, half, "blt_local_decoder_forward_ext: rope_cos_cache");
    check_2d(&model->rope_sin_cache, cfg.max_seq_len, half, "blt_local_decoder_forward_ext: rope_sin_cache");
    size_t covered = 0;
    for (size_t j = 0; j < num_patches; j++) { /* patches tile [0, seq_len) (patch_pool_cpu.c:98-118) */
        BLT_REQUIRE(patches[j].start_idx == covered && patches[j].length >= 1,
                    "blt_local_decoder_forward_ext: patches must tile the window without gaps");
        covered += patches[j].length;
    }
    BLT_REQUIRE(covered == seq_len, "blt_local_decoder_forward_ext: patches must tile [0, seq_len) exactly");

    /* ---- masks (local_decoder.c:64-121): host metadata ---- */
    std::vector<size_t> byte_groups(seq_len), kv_groups(num_patches * k);
    for (size_t i = 0; i < seq_len; i++) byte_groups[i] = blt_patch_decoder_latent_at(patches, num_patches, i);
    if (trailing_closed) byte_groups[seq_len - 1] = num_patches - 1;
    for (size_t j = 0; j < num_patches * k; j++) kv_groups[j] = j / k;
    blt_mask_config local_mask, cross_mask;
    std::memset(&local_mask, 0, sizeof(local_mask));
    std::memset(&cross_mask, 0, sizeof(cross_mask));
    local_mask.seq_len_q = local_mask.seq_len_kv = seq_len;
    local_mask.sliding_window = cfg.local_window;
    local_mask.doc_boundaries = doc_boundaries;
    local_mask.num_docs = num_docs;
    local_mask.is_causal = true;
    cross_mask.seq_len_q = seq_len;
    cross_mask.seq_len_kv = num_patches * k;
    cross_mask.query_group_ids = byte_groups.data();
    cross_mask.kv_group_ids = kv_groups.data();
    cross_mask.bidirectional_within_group = true;
    blt_tensor cos_view = view_2d(model->rope_cos_cache.data, seq_len, half);
    blt_tensor sin_view = view_2d(model->rope_sin_cache.data, seq_len, half);
    blt_transformer_config layer_cfg;
    std::memset(&layer_cfg, 0, sizeof(layer_cfg));
    layer_cfg.attn_config.embed_dim = E;
    layer_cfg.attn_config.num_heads = cfg.num_heads;
    layer_cfg.attn_config.is_causal = true;
    layer_cfg.attn_config.use_rope = true;
    layer_cfg.attn_config.rope_theta = cfg.rope_theta;
    layer_cfg.attn_config.rope_cos_cache = &cos_view;
    layer_cfg.attn_config.rope_sin_cache = &sin_view;
    layer_cfg.attn_config.mask_config = &local_mask;
    layer_cfg.hidden_dim = cfg.hidden_dim;
    layer_cfg.norm_type = BLT_NORM_RMSNORM;
    layer_cfg.activation_type = BLT_ACTIVATION_SWIGLU;
    blt_cross_attention_config cross_cfg;
    std::memset(&cross_cfg, 0, sizeof(cross_cfg));
    cross_cfg.embed_dim = E;
    cross_cfg.patch_dim = patch_dim;
    cross_cfg.split_mode = k == 1 ? BLT_CROSS_ATTN_NO_SPLIT : BLT_CROSS_ATTN_SPLIT_KV;
    cross_cfg.num_heads = cfg.cross_attn_heads;
    cross_cfg.mask_config = &cross_mask;

    /* ---- layers ---- */
    const size_t byte_shape[2] = {seq_len, E};
    blt_tensor latents = view_2d(patch_in->data, num_patches * k, E);
    blt_tensor d = view_2d(byte_hidden_in->data, seq_len, E);
    for (size_t l = 0; l < cfg.num_layers; l++) {
        blt_local_layer_storage *s = &model->layers[l];
        blt_tensor b = d;
        if (blt_local_cross_attn_fires(cfg.cross_attn_placement, cfg.cross_attn_all_layers, cfg.num_layers, l)) {
            blt_cross_attention_weights xw;
            xw.weight_q = &s->cross_weight_q, xw.weight_k = &s->cross_weight_k, xw.weight_v = &s->cross_weight_v;
            xw.weight_proj = &s->cross_weight_proj;
            b = blt_tensor_create_uninit(arena, byte_shape, 2, BLT_DTYPE_FP32);
            blt_cross_attention_run(&d, &latents, &xw, &b, &cross_cfg, arena, (const float *)s->cross_norm_weight.data,
                                    (const float *)d.data);
        }
        blt_transformer_weights w;
        std::memset(&w, 0, sizeof(w));
        w.norm1_weight = &s->norm1_weight, w.norm2_weight = &s->norm2_weight;
        w.attn_qkv_w = &s->attn_qkv_w, w.attn_proj_w = &s->attn_proj_w;
        w.ffn_up_w = &s->ffn_up_w, w.ffn_gate_w = &s->ffn_gate_w, w.ffn_down_w = &s->ffn_down_w;
        blt_tensor d_next = blt_tensor_create_uninit(arena, byte_shape, 2, BLT_DTYPE_FP32);
        blt_transformer_forward_hip(&b, &w, &d_next, &layer_cfg, arena);
        d = d_next;
    }
    blt_matmul_hip(&d, &model->lm_head_weight, logits_out);
}
