/*
 * blt_multihead_attention on the device (reference: csrc/models/attention.c:
 * 130-207): packed QKV projection, rotary embedding of Q and K, masked
 * attention of every head, output projection -- three launches instead of the
 * reference's 2 + 2H + H + 1:
 *
 *   1. qkv = input * weight_qkv with the rotation of the Q and K column
 *      blocks done in the product's epilogue;
 *   2. all heads in one attention launch, the mask as a descriptor whenever
 *      the configuration is a plain causal (offset / window) mask or none,
 *      otherwise the dense mask built on the device by the mask builder;
 *   3. output = combined * weight_proj.
 *
 * Work buffers come from the caller's device arena, like the reference's.
 */
#include "blt_hip.h"
#include "blt_fatal.h"
#include "hip_check.h"
#include "launch.h"
#include "matmul.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <vector>

namespace {

void check_2d_fp32(const blt_tensor *t, size_t rows, size_t cols, const char *what) {
    BLT_REQUIRE(t != NULL && t->data != NULL && t->ndim == 2 && t->dtype == BLT_DTYPE_FP32, "%s", what);
    BLT_REQUIRE((rows == 0 || t->shape[0] == rows) && (cols == 0 || t->shape[1] == cols), "%s", what);
    BLT_REQUIRE(t->backend == BLT_BACKEND_HIP, "%s (HIP implementation called with a non-HIP tensor)", what);
}

} // namespace

namespace {

/* The attention block; with norm_w the rows of `input` are RMS-normalised first (in the packed
 * projection's own pass where that kernel takes it, csrc/models/transformer.c:60-66), with
 * residual that [seq_len, embed_dim] array is added to the projected output (transformer.c:
 * 116-117) -- the two statements a transformer block wraps around its attention. */
void mha_run(const blt_tensor *input, const blt_tensor *weight_qkv, const blt_tensor *weight_proj, blt_tensor *output,
             const blt_attention_config *config, blt_arena *arena, const float *norm_w, const float *residual) {
    BLT_REQUIRE(config != NULL && arena != NULL, "blt_multihead_attention: config and arena cannot be NULL");
    BLT_REQUIRE(arena->backend == BLT_BACKEND_HIP, "blt_multihead_attention: HIP implementation needs a device arena");
    const size_t E = config->embed_dim, H = config->num_heads;
    BLT_REQUIRE(H != 0 && E % H == 0, "blt_multihead_attention: embed_dim must be divisible by num_heads");
    check_2d_fp32(input, 0, E, "blt_multihead_attention: input must be [seq_len, embed_dim] FP32");
    const size_t T = input->shape[0];
    BLT_REQUIRE(weight_qkv != NULL && weight_qkv->ndim == 2 && weight_qkv->shape[0] == E &&
                    weight_qkv->shape[1] == 3 * E,
                "blt_multihead_attention: weight_qkv must be [embed_dim, 3*embed_dim]");
    BLT_REQUIRE(weight_proj != NULL && weight_proj->ndim == 2 && weight_proj->shape[0] == E &&
                    weight_proj->shape[1] == E,
                "blt_multihead_attention: weight_proj must be [embed_dim, embed_dim]");
    BLT_REQUIRE(weight_qkv->dtype == BLT_DTYPE_FP32 && weight_proj->dtype == BLT_DTYPE_FP32,
                "blt_multihead_attention: the HIP backend takes FP32 weights only (BF16 weights are not supported)");
    BLT_REQUIRE(weight_qkv->backend == BLT_BACKEND_HIP && weight_proj->backend == BLT_BACKEND_HIP,
                "blt_multihead_attention: HIP implementation called with a non-HIP tensor");
    check_2d_fp32(output, T, E, "blt_multihead_attention: output must be [seq_len, embed_dim] FP32");
    const size_t hd = config->head_dim != 0 ? config->head_dim : E / H;
    BLT_REQUIRE(hd * H == E, "blt_multihead_attention: head_dim * num_heads must equal embed_dim");
    if (config->use_rope) {
        BLT_REQUIRE(hd % 2 == 0, "blt_multihead_attention: RoPE requires an even head_dim");
        BLT_REQUIRE(config->rope_theta > 0.0f,
                    "blt_multihead_attention: rope_theta must be positive when use_rope is true");
    }
    if (T == 0) return;
    BLT_REQUIRE(T <= 0x7FFFFFFFu && E <= 0x3FFFFFFFu, "blt_multihead_attention: dimensions exceed 2^31-1");

    float *qkv = (float *)blt_arena_alloc(arena, T * 3 * E * sizeof(float), 64);
    float *combined = (float *)blt_arena_alloc(arena, T * E * sizeof(float), 64);

    /* rotation tables: the caller's cache, or the reference's own formula on the host, uploaded */
    const float *rope_cos = nullptr, *rope_sin = nullptr;
    if (config->use_rope) {
        const size_t half = hd / 2;
        if (config->rope_cos_cache != NULL && config->rope_sin_cache != NULL) {
            check_2d_fp32(config->rope_cos_cache, T, half,
                          "blt_multihead_attention: rope_cos_cache must be [seq_len, head_dim/2] FP32");
            check_2d_fp32(config->rope_sin_cache, T, half,
                          "blt_multihead_attention: rope_sin_cache must be [seq_len, head_dim/2] FP32");
            rope_cos = (const float *)config->rope_cos_cache->data;
            rope_sin = (const float *)config->rope_sin_cache->data;
        } else {
            blt_tensor ct, st;
            const size_t shape[2] = {T, half};
            ct = blt_tensor_create_uninit(arena, shape, 2, BLT_DTYPE_FP32);
            st = blt_tensor_create_uninit(arena, shape, 2, BLT_DTYPE_FP32);
            blt_rope_config rc;
            rc.theta = config->rope_theta;
            rc.head_dim = hd;
            blt_rope_precompute(T, &rc, &ct, &st);
            rope_cos = (const float *)ct.data;
            rope_sin = (const float *)st.data;
        }
    }

    /* 1. packed projection (+ rotation of the Q and K blocks) */
    MatmulArgs g;
    std::memset(&g, 0, sizeof(g));
    g.a = (const float *)input->data;
    g.b = (const float *)weight_qkv->data;
    g.out = qkv;
    g.m = (uint32_t)T, g.k = (uint32_t)E, g.n = (uint32_t)(3 * E);
    g.lda = (uint32_t)E, g.ldb = (uint32_t)(3 * E), g.ldo = (uint32_t)(3 * E);
    const bool fuse_rope = config->use_rope && hd % 4 == 0 && T > 32;
    if (fuse_rope) {
        g.rope_cos = rope_cos, g.rope_sin = rope_sin;
        g.rope_cols = (uint32_t)(2 * E), g.head_dim = (uint32_t)hd;
    }
    if (norm_w != nullptr) {
        if (matmul_takes_norm(g)) {
            g.norm_w = norm_w;
        } else { /* the row norm as a pass of its own */
            const size_t shape[2] = {T, E};
            blt_tensor normed = blt_tensor_create_uninit(arena, shape, 2, BLT_DTYPE_FP32);
            blt_tensor wt;
            std::memset(&wt, 0, sizeof(wt));
            wt.data = const_cast<float *>(norm_w), wt.ndim = 1, wt.shape[0] = E, wt.strides[0] = 1, wt.numel = E;
            wt.dtype = BLT_DTYPE_FP32, wt.backend = BLT_BACKEND_HIP, wt.is_view = true;
            blt_rmsnorm_forward_hip(input, &wt, &normed);
            g.a = (const float *)normed.data;
        }
    }
    matmul_f32_launch(g, 0);
    if (config->use_rope && !fuse_rope) {
        for (size_t head = 0; head < H; head++) {
            blt_rope_apply_packed_hip(qkv, 3 * E, head * hd, T, hd, rope_cos, rope_sin);
            blt_rope_apply_packed_hip(qkv, 3 * E, E + head * hd, T, hd, rope_cos, rope_sin);
        }
    }

    /* 2. every head in one launch */
    const blt_mask_config *mc = config->mask_config;
    const float *dense = nullptr;
    const uint32_t *row_lo = nullptr, *row_hi = nullptr;
    bool causal_desc = false;
    size_t causal_off = 0, window = 0;
    uint32_t row_span = 0;
    std::vector<size_t> doc_start; /* document-causal: first row of every document, then T */
    if (mc != NULL) {
        BLT_REQUIRE(mc->seq_len_q == T && mc->seq_len_kv == T,
                    "blt_multihead_attention: mask_config seq_len_q/seq_len_kv must match input seq_len ");
        const bool plain = mc->doc_boundaries == NULL && mc->query_group_ids == NULL && mc->kv_group_ids == NULL;
        const bool documents = mc->doc_boundaries != NULL && mc->num_docs > 0 && mc->query_group_ids == NULL &&
                               mc->kv_group_ids == NULL;
        if (plain && mc->is_causal) {
            causal_desc = true;
            causal_off = mc->causal_offset;
            window = mc->sliding_window;
        } else if (documents && mc->is_causal && mc->causal_offset == 0) {
            /* Document-causal (csrc/ops/mask_builder_cpu.c:10-19, 52-79: same document, not after the
             * row, inside the window): a row never looks past the start of its document, so every
             * document is a causal problem of its own over its own rows -- the shape the causal
             * kernels are built for, with no key outside the document ever touched.  Documents are
             * runs of the position -> document map the builder uses. */
            causal_desc = true;
            window = mc->sliding_window;
            size_t d = 0;
            doc_start.push_back(0);
            for (size_t pos = 0; pos < T; pos++) {
                const size_t before = d;
                while (d + 1 < mc->num_docs && pos >= mc->doc_boundaries[d]) d++;
                if (d != before && pos != 0) doc_start.push_back(pos);
            }
            doc_start.push_back(T);
        } else if (plain && mc->sliding_window == 0) {
            /* nothing masked */
        } else {
            /* document boundaries, groups: one key range per row when the allowed keys of every row
             * are contiguous (they are for the document-causal masks of the patch transformer and of
             * the local encoder, csrc/models/global_transformer.c:19-33), 8 bytes per row through
             * the pinned ring; the dense matrix from the device builder otherwise */
            std::vector<uint32_t> lohi(2 * T);
            if (blt_mask_config_row_ranges(mc, lohi.data(), lohi.data() + T) == 1) {
                for (size_t i = 0; i < T; i++) { /* the dense builder refuses such a mask (mask_builder_cpu.c:93) */
                    BLT_REQUIRE(lohi[i] < lohi[T + i], "blt_build_attention_mask: query position has no valid key");
                    row_span = std::max(row_span, lohi[T + i] - lohi[i]);
                }
                uint32_t *dev = (uint32_t *)blt_arena_alloc(arena, 2 * T * sizeof(uint32_t), 64);
                blt_upload_staged(dev, lohi.data(), 2 * T * sizeof(uint32_t));
                row_lo = dev, row_hi = dev + T;
            } else {
                blt_tensor mask_tensor;
                std::memset(&mask_tensor, 0, sizeof(mask_tensor));
                blt_build_attention_mask_hip(mc, &mask_tensor, arena);
                dense = (const float *)mask_tensor.data;
            }
        }
    }
    if (doc_start.empty()) doc_start = {0, T}; /* one problem per head over all rows */
    const size_t docs = doc_start.size() - 1;
    std::vector<blt_attention_problem> pr(docs * H);
    const float scale = 1.0f / sqrtf((float)hd);
    for (size_t t = 0; t < docs * H; t++) {
        const size_t head = t % H, first = doc_start[t / H], rows = doc_start[t / H + 1] - first;
        blt_attention_problem &p = pr[t];
        std::memset(&p, 0, sizeof(p));
        p.head.q = qkv + first * 3 * E + head * hd;
        p.head.k = qkv + first * 3 * E + E + head * hd;
        p.head.v = qkv + first * 3 * E + 2 * E + head * hd;
        p.head.q_stride = p.head.k_stride = p.head.v_stride = 3 * E;
        p.head.combined = combined + first * E;
        p.head.combined_stride = E;
        p.head.combined_col_offset = head * hd;
        p.head.nq = p.head.nk = rows;
        p.head.head_dim = hd;
        p.head.scale = scale;
        if (causal_desc) {
            p.mask_kind = BLT_ATTN_MASK_CAUSAL;
            p.causal_offset = causal_off;
            p.window = window;
        } else if (row_lo != nullptr) {
            p.mask_kind = BLT_ATTN_MASK_ROW_RANGE;
            p.row_lo = row_lo;
            p.row_hi = row_hi;
            p.row_span = row_span;
        } else {
            p.mask_kind = BLT_ATTN_MASK_FROM_HEAD;
            p.head.mask = dense;
            p.head.is_causal = mc == NULL && config->is_causal;
        }
    }
    blt_attention_batch_hip(pr.data(), pr.size());

    /* 3. output projection (+ residual) */
    std::memset(&g, 0, sizeof(g));
    g.a = combined;
    g.b = (const float *)weight_proj->data;
    g.out = (float *)output->data;
    g.residual = residual;
    g.m = (uint32_t)T, g.k = (uint32_t)E, g.n = (uint32_t)E;
    g.lda = g.ldb = g.ldo = (uint32_t)E;
    matmul_f32_launch(g, 0);
    HIP_CHECK_LAUNCH("blt_multihead_attention");
}

} // namespace

extern "C" void blt_multihead_attention_hip(const blt_tensor *input, const blt_tensor *weight_qkv,
                                            const blt_tensor *weight_proj, blt_tensor *output,
                                            const blt_attention_config *config, blt_arena *arena) {
    mha_run(input, weight_qkv, weight_proj, output, config, arena, nullptr, nullptr);
}

/*
 * blt_transformer_forward on the device (reference: csrc/models/transformer.c:97-128), the block
 * the patch transformer stacks (csrc/models/global_transformer.c:69-97 through
 * transformer_stack.c:228-248) and the local encoder runs per byte layer (csrc/models/
 * local_encoder.c:243-248): RMSNorm, attention block, residual, RMSNorm, gated feed-forward,
 * residual -- five launches where the small-output projection kernel takes the fused forms:
 *
 *   1. qkv = RMSNorm(input) * attn_qkv_w, Q and K rotated in the epilogue;
 *   2. all heads in one attention launch (mask as a descriptor or as row ranges);
 *   3. attn_residual = input + combined * attn_proj_w;
 *   4. act = silu(RMSNorm(attn_residual) * ffn_gate_w) .* (RMSNorm(attn_residual) * ffn_up_w);
 *   5. output = attn_residual + act * ffn_down_w.
 *
 * RMSNorm + SwiGLU blocks with FP32 weights (what every BLT block is, csrc/models/
 * local_common.c:99-115); LayerNorm / GELU blocks and BF16 weight copies end with a message.
 */
extern "C" void blt_transformer_forward_hip(const blt_tensor *input, const blt_transformer_weights *w, blt_tensor *output,
                                            const blt_transformer_config *config, blt_arena *arena) {
    BLT_REQUIRE(input != NULL && w != NULL && output != NULL && config != NULL,
                "Transformer: input, weights, output, and config cannot be NULL");
    BLT_REQUIRE(arena != NULL, "Transformer: arena cannot be NULL");
    BLT_REQUIRE(arena->backend == BLT_BACKEND_HIP, "Transformer: HIP implementation needs a device arena");
    BLT_REQUIRE(config->norm_type == BLT_NORM_RMSNORM && config->activation_type == BLT_ACTIVATION_SWIGLU,
                "Transformer: the HIP backend implements RMSNorm + SwiGLU blocks only");
    BLT_REQUIRE(config->use_bf16 == 0, "Transformer: the HIP backend takes FP32 weights only (BF16 copies are not supported)");
    BLT_REQUIRE(input->ndim == 2 && input->dtype == BLT_DTYPE_FP32, "Transformer: input must be a 2D FP32 tensor [seq_len, embed_dim]");
    const size_t T = input->shape[0], E = input->shape[1];
    check_2d_fp32(input, T, E, "Transformer: input must be a 2D FP32 tensor [seq_len, embed_dim]");
    check_2d_fp32(output, T, E, "Transformer: output shape must match input [seq_len, embed_dim]");
    BLT_REQUIRE(w->norm1_weight != NULL && w->norm1_weight->ndim == 1 && w->norm1_weight->shape[0] == E &&
                    w->norm1_weight->dtype == BLT_DTYPE_FP32 && w->norm1_weight->backend == BLT_BACKEND_HIP,
                "Transformer: norm1_weight must be [embed_dim] FP32");
    BLT_REQUIRE(w->norm2_weight != NULL && w->norm2_weight->ndim == 1 && w->norm2_weight->shape[0] == E &&
                    w->norm2_weight->dtype == BLT_DTYPE_FP32 && w->norm2_weight->backend == BLT_BACKEND_HIP,
                "Transformer: norm2_weight must be [embed_dim] FP32");
    BLT_REQUIRE(w->attn_qkv_w != NULL && w->attn_proj_w != NULL, "Transformer: attn_qkv_w and attn_proj_w cannot be NULL");
    BLT_REQUIRE(w->ffn_up_w != NULL && w->ffn_up_w->ndim == 2 && w->ffn_up_w->shape[0] == E,
                "Transformer: ffn_up_w must be [embed_dim, hidden_dim]");
    const size_t hidden = w->ffn_up_w->shape[1];
    BLT_REQUIRE(hidden == config->hidden_dim, "Transformer: ffn_up_w hidden dimension mismatch with config");
    check_2d_fp32(w->ffn_up_w, E, hidden, "Transformer: ffn_up_w must be FP32 or BF16");
    check_2d_fp32(w->ffn_gate_w, E, hidden, "Transformer: ffn_gate_w must be [embed_dim, hidden_dim] for SwiGLU");
    check_2d_fp32(w->ffn_down_w, hidden, E, "Transformer: ffn_down_w must be [hidden_dim, embed_dim]");
    if (T == 0) return;

    const size_t embed_shape[2] = {T, E}, hidden_shape[2] = {T, hidden};
    blt_tensor attn_residual = blt_tensor_create_uninit(arena, embed_shape, 2, BLT_DTYPE_FP32);
    mha_run(input, w->attn_qkv_w, w->attn_proj_w, &attn_residual, &config->attn_config, arena,
            (const float *)w->norm1_weight->data, (const float *)input->data);

    blt_tensor act = blt_tensor_create_uninit(arena, hidden_shape, 2, BLT_DTYPE_FP32);
    MatmulArgs g;
    std::memset(&g, 0, sizeof(g));
    g.a = (const float *)attn_residual.data;
    g.b = (const float *)w->ffn_up_w->data;
    g.out = (float *)act.data;
    g.m = (uint32_t)T, g.k = (uint32_t)E, g.n = (uint32_t)hidden;
    g.lda = (uint32_t)E, g.ldb = g.ldo = (uint32_t)hidden;
    if (matmul_takes_gated(g) && matmul_takes_norm(g)) { /* norm, up, gate and the activation in one pass */
        g.b2 = (const float *)w->ffn_gate_w->data;
        g.norm_w = (const float *)w->norm2_weight->data;
        matmul_f32_launch(g, 0);
    } else {
        blt_tensor normed = blt_tensor_create_uninit(arena, embed_shape, 2, BLT_DTYPE_FP32);
        blt_rmsnorm_forward_hip(&attn_residual, w->norm2_weight, &normed);
        g.a = (const float *)normed.data;
        if (matmul_takes_gated(g)) {
            g.b2 = (const float *)w->ffn_gate_w->data;
            matmul_f32_launch(g, 0);
        } else {
            blt_tensor gate = blt_tensor_create_uninit(arena, hidden_shape, 2, BLT_DTYPE_FP32);
            matmul_f32_launch(g, 0);
            g.b = (const float *)w->ffn_gate_w->data, g.out = (float *)gate.data;
            matmul_f32_launch(g, 0);
            blt_swiglu_forward_hip(&gate, &act, &act);
        }
    }
    std::memset(&g, 0, sizeof(g));
    g.a = (const float *)act.data;
    g.b = (const float *)w->ffn_down_w->data;
    g.out = (float *)output->data;
    g.residual = (const float *)attn_residual.data;
    g.m = (uint32_t)T, g.k = (uint32_t)hidden, g.n = (uint32_t)E;
    g.lda = (uint32_t)hidden, g.ldb = g.ldo = (uint32_t)E;
    matmul_f32_launch(g, 0);
    HIP_CHECK_LAUNCH("blt_transformer_forward");
}

/*
 * blt_cross_attention_forward on the device (reference: csrc/models/
 * cross_attention.c:101-157): patch queries against byte keys and values under
 * the block-diagonal patch mask -- four launches, where the reference runs
 * three products, a clear, the dense mask builder, the per-head core H times
 * and the output product:
 *
 *   1. q = query_in * weight_q;
 *   2. k = kv_in * weight_k and v = kv_in * weight_v in one pass over kv_in
 *      (two launches when the product is large enough for the 64x64 kernel;
 *      at small sizes 1 and 2 share one launch);
 *   3. all heads in one attention launch.  The mask configuration is reduced
 *      on the host to one key range per query row (a patch sees the bytes of
 *      its own group, which are contiguous) and uploaded as 8 bytes per row;
 *      a configuration that does not reduce falls back to the dense mask
 *      built by the device mask builder;
 *   4. output = combined * weight_proj.
 *
 * A patch that owns no byte is fatal, as in the reference's mask builder.
 */
void blt_cross_attention_run(const blt_tensor *query_in, const blt_tensor *kv_in,
                             const blt_cross_attention_weights *weights, blt_tensor *output,
                             const blt_cross_attention_config *config, blt_arena *arena, const float *norm_w,
                             const float *residual) {
    BLT_REQUIRE(config != NULL && arena != NULL, "blt_cross_attention: config and arena cannot be NULL");
    BLT_REQUIRE(config->mask_config != NULL,
                "blt_cross_attention: mask_config is required (block-diagonal patch mask)");
    BLT_REQUIRE(arena->backend == BLT_BACKEND_HIP, "blt_cross_attention: HIP implementation needs a device arena");
    BLT_REQUIRE(weights != NULL, "blt_cross_attention: weights cannot be NULL");
    const size_t E = config->embed_dim, H = config->num_heads;
    BLT_REQUIRE(H != 0 && E % H == 0, "blt_cross_attention: embed_dim must be divisible by num_heads");
    check_2d_fp32(query_in, 0, E, "blt_cross_attention: query_in must be [num_patches, embed_dim] FP32");
    check_2d_fp32(kv_in, 0, E, "blt_cross_attention: kv_in must be [seq_len, embed_dim] FP32");
    const size_t P = query_in->shape[0], T = kv_in->shape[0];
    check_2d_fp32(weights->weight_q, E, E, "blt_cross_attention: weight_q must be [embed_dim, embed_dim] FP32");
    check_2d_fp32(weights->weight_k, E, E, "blt_cross_attention: weight_k must be [embed_dim, embed_dim] FP32");
    check_2d_fp32(weights->weight_v, E, E, "blt_cross_attention: weight_v must be [embed_dim, embed_dim] FP32");
    check_2d_fp32(weights->weight_proj, E, E,
                  "blt_cross_attention: weight_proj must be [embed_dim, embed_dim] FP32");
    const size_t hd = config->head_dim != 0 ? config->head_dim : E / H;
    BLT_REQUIRE(hd * H == E, "blt_cross_attention: head_dim * num_heads must equal embed_dim");
    check_2d_fp32(output, P, E, "blt_cross_attention: output must be [num_patches, embed_dim] FP32");
    const blt_mask_config *mc = config->mask_config;
    BLT_REQUIRE(mc->seq_len_q == P && mc->seq_len_kv == T,
                "blt_cross_attention: mask_config seq_len_q/seq_len_kv must match "
                "num_patches (query rows) and seq_len (kv rows)");
    if (P == 0) return;
    BLT_REQUIRE(P <= 0x7FFFFFFFu && T <= 0x7FFFFFFFu && E <= 0x3FFFFFFFu,
                "blt_cross_attention: dimensions exceed 2^31-1");

    float *q = (float *)blt_arena_alloc(arena, P * E * sizeof(float), 64);
    float *k = (float *)blt_arena_alloc(arena, (T ? T : 1) * E * sizeof(float), 64);
    float *v = (float *)blt_arena_alloc(arena, (T ? T : 1) * E * sizeof(float), 64);
    float *combined = (float *)blt_arena_alloc(arena, P * E * sizeof(float), 64);

    /* 1, 2. projections */
    MatmulArgs g;
    std::memset(&g, 0, sizeof(g));
    g.a = (const float *)query_in->data;
    g.b = (const float *)weights->weight_q->data;
    g.out = q;
    g.m = (uint32_t)P, g.k = (uint32_t)E, g.n = (uint32_t)E;
    g.lda = g.ldb = g.ldo = (uint32_t)E;
    MatmulArgs gkv = g;
    g.norm_w = norm_w; /* the query rows only */
    if (norm_w != nullptr && !matmul_takes_norm(g)) { /* shapes the fused norm does not cover: a pass of its own */
        blt_tensor normed = blt_tensor_create_uninit(arena, query_in->shape, 2, BLT_DTYPE_FP32);
        blt_tensor wt;
        std::memset(&wt, 0, sizeof(wt));
        wt.data = const_cast<float *>(norm_w), wt.ndim = 1, wt.shape[0] = E, wt.strides[0] = 1, wt.numel = E;
        wt.dtype = BLT_DTYPE_FP32, wt.backend = BLT_BACKEND_HIP, wt.is_view = true;
        blt_rmsnorm_forward_hip(query_in, &wt, &normed);
        g.a = (const float *)normed.data;
        g.norm_w = nullptr;
    }
    gkv.a = (const float *)kv_in->data;
    gkv.b = (const float *)weights->weight_k->data;
    gkv.out = k;
    gkv.m = (uint32_t)T;
    gkv.b2 = (const float *)weights->weight_v->data;
    gkv.out2 = v;
    if (T != 0 && matmul_pair_ok(g, gkv)) {
        matmul_f32_launch_pair(g, gkv, 0); /* all three in one launch */
    } else {
        matmul_f32_launch(g, 0);
        if (T != 0 && matmul_takes_gated(gkv)) {
            matmul_f32_launch(gkv, 0);
        } else if (T != 0) {
            gkv.b2 = nullptr, gkv.out2 = nullptr;
            matmul_f32_launch(gkv, 0);
            gkv.b = (const float *)weights->weight_v->data;
            gkv.out = v;
            matmul_f32_launch(gkv, 0);
        }
    }

    /* 3. mask as row ranges when it reduces, then every head in one launch */
    const uint32_t *row_lo = nullptr, *row_hi = nullptr;
    const float *dense = nullptr;
    uint32_t row_span = 0;
    {
        std::vector<uint32_t> lohi(2 * P);
        if (blt_mask_config_row_ranges(mc, lohi.data(), lohi.data() + P) == 1) {
            for (size_t i = 0; i < P; i++) { /* the dense builder refuses such a mask (mask_builder_cpu.c:93) */
                BLT_REQUIRE(lohi[i] < lohi[P + i], "blt_build_attention_mask: query position has no valid key");
                row_span = std::max(row_span, lohi[P + i] - lohi[i]);
            }
            uint32_t *dev = (uint32_t *)blt_arena_alloc(arena, 2 * P * sizeof(uint32_t), 64);
            blt_upload_staged(dev, lohi.data(), 2 * P * sizeof(uint32_t));
            row_lo = dev, row_hi = dev + P;
        } else {
            blt_tensor mask_tensor;
            std::memset(&mask_tensor, 0, sizeof(mask_tensor));
            blt_build_attention_mask_hip(mc, &mask_tensor, arena);
            dense = (const float *)mask_tensor.data;
        }
    }
    std::vector<blt_attention_problem> pr(H);
    const float scale = 1.0f / sqrtf((float)hd);
    for (size_t head = 0; head < H; head++) {
        blt_attention_problem &p = pr[head];
        std::memset(&p, 0, sizeof(p));
        p.head.q = q + head * hd;
        p.head.k = k + head * hd;
        p.head.v = v + head * hd;
        p.head.q_stride = p.head.k_stride = p.head.v_stride = E;
        p.head.combined = combined;
        p.head.combined_stride = E;
        p.head.combined_col_offset = head * hd;
        p.head.nq = P;
        p.head.nk = T;
        p.head.head_dim = hd;
        p.head.scale = scale;
        if (row_lo != nullptr) {
            p.mask_kind = BLT_ATTN_MASK_ROW_RANGE;
            p.row_lo = row_lo;
            p.row_hi = row_hi;
            p.row_span = row_span;
        } else {
            p.mask_kind = BLT_ATTN_MASK_FROM_HEAD;
            p.head.mask = dense;
        }
    }
    blt_attention_batch_hip(pr.data(), H);

    /* 4. output projection */
    std::memset(&g, 0, sizeof(g));
    g.a = combined;
    g.b = (const float *)weights->weight_proj->data;
    g.out = (float *)output->data;
    g.residual = residual;
    g.m = (uint32_t)P, g.k = (uint32_t)E, g.n = (uint32_t)E;
    g.lda = g.ldb = g.ldo = (uint32_t)E;
    matmul_f32_launch(g, 0);
    HIP_CHECK_LAUNCH("blt_cross_attention_forward");
}

extern "C" void blt_cross_attention_forward_hip(const blt_tensor *query_in, const blt_tensor *kv_in,
                                                const blt_cross_attention_weights *weights, blt_tensor *output,
                                                const blt_cross_attention_config *config, blt_arena *arena) {
    blt_cross_attention_run(query_in, kv_in, weights, output, config, arena, nullptr, nullptr);
}
