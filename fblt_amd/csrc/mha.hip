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

extern "C" void blt_multihead_attention_hip(const blt_tensor *input, const blt_tensor *weight_qkv,
                                            const blt_tensor *weight_proj, blt_tensor *output,
                                            const blt_attention_config *config, blt_arena *arena) {
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
    bool causal_desc = false;
    size_t causal_off = 0, window = 0;
    if (mc != NULL) {
        BLT_REQUIRE(mc->seq_len_q == T && mc->seq_len_kv == T,
                    "blt_multihead_attention: mask_config seq_len_q/seq_len_kv must match input seq_len ");
        const bool plain = mc->doc_boundaries == NULL && mc->query_group_ids == NULL && mc->kv_group_ids == NULL;
        if (plain && mc->is_causal) {
            causal_desc = true;
            causal_off = mc->causal_offset;
            window = mc->sliding_window;
        } else if (plain && mc->sliding_window == 0) {
            /* nothing masked */
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
        p.head.q = qkv + head * hd;
        p.head.k = qkv + E + head * hd;
        p.head.v = qkv + 2 * E + head * hd;
        p.head.q_stride = p.head.k_stride = p.head.v_stride = 3 * E;
        p.head.combined = combined;
        p.head.combined_stride = E;
        p.head.combined_col_offset = head * hd;
        p.head.nq = p.head.nk = T;
        p.head.head_dim = hd;
        p.head.scale = scale;
        if (causal_desc) {
            p.mask_kind = BLT_ATTN_MASK_CAUSAL;
            p.causal_offset = causal_off;
            p.window = window;
        } else {
            p.mask_kind = BLT_ATTN_MASK_FROM_HEAD;
            p.head.mask = dense;
            p.head.is_causal = mc == NULL && config->is_causal;
        }
    }
    blt_attention_batch_hip(pr.data(), H);

    /* 3. output projection */
    std::memset(&g, 0, sizeof(g));
    g.a = combined;
    g.b = (const float *)weight_proj->data;
    g.out = (float *)output->data;
    g.m = (uint32_t)T, g.k = (uint32_t)E, g.n = (uint32_t)E;
    g.lda = g.ldb = g.ldo = (uint32_t)E;
    matmul_f32_launch(g, 0);
    HIP_CHECK_LAUNCH("blt_multihead_attention");
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
extern "C" void blt_cross_attention_forward_hip(const blt_tensor *query_in, const blt_tensor *kv_in,
                                                const blt_cross_attention_weights *weights, blt_tensor *output,
                                                const blt_cross_attention_config *config, blt_arena *arena) {
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
    {
        std::vector<uint32_t> lohi(2 * P);
        if (blt_mask_config_row_ranges(mc, lohi.data(), lohi.data() + P) == 1) {
            for (size_t i = 0; i < P; i++) /* the dense builder refuses such a mask (mask_builder_cpu.c:93) */
                BLT_REQUIRE(lohi[i] < lohi[P + i], "blt_build_attention_mask: query position has no valid key");
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
    g.m = (uint32_t)P, g.k = (uint32_t)E, g.n = (uint32_t)E;
    g.lda = g.ldb = g.ldo = (uint32_t)E;
    matmul_f32_launch(g, 0);
    HIP_CHECK_LAUNCH("blt_cross_attention_forward");
}
