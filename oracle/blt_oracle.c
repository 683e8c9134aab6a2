/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.  See blt_oracle.h.
 *
 * Scalar, single-threaded restatement of the reference's CPU attention path.
 * Floating-point statements keep the reference's operand order and rounding
 * points (one multiply, then one add, per term; libm expf; true division) so
 * that results agree bit for bit with the reference compiled by the same gcc.
 */
#include "blt_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ---------------------------------------------------------------------- */
/* csrc/ops/vecmath_cpu.c:6-14: float accumulator, ascending index.        */
float orc_vec_dot(const float *a, const float *b, size_t n) {
    float acc = 0.0f;
    size_t t = 0;
    while (t < n) {
        acc += a[t] * b[t];
        t++;
    }
    return acc;
}

/* csrc/ops/vecmath_cpu.c:16-53.
 * Pass 1 rewrites each entry (scale, then mask or causal cut) and tracks the
 * largest FINITE entry; pass 2 exponentiates finite entries against that
 * maximum and zeroes the rest; pass 3 divides when the sum is positive. */
void orc_softmax_masked_row_inplace(float *row, size_t row_len, size_t row_idx, bool is_causal,
                                    const float *mask_row, float scale) {
    float top = -INFINITY;
    for (size_t c = 0; c < row_len; c++) {
        float x;
        if (mask_row) {
            x = row[c] * scale + mask_row[c];
        } else if (is_causal && c > row_idx) {
            x = -INFINITY;
        } else {
            x = row[c] * scale;
        }
        row[c] = x;
        if (isfinite(x) && x > top) top = x;
    }

    float total = 0.0f;
    for (size_t c = 0; c < row_len; c++) {
        if (!isfinite(row[c])) {
            row[c] = 0.0f;
            continue;
        }
        row[c] = expf(row[c] - top);
        total += row[c];
    }

    if (total > 0.0f) {
        for (size_t c = 0; c < row_len; c++) row[c] /= total;
    }
}

/* csrc/ops/vecmath_cpu.c:55-63 */
void orc_strided_copy(float *dst, size_t dst_stride, const float *src, size_t src_stride, size_t rows,
                      size_t cols) {
    for (size_t r = 0; r < rows; r++) memcpy(dst + r * dst_stride, src + r * src_stride, cols * sizeof(float));
}

/* csrc/ops/attn_core_cpu.c:16-57.
 * All nq*nk dot products are formed (masked pairs too), each row goes through
 * the masked softmax, then the output row is cleared and accumulated in
 * ascending key order, skipping keys whose weight is exactly zero. */
int orc_attention_head_core(const blt_attention_head_args *a) {
    if (!a || !a->q || !a->k || !a->v || !a->combined) return ORC_ERR_NULL_BUFFER;
    if (!a->weights_out && !a->scores_scratch) return ORC_ERR_NO_SCORE_BUFFER;

    float *w = a->weights_out ? a->weights_out : a->scores_scratch;
    const size_t nq = a->nq, nk = a->nk, hd = a->head_dim;

    for (size_t i = 0; i < nq; i++) {
        float *wi = w + i * nk;
        const float *qi = a->q + i * a->q_stride;
        for (size_t j = 0; j < nk; j++) wi[j] = orc_vec_dot(qi, a->k + j * a->k_stride, hd);
        orc_softmax_masked_row_inplace(wi, nk, i, a->is_causal, a->mask ? a->mask + i * nk : NULL, a->scale);
    }

    for (size_t i = 0; i < nq; i++) {
        const float *wi = w + i * nk;
        float *o = a->combined + i * a->combined_stride + a->combined_col_offset;
        for (size_t d = 0; d < hd; d++) o[d] = 0.0f;
        for (size_t j = 0; j < nk; j++) {
            const float p = wi[j];
            if (p == 0.0f) continue;
            const float *vj = a->v + j * a->v_stride;
            for (size_t d = 0; d < hd; d++) o[d] += p * vj[d];
        }
    }
    return ORC_OK;
}

/* csrc/models/attention.c:199-202: heads (and sequences) are a caller loop. */
int orc_attention_head_core_many(const blt_attention_head_args *a, size_t count) {
    for (size_t t = 0; t < count; t++) {
        const int rc = orc_attention_head_core(a + t);
        if (rc != ORC_OK) return rc;
    }
    return ORC_OK;
}

/* ---------------------------------------------------------------------- */
/* csrc/ops/mask_builder_cpu.c:11-19: boundary d opens document d+1.       */
static void doc_ids_from_boundaries(const size_t *bounds, size_t num_docs, size_t len, size_t *ids) {
    size_t cur = 0;
    for (size_t p = 0; p < len; p++) {
        while (cur + 1 < num_docs && p >= bounds[cur]) cur++;
        ids[p] = cur;
    }
}

/* csrc/ops/mask_builder_cpu.c:21-95 */
int orc_build_attention_mask(const blt_mask_config *c, float *out) {
    if (!c || !out) return ORC_ERR_NULL_BUFFER;
    const size_t nq = c->seq_len_q, nk = c->seq_len_kv;
    if (nq == 0 || nk == 0) return ORC_ERR_EMPTY_SHAPE;

    const bool docs = c->doc_boundaries != NULL && c->num_docs > 0;
    const bool groups = c->query_group_ids != NULL && c->kv_group_ids != NULL;
    const size_t W = c->sliding_window;

    size_t *dq = NULL, *dk = NULL;
    if (docs) {
        dq = (size_t *)malloc(nq * sizeof(size_t));
        dk = (size_t *)malloc(nk * sizeof(size_t));
        doc_ids_from_boundaries(c->doc_boundaries, c->num_docs, nq, dq);
        doc_ids_from_boundaries(c->doc_boundaries, c->num_docs, nk, dk);
    }

    int rc = ORC_OK;
    for (size_t i = 0; i < nq && rc == ORC_OK; i++) {
        bool any = false;
        for (size_t j = 0; j < nk; j++) {
            bool ok = true;
            if (c->is_causal && j > i + c->causal_offset) ok = false;
            if (W > 0) {
                size_t dist;
                if (c->is_causal) {
                    const size_t diag = i + c->causal_offset;
                    dist = diag >= j ? diag - j : j - diag;
                } else {
                    dist = i >= j ? i - j : j - i;
                }
                if (dist >= W) ok = false;
            }
            if (docs && dq[i] != dk[j]) ok = false;
            if (groups) {
                if (c->query_group_ids[i] != c->kv_group_ids[j]) ok = false;
                else if (!c->bidirectional_within_group && j > i) ok = false;
            }
            out[i * nk + j] = ok ? 0.0f : -INFINITY;
            any = any || ok;
        }
        /* The reference aborts after filling the first row that has no key. */
        if (!any) rc = ORC_ERR_ROW_WITHOUT_KEY;
    }
    free(dq);
    free(dk);
    return rc;
}

/* csrc/ops/mask_builder_cpu.c:97-154 */
int orc_build_block_diffusion_mask(const blt_block_diffusion_config *c, float *out) {
    if (!c || !out) return ORC_ERR_NULL_BUFFER;
    const size_t S = c->seq_len, N = c->num_clean, B = c->block_size;
    if (!(S >= 1 && N >= 1 && N <= S)) return ORC_ERR_BAD_BLOCK_CONFIG;
    const bool train = c->mode == BLT_BDM_TRAIN;
    if (train) {
        if (B < 1 || (S - N) % B != 0 || !c->block_starts || c->num_blocks != (S - N) / B)
            return ORC_ERR_BAD_BLOCK_CONFIG;
        for (size_t b = 0; b < c->num_blocks; b++)
            if (c->block_starts[b] >= N) return ORC_ERR_BAD_BLOCK_CONFIG;
    }

    for (size_t i = 0; i < S; i++) {
        bool any = false;
        for (size_t j = 0; j < S; j++) {
            bool ok;
            if (i < N) {
                ok = j < N && j <= i; /* clean rows: causal over the prefix */
            } else if (!train) {
                ok = true; /* INFER: the one live block sees everything */
            } else {
                const size_t blk = (i - N) / B;
                const bool own = j >= N && (j - N) / B == blk;
                ok = j < c->block_starts[blk] || own;
            }
            out[i * S + j] = ok ? 0.0f : -INFINITY;
            any = any || ok;
        }
        if (!any) return ORC_ERR_ROW_WITHOUT_KEY;
    }
    return ORC_OK;
}

/* ---------------------------------------------------------------------- */
/* csrc/ops/patch_pool_cpu.c:98-112 */
int orc_patch_build_group_ids(const blt_patch_info *patches, size_t num_patches, size_t seq_len,
                              size_t *q_ids, size_t *kv_ids) {
    if ((!patches && num_patches) || !q_ids || !kv_ids) return ORC_ERR_NULL_BUFFER;
    for (size_t p = 0; p < num_patches; p++) q_ids[p] = p;
    size_t at = 0;
    for (size_t p = 0; p < num_patches; p++) {
        if (patches[p].start_idx != at || patches[p].length < 1) return ORC_ERR_PATCH_TILING;
        for (size_t t = 0; t < patches[p].length; t++) kv_ids[at++] = p;
    }
    return at == seq_len ? ORC_OK : ORC_ERR_PATCH_TILING;
}

/* csrc/ops/patch_pool_cpu.c:114-131: a byte is "final" when it closes a patch
 * that has a successor; final bytes read their own patch's latent, all others
 * the previous one (patch 0 reads itself); uncovered positions read the last. */
size_t orc_patch_decoder_latent_at(const blt_patch_info *patches, size_t num_patches, size_t pos) {
    if (pos < patches[0].start_idx) return 0;
    for (size_t p = 0; p < num_patches; p++) {
        const size_t lo = patches[p].start_idx;
        if (lo > pos) break;
        const size_t hi = lo + patches[p].length;
        if (pos < hi) {
            if (pos + 1 == hi && p + 1 < num_patches) return p;
            return p ? p - 1 : 0;
        }
    }
    return num_patches - 1;
}

/* csrc/ops/patch_pool_cpu.c:133-142 */
void orc_patch_expand_group_ids(const size_t *in, size_t n, size_t k, size_t *out) {
    for (size_t i = 0; i < n; i++)
        for (size_t r = 0; r < k; r++) out[i * k + r] = in[i];
}

/* ---------------------------------------------------------------------- */
size_t orc_kv_row(size_t b, size_t pos, size_t max_seq_len) { return b * max_seq_len + pos; }

size_t orc_kv_slot(size_t b, size_t pos, size_t head, size_t d, size_t max_seq_len, size_t embed_dim,
                   size_t head_dim) {
    return orc_kv_row(b, pos, max_seq_len) * embed_dim + head * head_dim + d;
}

/* csrc/infer/kv_cache.c:224-238 */
void orc_kv_self_mask(float *out, size_t n, size_t base, size_t window) {
    const size_t total = base + n;
    for (size_t r = 0; r < n; r++) {
        const size_t p = base + r;
        for (size_t j = 0; j < total; j++) {
            bool ok = j <= p;
            if (ok && window > 0 && p - j >= window) ok = false;
            out[r * total + j] = ok ? 0.0f : -INFINITY;
        }
    }
}

/* csrc/infer/kv_cache.c:343-390 (attention statements only) */
int orc_kv_attend_step(float *self_k, float *self_v, size_t max_seq_len, size_t E, size_t H, size_t b,
                       size_t base, size_t n, size_t window, const float *q_rows, const float *k_rows,
                       const float *v_rows, float *combined) {
    return orc_kv_attend_step_kind(self_k, self_v, max_seq_len, E, H, b, base, n, window, 0, q_rows, k_rows, v_rows,
                                   combined);
}

/* The same statements; block_kind != 0: every new row sees all base + n keys, the rows of a single
 * live block under the INFER rule (csrc/ops/mask_builder_cpu.c:133-135), cached prefix included. */
int orc_kv_attend_step_kind(float *self_k, float *self_v, size_t max_seq_len, size_t E, size_t H, size_t b,
                            size_t base, size_t n, size_t window, int block_kind, const float *q_rows,
                            const float *k_rows, const float *v_rows, float *combined) {
    const size_t total = base + n;
    if (total > max_seq_len) return ORC_ERR_CAPACITY;
    const size_t hd = E / H;
    float *kd = self_k + orc_kv_row(b, 0, max_seq_len) * E;
    float *vd = self_v + orc_kv_row(b, 0, max_seq_len) * E;

    /* write-through, one head slice at a time (kv_cache.c:363-365) */
    for (size_t h = 0; h < H; h++) {
        orc_strided_copy(kd + base * E + h * hd, E, k_rows + h * hd, E, n, hd);
        orc_strided_copy(vd + base * E + h * hd, E, v_rows + h * hd, E, n, hd);
    }

    float *mask = (float *)malloc(n * total * sizeof(float));
    float *scratch = (float *)malloc(n * total * sizeof(float));
    if (block_kind) {
        for (size_t e = 0; e < n * total; e++) mask[e] = 0.0f;
    } else {
        orc_kv_self_mask(mask, n, base, window);
    }
    memset(combined, 0, n * E * sizeof(float));

    int rc = ORC_OK;
    for (size_t h = 0; h < H && rc == ORC_OK; h++) {
        blt_attention_head_args a;
        memset(&a, 0, sizeof(a));
        a.q = q_rows + h * hd;
        a.q_stride = E;
        a.k = kd + h * hd;
        a.k_stride = E;
        a.v = vd + h * hd;
        a.v_stride = E;
        a.combined = combined;
        a.combined_stride = E;
        a.combined_col_offset = h * hd;
        a.scores_scratch = scratch;
        a.mask = mask;
        a.nq = n;
        a.nk = total;
        a.head_dim = hd;
        a.is_causal = false;
        a.scale = 1.0f / sqrtf((float)hd);
        rc = orc_attention_head_core(&a);
    }
    free(mask);
    free(scratch);
    return rc;
}

/* csrc/ops/reductions_cpu.c:179-197: angle = pos / theta^(2i/head_dim), in float */
int orc_rope_precompute(size_t max_seq_len, float theta, size_t head_dim, float *cos_out, float *sin_out) {
    if (head_dim % 2 != 0) return ORC_ERR_ARG;
    const size_t half = head_dim / 2;
    for (size_t pos = 0; pos < max_seq_len; pos++) {
        for (size_t i = 0; i < half; i++) {
            float freq = 1.0f / powf(theta, (float)(2 * i) / (float)head_dim);
            float angle = (float)pos * freq;
            cos_out[pos * half + i] = cosf(angle);
            sin_out[pos * half + i] = sinf(angle);
        }
    }
    return ORC_OK;
}

/* csrc/ops/reductions_cpu.c:199-229: x, out are [seq_len, num_heads, head_dim]; row t uses cos/sin row t */
void orc_rope_apply(const float *x, size_t seq_len, size_t num_heads, size_t head_dim, const float *cos_rows,
                    const float *sin_rows, float *out) {
    const size_t half = head_dim / 2;
    for (size_t t = 0; t < seq_len; t++) {
        for (size_t h = 0; h < num_heads; h++) {
            const float *xv = x + (t * num_heads + h) * head_dim;
            float *ov = out + (t * num_heads + h) * head_dim;
            const float *c = cos_rows + t * half;
            const float *s = sin_rows + t * half;
            for (size_t i = 0; i < half; i++) {
                float x0 = xv[2 * i];
                float x1 = xv[2 * i + 1];
                ov[2 * i] = x0 * c[i] - x1 * s[i];
                ov[2 * i + 1] = x1 * c[i] + x0 * s[i];
            }
        }
    }
}

/* csrc/infer/rope_gather.c:5-35: out row i = cache row positions[i] */
int orc_rope_position_gather(const float *cos_cache, const float *sin_cache, size_t cache_rows, size_t half,
                             const size_t *positions, size_t n, float *cos_out, float *sin_out) {
    for (size_t i = 0; i < n; i++)
        if (positions[i] >= cache_rows) return ORC_ERR_ARG;
    for (size_t i = 0; i < n; i++) {
        memcpy(cos_out + i * half, cos_cache + positions[i] * half, half * sizeof(float));
        memcpy(sin_out + i * half, sin_cache + positions[i] * half, half * sizeof(float));
    }
    return ORC_OK;
}

/* csrc/infer/kv_cache.c:262-271 and 343-390: the new rows arrive un-rotated
 * (q/k/v rows with their own strides, as slices of the packed QKV rows); per
 * head Q and K are copied out, rotated at positions base..base+n-1, Q is
 * collected, rotated K and plain V are written through, then the heads attend. */
int orc_kv_rope_attend_step(float *self_k, float *self_v, size_t max_seq_len, size_t E, size_t H, size_t b,
                            size_t base, size_t n, size_t window, const float *q_rows, size_t q_stride,
                            const float *k_rows, size_t k_stride, const float *v_rows, size_t v_stride,
                            const float *cos_cache, const float *sin_cache, size_t cache_rows, float *combined) {
    return orc_kv_rope_attend_step_kind(self_k, self_v, max_seq_len, E, H, b, base, n, window, 0, NULL, q_rows,
                                        q_stride, k_rows, k_stride, v_rows, v_stride, cos_cache, sin_cache,
                                        cache_rows, combined);
}

/* The same with the step kind of orc_kv_attend_step_kind and, when row_positions is given, the
 * rotary position of every new row taken from it (block rows carry their own positions,
 * csrc/models/block_diffusion.c:148-157) instead of base + r. */
int orc_kv_rope_attend_step_kind(float *self_k, float *self_v, size_t max_seq_len, size_t E, size_t H, size_t b,
                                 size_t base, size_t n, size_t window, int block_kind, const size_t *row_positions,
                                 const float *q_rows, size_t q_stride, const float *k_rows, size_t k_stride,
                                 const float *v_rows, size_t v_stride, const float *cos_cache,
                                 const float *sin_cache, size_t cache_rows, float *combined) {
    if (base + n > max_seq_len) return ORC_ERR_CAPACITY;
    const size_t hd = E / H, half = hd / 2;
    size_t *positions = (size_t *)malloc(n * sizeof(size_t));
    float *rc = (float *)malloc(n * half * sizeof(float));
    float *rs = (float *)malloc(n * half * sizeof(float));
    float *q_head = (float *)malloc(n * hd * sizeof(float));
    float *k_head = (float *)malloc(n * hd * sizeof(float));
    float *q_rot = (float *)malloc(n * hd * sizeof(float));
    float *k_rot = (float *)malloc(n * hd * sizeof(float));
    float *q_full = (float *)malloc(n * E * sizeof(float));
    float *k_full = (float *)malloc(n * E * sizeof(float));
    float *v_full = (float *)malloc(n * E * sizeof(float));
    for (size_t r = 0; r < n; r++) positions[r] = row_positions ? row_positions[r] : base + r;
    int rcode = orc_rope_position_gather(cos_cache, sin_cache, cache_rows, half, positions, n, rc, rs);
    if (rcode == ORC_OK) {
        for (size_t h = 0; h < H; h++) {
            orc_strided_copy(q_head, hd, q_rows + h * hd, q_stride, n, hd);
            orc_strided_copy(k_head, hd, k_rows + h * hd, k_stride, n, hd);
            orc_rope_apply(q_head, n, 1, hd, rc, rs, q_rot);
            orc_rope_apply(k_head, n, 1, hd, rc, rs, k_rot);
            orc_strided_copy(q_full + h * hd, E, q_rot, hd, n, hd);
            orc_strided_copy(k_full + h * hd, E, k_rot, hd, n, hd);
            orc_strided_copy(v_full + h * hd, E, v_rows + h * hd, v_stride, n, hd);
        }
        rcode = orc_kv_attend_step_kind(self_k, self_v, max_seq_len, E, H, b, base, n, window, block_kind, q_full,
                                        k_full, v_full, combined);
    }
    free(positions), free(rc), free(rs), free(q_head), free(k_head), free(q_rot), free(k_rot);
    free(q_full), free(k_full), free(v_full);
    return rcode;
}

/* csrc/ops/linalg_cpu.c:8-18 */
void orc_matmul(const float *a, const float *b, float *out, size_t m, size_t k, size_t n) {
    for (size_t row = 0; row < m; ++row) {
        for (size_t col = 0; col < n; ++col) {
            float sum = 0.0f;
            for (size_t inner = 0; inner < k; ++inner) sum += a[row * k + inner] * b[inner * n + col];
            out[row * n + col] = sum;
        }
    }
}

/* csrc/core/backend.c:331-344: in-place rotation of one head's column block of packed rows */
void orc_rope_apply_packed(float *qkv, size_t qkv_stride, size_t head_offset, size_t seq_len, size_t head_dim,
                           const float *cos_rows, const float *sin_rows) {
    const size_t half = head_dim / 2;
    for (size_t t = 0; t < seq_len; t++) {
        float *base = qkv + t * qkv_stride + head_offset;
        const float *c = cos_rows + t * half;
        const float *s = sin_rows + t * half;
        for (size_t i = 0; i < half; i++) {
            float x0 = base[2 * i];
            float x1 = base[2 * i + 1];
            base[2 * i] = x0 * c[i] - x1 * s[i];
            base[2 * i + 1] = x1 * c[i] + x0 * s[i];
        }
    }
}

/* csrc/models/attention.c:130-207 (BLT_FLASH_ATTN unset): packed projection,
 * rotation of the Q and K blocks head by head (76-90), dense mask from the
 * mask configuration when there is one (58-74), one core call per head with
 * weights_out (92-128), output projection. */
int orc_multihead_attention(const float *input, const float *weight_qkv, const float *weight_proj, float *output,
                            size_t seq_len, size_t embed_dim, size_t num_heads, int is_causal, int use_rope,
                            float rope_theta, const float *rope_cos_cache, const float *rope_sin_cache,
                            const blt_mask_config *mask_config) {
    if (num_heads == 0 || embed_dim % num_heads != 0) return ORC_ERR_ARG;
    const size_t hd = embed_dim / num_heads, half = hd / 2, E = embed_dim;
    if (use_rope && (hd % 2 != 0 || !(rope_theta > 0.0f))) return ORC_ERR_ARG;
    float *qkv = (float *)malloc(seq_len * 3 * E * sizeof(float));
    float *combined = (float *)calloc(seq_len * E, sizeof(float));
    float *scores = (float *)malloc(seq_len * seq_len * sizeof(float));
    float *mask = NULL, *cs = NULL, *sn = NULL;
    int rc = ORC_OK;
    orc_matmul(input, weight_qkv, qkv, seq_len, E, 3 * E);
    if (use_rope) {
        const float *c = rope_cos_cache, *s = rope_sin_cache;
        if (!(c && s)) {
            cs = (float *)malloc(seq_len * half * sizeof(float));
            sn = (float *)malloc(seq_len * half * sizeof(float));
            rc = orc_rope_precompute(seq_len, rope_theta, hd, cs, sn);
            c = cs, s = sn;
        }
        for (size_t h = 0; h < num_heads && rc == ORC_OK; h++) {
            orc_rope_apply_packed(qkv, 3 * E, h * hd, seq_len, hd, c, s);
            orc_rope_apply_packed(qkv, 3 * E, E + h * hd, seq_len, hd, c, s);
        }
    }
    if (rc == ORC_OK && mask_config != NULL) {
        if (mask_config->seq_len_q != seq_len || mask_config->seq_len_kv != seq_len) rc = ORC_ERR_ARG;
        else {
            mask = (float *)malloc(seq_len * seq_len * sizeof(float));
            rc = orc_build_attention_mask(mask_config, mask);
        }
    }
    for (size_t h = 0; h < num_heads && rc == ORC_OK; h++) {
        blt_attention_head_args a;
        memset(&a, 0, sizeof(a));
        a.q = qkv + h * hd;
        a.k = qkv + E + h * hd;
        a.v = qkv + 2 * E + h * hd;
        a.q_stride = a.k_stride = a.v_stride = 3 * E;
        a.combined = combined;
        a.combined_stride = E;
        a.combined_col_offset = h * hd;
        a.weights_out = scores;
        a.mask = mask;
        a.nq = a.nk = seq_len;
        a.head_dim = hd;
        a.is_causal = is_causal != 0;
        a.scale = 1.0f / sqrtf((float)hd);
        rc = orc_attention_head_core(&a);
    }
    if (rc == ORC_OK) orc_matmul(combined, weight_proj, output, seq_len, E, E);
    free(qkv), free(combined), free(scores), free(mask), free(cs), free(sn);
    return rc;
}

/* csrc/ops/reductions_cpu.c:325-352 */
void orc_rmsnorm_forward(const float *x, const float *weight, float *out, size_t rows, size_t dim) {
    for (size_t i = 0; i < rows; i++) {
        const float *row = x + i * dim;
        float *out_row = out + i * dim;
        float sumsq = 0.0f;
        for (size_t j = 0; j < dim; j++) sumsq += row[j] * row[j];
        float mean_sq = sumsq / (float)dim;
        float inv_rms = 1.0f / sqrtf(mean_sq + 1e-6f);
        for (size_t j = 0; j < dim; j++) out_row[j] = row[j] * inv_rms * weight[j];
    }
}

/* csrc/ops/elementwise_cpu.c:9-18 */
void orc_add(const float *a, const float *b, float *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = a[i] + b[i];
}

/* csrc/ops/elementwise_cpu.c:86-99 */
void orc_swiglu_forward(const float *gate, const float *up, float *out, size_t n) {
    for (size_t i = 0; i < n; i++) {
        float gv = gate[i];
        float silu = gv / (1.0f + expf(-gv));
        out[i] = silu * up[i];
    }
}

/* One decoder layer of csrc/infer/kv_cache.c:326-414 for the n new rows of
 * sequence b, without the optional cross-attention: rows_in [n, E] is the
 * layer input (`b` in the reference's code), rows_out the layer output. */
int orc_kv_decode_layer(float *self_k, float *self_v, size_t max_seq_len, size_t E, size_t H, size_t b, size_t base,
                        size_t n, size_t window, const float *norm1_w, const float *qkv_w, const float *proj_w,
                        const float *norm2_w, const float *up_w, const float *gate_w, const float *down_w,
                        size_t hidden, const float *cos_cache, const float *sin_cache, size_t cache_rows,
                        const float *rows_in, float *rows_out) {
    return orc_kv_decode_layer_kind(self_k, self_v, max_seq_len, E, H, b, base, n, window, 0, NULL, norm1_w, qkv_w,
                                    proj_w, norm2_w, up_w, gate_w, down_w, hidden, cos_cache, sin_cache, cache_rows,
                                    rows_in, rows_out);
}

int orc_kv_decode_layer_kind(float *self_k, float *self_v, size_t max_seq_len, size_t E, size_t H, size_t b,
                             size_t base, size_t n, size_t window, int block_kind, const size_t *row_positions,
                             const float *norm1_w, const float *qkv_w, const float *proj_w, const float *norm2_w,
                             const float *up_w, const float *gate_w, const float *down_w, size_t hidden,
                             const float *cos_cache, const float *sin_cache, size_t cache_rows, const float *rows_in,
                             float *rows_out) {
    float *normed = (float *)malloc(n * E * sizeof(float));
    float *qkv = (float *)malloc(n * 3 * E * sizeof(float));
    float *combined = (float *)malloc(n * E * sizeof(float));
    float *attn_out = (float *)malloc(n * E * sizeof(float));
    float *resid1 = (float *)malloc(n * E * sizeof(float));
    float *up = (float *)malloc(n * hidden * sizeof(float));
    float *gate = (float *)malloc(n * hidden * sizeof(float));
    float *act = (float *)malloc(n * hidden * sizeof(float));
    orc_rmsnorm_forward(rows_in, norm1_w, normed, n, E);
    orc_matmul(normed, qkv_w, qkv, n, E, 3 * E);
    int rc = orc_kv_rope_attend_step_kind(self_k, self_v, max_seq_len, E, H, b, base, n, window, block_kind,
                                          row_positions, qkv, 3 * E, qkv + E, 3 * E, qkv + 2 * E, 3 * E, cos_cache,
                                          sin_cache, cache_rows, combined);
    if (rc == ORC_OK) {
        orc_matmul(combined, proj_w, attn_out, n, E, E);
        orc_add(rows_in, attn_out, resid1, n * E);
        orc_rmsnorm_forward(resid1, norm2_w, normed, n, E);
        orc_matmul(normed, up_w, up, n, E, hidden);
        orc_matmul(normed, gate_w, gate, n, E, hidden);
        orc_swiglu_forward(gate, up, act, n * hidden);
        orc_matmul(act, down_w, attn_out, n, hidden, E);
        orc_add(resid1, attn_out, rows_out, n * E);
    }
    free(normed), free(qkv), free(combined), free(attn_out), free(resid1), free(up), free(gate), free(act);
    return rc;
}

/* csrc/models/cross_attention.c:101-157: Q from query_in, K and V from kv_in,
 * dense mask from the (required) mask configuration, one core call per head
 * with weights_out, output projection; no positional embedding, no residual. */
int orc_cross_attention_forward(const float *query_in, const float *kv_in, const float *wq, const float *wk,
                                const float *wv, const float *wproj, float *output, size_t num_patches,
                                size_t seq_len, size_t embed_dim, size_t num_heads,
                                const blt_mask_config *mask_config) {
    if (mask_config == NULL || num_heads == 0 || embed_dim % num_heads != 0) return ORC_ERR_ARG;
    if (mask_config->seq_len_q != num_patches || mask_config->seq_len_kv != seq_len) return ORC_ERR_ARG;
    const size_t E = embed_dim, hd = E / num_heads;
    float *q = (float *)malloc(num_patches * E * sizeof(float));
    float *k = (float *)malloc(seq_len * E * sizeof(float));
    float *v = (float *)malloc(seq_len * E * sizeof(float));
    float *combined = (float *)calloc(num_patches * E, sizeof(float));
    float *scores = (float *)malloc(num_patches * seq_len * sizeof(float));
    float *mask = (float *)malloc(num_patches * seq_len * sizeof(float));
    orc_matmul(query_in, wq, q, num_patches, E, E);
    orc_matmul(kv_in, wk, k, seq_len, E, E);
    orc_matmul(kv_in, wv, v, seq_len, E, E);
    int rc = orc_build_attention_mask(mask_config, mask);
    for (size_t h = 0; h < num_heads && rc == ORC_OK; h++) {
        blt_attention_head_args a;
        memset(&a, 0, sizeof(a));
        a.q = q + h * hd, a.k = k + h * hd, a.v = v + h * hd;
        a.q_stride = a.k_stride = a.v_stride = E;
        a.combined = combined;
        a.combined_stride = E;
        a.combined_col_offset = h * hd;
        a.weights_out = scores;
        a.mask = mask;
        a.nq = num_patches;
        a.nk = seq_len;
        a.head_dim = hd;
        a.is_causal = false;
        a.scale = 1.0f / sqrtf((float)hd);
        rc = orc_attention_head_core(&a);
    }
    if (rc == ORC_OK) orc_matmul(combined, wproj, output, num_patches, E, E);
    free(q), free(k), free(v), free(combined), free(scores), free(mask);
    return rc;
}

/* csrc/models/local_common.c:49-64 */
int orc_local_cross_attn_fires(int placement, int cross_attn_all_layers, size_t num_layers, size_t layer) {
    switch (placement) {
    case BLT_XATTN_NONE: return 0;
    case BLT_XATTN_LAST: return layer + 1 == num_layers;
    case BLT_XATTN_ALL: return 1;
    case BLT_XATTN_FIRST: return layer == 0;
    default: return cross_attn_all_layers || layer + 1 == num_layers;
    }
}

/* csrc/infer/kv_cache.c:112-159: K and V of the sub-tokens of patches
 * [from_patch, num_patches) of sequence `b`, for every layer whose cross block
 * fires, written in place into the tier-2 slabs. */
int orc_kv_cache_refresh_cross(blt_kv_cache *cache, size_t b, const float *patch_in, size_t num_patches,
                               size_t from_patch) {
    const blt_local_decoder *dec = cache->decoder;
    const size_t E = cache->embed_dim, L = dec->config.num_layers;
    if (num_patches < 1 || from_patch >= num_patches || num_patches * cache->k > cache->max_subtokens)
        return ORC_ERR_ARG;
    const size_t first = from_patch * cache->k, count = (num_patches - from_patch) * cache->k;
    for (size_t l = 0; l < L; l++) {
        if (!orc_local_cross_attn_fires(dec->config.cross_attn_placement, dec->config.cross_attn_all_layers, L, l))
            continue;
        const blt_local_layer_storage *s = &dec->layers[l];
        const size_t row0 = b * cache->max_subtokens + first;
        orc_matmul(patch_in + first * E, (const float *)s->cross_weight_k.data,
                   (float *)cache->cross_k[l].data + row0 * E, count, E, E);
        orc_matmul(patch_in + first * E, (const float *)s->cross_weight_v.data,
                   (float *)cache->cross_v[l].data + row0 * E, count, E, E);
    }
    return ORC_OK;
}

/* csrc/infer/kv_cache.c:303-341: the cross block in front of a decoder layer
 * for the n new rows of sequence b: RMSNorm, Q projection, every head over
 * the total_sub cached sub-tokens under the one-hot group mask
 * (kv_cache.c:240-251), output projection, residual. */
int orc_kv_cross_block(const float *cross_k, const float *cross_v, size_t max_subtokens, size_t E, size_t heads,
                       size_t b, size_t total_sub, size_t k_split, const size_t *q_group, size_t n,
                       const float *norm_w, const float *wq, const float *wproj, const float *rows_in,
                       float *rows_out) {
    const size_t xhd = E / heads;
    float *normed = (float *)malloc(n * E * sizeof(float));
    float *q = (float *)malloc(n * E * sizeof(float));
    float *combined = (float *)calloc(n * E, sizeof(float));
    float *out = (float *)malloc(n * E * sizeof(float));
    float *mask = (float *)malloc(n * total_sub * sizeof(float));
    float *scratch = (float *)malloc(n * total_sub * sizeof(float));
    for (size_t r = 0; r < n; r++)
        for (size_t j = 0; j < total_sub; j++) mask[r * total_sub + j] = (j / k_split == q_group[r]) ? 0.0f : -INFINITY;
    orc_rmsnorm_forward(rows_in, norm_w, normed, n, E);
    orc_matmul(normed, wq, q, n, E, E);
    int rc = ORC_OK;
    for (size_t h = 0; h < heads && rc == ORC_OK; h++) {
        blt_attention_head_args a;
        memset(&a, 0, sizeof(a));
        a.q = q + h * xhd;
        a.k = cross_k + b * max_subtokens * E + h * xhd;
        a.v = cross_v + b * max_subtokens * E + h * xhd;
        a.q_stride = a.k_stride = a.v_stride = E;
        a.combined = combined;
        a.combined_stride = E;
        a.combined_col_offset = h * xhd;
        a.scores_scratch = scratch;
        a.mask = mask;
        a.nq = n;
        a.nk = total_sub;
        a.head_dim = xhd;
        a.scale = 1.0f / sqrtf((float)xhd);
        rc = orc_attention_head_core(&a);
    }
    if (rc == ORC_OK) {
        orc_matmul(combined, wproj, out, n, E, E);
        orc_add(rows_in, out, rows_out, n * E);
    }
    free(normed), free(q), free(combined), free(out), free(mask), free(scratch);
    return rc;
}

/* csrc/infer/kv_cache.c:161-416 for sequence `b` of a (possibly batched)
 * cache whose valid length is `base`: group of every new row by the decoder
 * latent rule (199-213), then per layer the cross block where it fires and the
 * self-attention / feed-forward layer, then the LM head.  The caller advances
 * the sequence's length. */
int orc_kv_decode_step(blt_kv_cache *cache, size_t b, size_t base, const blt_patch_info *patches,
                       size_t num_patches, const float *d0_rows, size_t n, int trailing_closed,
                       float *logits_out) {
    const blt_local_decoder *dec = cache->decoder;
    const blt_local_decoder_config *cfg = &dec->config;
    const size_t E = cache->embed_dim, L = cfg->num_layers, H = cfg->num_heads, XH = cfg->cross_attn_heads;
    if (n < 1 || num_patches < 1) return ORC_ERR_ARG;
    if (base + n > cache->max_seq_len || num_patches * cache->k > cache->max_subtokens) return ORC_ERR_CAPACITY;
    size_t *q_group = (size_t *)malloc(n * sizeof(size_t));
    for (size_t r = 0; r < n; r++) q_group[r] = orc_patch_decoder_latent_at(patches, num_patches, base + r);
    if (trailing_closed) q_group[n - 1] = num_patches - 1;
    float *cur = (float *)malloc(n * E * sizeof(float));
    float *mid = (float *)malloc(n * E * sizeof(float));
    memcpy(cur, d0_rows, n * E * sizeof(float));
    int rc = ORC_OK;
    for (size_t l = 0; l < L && rc == ORC_OK; l++) {
        const blt_local_layer_storage *s = &dec->layers[l];
        const float *in = cur;
        if (orc_local_cross_attn_fires(cfg->cross_attn_placement, cfg->cross_attn_all_layers, L, l)) {
            rc = orc_kv_cross_block((const float *)cache->cross_k[l].data, (const float *)cache->cross_v[l].data,
                                    cache->max_subtokens, E, XH, b, num_patches * cache->k, cache->k, q_group, n,
                                    (const float *)s->cross_norm_weight.data, (const float *)s->cross_weight_q.data,
                                    (const float *)s->cross_weight_proj.data, cur, mid);
            in = mid;
        }
        if (rc != ORC_OK) break;
        rc = orc_kv_decode_layer((float *)cache->self_k[l].data, (float *)cache->self_v[l].data, cache->max_seq_len,
                                 E, H, b, base, n, cfg->local_window, (const float *)s->norm1_weight.data,
                                 (const float *)s->attn_qkv_w.data, (const float *)s->attn_proj_w.data,
                                 (const float *)s->norm2_weight.data, (const float *)s->ffn_up_w.data,
                                 (const float *)s->ffn_gate_w.data, (const float *)s->ffn_down_w.data,
                                 s->ffn_up_w.shape[1], (const float *)dec->rope_cos_cache.data,
                                 (const float *)dec->rope_sin_cache.data, dec->rope_cos_cache.shape[0], in, cur);
    }
    if (rc == ORC_OK) orc_matmul(cur, (const float *)dec->lm_head_weight.data, logits_out, n, E, cfg->vocab_size);
    free(q_group), free(cur), free(mid);
    return rc;
}

/* D_0 rows of the block section (csrc/models/block_diffusion.c:137-146): zeros, or row tokens[r] of
 * the learned table (csrc/ops/gather_scatter_cpu.c:7-29) */
static int orc_block_d0_rows(const blt_local_decoder *dec, const blt_block_batch *batch, int d0_mode, float *rows) {
    const size_t E = dec->config.embed_dim, R = batch->n_block_rows;
    memset(rows, 0, R * E * sizeof(float));
    if (d0_mode != BLT_D0_LEARNED) return ORC_OK;
    const blt_tensor *table = &dec->d0_embed_weight;
    if (table->data == NULL || table->ndim != 2 || table->shape[1] != E || batch->tokens == NULL) return ORC_ERR_ARG;
    for (size_t r = 0; r < R; r++) {
        if (batch->tokens[r] >= table->shape[0]) return ORC_ERR_ARG;
        memcpy(rows + r * E, (const float *)table->data + (size_t)batch->tokens[r] * E, E * sizeof(float));
    }
    return ORC_OK;
}


/* csrc/models/local_decoder.c:233-351 with d0_opts == NULL and loss_out == NULL: D_0 is the encoder's
 * byte states; per layer the cross block where it fires -- queries RMSNorm(D), keys and values the
 * k sub-tokens of every patch, byte i reading the latent blt_patch_decoder_latent_at assigns it
 * (:75-88), the last byte its own patch when trailing_closed -- then the byte transformer block
 * under the causal / window / document mask (:96-102); logits = D_L * lm_head (:340).
 * doc_boundaries in the mask builder's convention (entry d starts document d + 1). */
int orc_local_decoder_forward(const blt_local_decoder *dec, const float *byte_hidden, size_t seq_len,
                              const float *patch_in, const blt_patch_info *patches, size_t num_patches,
                              const size_t *doc_boundaries, size_t num_docs, int trailing_closed, float *logits_out) {
    const blt_local_decoder_config *cfg = &dec->config;
    const size_t E = cfg->embed_dim, V = cfg->vocab_size, L = cfg->num_layers;
    const size_t pdim = cfg->patch_dim ? cfg->patch_dim : E, k = pdim / E;
    if (seq_len < 2 || seq_len > cfg->max_seq_len || num_patches < 1 || k < 1 || pdim % E != 0) return ORC_ERR_ARG;

    size_t *q_ids = (size_t *)malloc(seq_len * sizeof(size_t));
    size_t *kv_ids = (size_t *)malloc(num_patches * k * sizeof(size_t));
    for (size_t i = 0; i < seq_len; i++) q_ids[i] = orc_patch_decoder_latent_at(patches, num_patches, i);
    if (trailing_closed) q_ids[seq_len - 1] = num_patches - 1;
    for (size_t p = 0; p < num_patches; p++)
        for (size_t s2 = 0; s2 < k; s2++) kv_ids[p * k + s2] = p;

    blt_mask_config local, cross;
    memset(&local, 0, sizeof(local));
    memset(&cross, 0, sizeof(cross));
    local.seq_len_q = local.seq_len_kv = seq_len;
    local.sliding_window = cfg->local_window;
    local.doc_boundaries = doc_boundaries, local.num_docs = num_docs;
    local.is_causal = true;
    cross.seq_len_q = seq_len, cross.seq_len_kv = num_patches * k;
    cross.query_group_ids = q_ids, cross.kv_group_ids = kv_ids;
    cross.bidirectional_within_group = true;

    float *cur = (float *)malloc(seq_len * E * sizeof(float));
    float *next = (float *)malloc(seq_len * E * sizeof(float));
    float *normed = (float *)malloc(seq_len * E * sizeof(float));
    float *tmp = (float *)malloc(seq_len * E * sizeof(float));
    float *mid = (float *)malloc(seq_len * E * sizeof(float));
    memcpy(cur, byte_hidden, seq_len * E * sizeof(float));
    int rc = ORC_OK;
    for (size_t l = 0; l < L && rc == ORC_OK; l++) {
        const blt_local_layer_storage *s = &dec->layers[l];
        const float *b_in = cur;
        if (orc_local_cross_attn_fires(cfg->cross_attn_placement, cfg->cross_attn_all_layers, L, l)) {
            orc_rmsnorm_forward(cur, (const float *)s->cross_norm_weight.data, normed, seq_len, E);
            rc = orc_cross_attention_forward(normed, patch_in, (const float *)s->cross_weight_q.data,
                                             (const float *)s->cross_weight_k.data, (const float *)s->cross_weight_v.data,
                                             (const float *)s->cross_weight_proj.data, tmp, seq_len, num_patches * k, E,
                                             cfg->cross_attn_heads, &cross);
            if (rc != ORC_OK) break;
            orc_add(cur, tmp, mid, seq_len * E);
            b_in = mid;
        }
        rc = orc_transformer_forward(b_in, (const float *)s->norm1_weight.data, (const float *)s->attn_qkv_w.data,
                                     (const float *)s->attn_proj_w.data, (const float *)s->norm2_weight.data,
                                     (const float *)s->ffn_up_w.data, (const float *)s->ffn_gate_w.data,
                                     (const float *)s->ffn_down_w.data, next, seq_len, E, s->ffn_up_w.shape[1],
                                     cfg->num_heads, 1, 1, cfg->rope_theta, (const float *)dec->rope_cos_cache.data,
                                     (const float *)dec->rope_sin_cache.data, &local);
        float *t = cur;
        cur = next, next = t;
    }
    if (rc == ORC_OK) orc_matmul(cur, (const float *)dec->lm_head_weight.data, logits_out, seq_len, E, V);
    free(q_ids), free(kv_ids), free(cur), free(next), free(normed), free(tmp), free(mid);
    return rc;
}

/* csrc/models/block_diffusion.c:776-795: the inference-mode forward over [clean prefix ; block
 * rows] as the reference computes it -- all S = N + R rows densely: context 110-204 (D_0, gathered
 * rotary rows, group ids, the S x S INFER mask), layers 336-398 (cross block where it fires,
 * self-attention 246-323 with one core call per head against the mask, feed-forward), LM head.
 * byte_hidden is [N, E], patch_in [num_patches, patch_dim], logits_out [S, vocab]. */
int orc_local_decoder_forward_diffusion_infer(const blt_local_decoder *dec, const float *byte_hidden,
                                              const float *patch_in, const blt_patch_info *patches,
                                              size_t num_patches, const blt_block_batch *batch, int d0_mode,
                                              float *logits_out) {
    const blt_local_decoder_config *cfg = &dec->config;
    const size_t N = batch->num_clean, R = batch->n_block_rows, S = N + R;
    const size_t E = cfg->embed_dim, V = cfg->vocab_size, H = cfg->num_heads, XH = cfg->cross_attn_heads;
    const size_t hd = E / H, half = hd / 2, L = cfg->num_layers;
    const size_t pdim = cfg->patch_dim ? cfg->patch_dim : E, k = pdim / E;
    if (hd == 0 || hd % 2 != 0 || N < 1 || num_patches < 1) return ORC_ERR_ARG;
    if (S < 2 || S > cfg->max_seq_len) return ORC_ERR_ARG;

    float *cur = (float *)calloc(S * E, sizeof(float));
    float *next = (float *)malloc(S * E * sizeof(float));
    memcpy(cur, byte_hidden, N * E * sizeof(float));
    int rc = orc_block_d0_rows(dec, batch, d0_mode, cur + N * E);

    size_t *positions = (size_t *)malloc(S * sizeof(size_t));
    for (size_t i = 0; i < N; i++) positions[i] = i;
    for (size_t r = 0; r < R; r++) positions[N + r] = batch->positions[r];
    float *rope_c = (float *)malloc(S * half * sizeof(float));
    float *rope_s = (float *)malloc(S * half * sizeof(float));
    if (rc == ORC_OK)
        rc = orc_rope_position_gather((const float *)dec->rope_cos_cache.data, (const float *)dec->rope_sin_cache.data,
                                      dec->rope_cos_cache.shape[0], half, positions, S, rope_c, rope_s);

    size_t *q_ids = (size_t *)malloc(S * sizeof(size_t));
    size_t *kv_ids = (size_t *)malloc(num_patches * k * sizeof(size_t));
    for (size_t i = 0; i < N; i++) q_ids[i] = orc_patch_decoder_latent_at(patches, num_patches, i);
    if (batch->trailing_closed) q_ids[N - 1] = num_patches - 1;
    for (size_t r = 0; r < R; r++) q_ids[N + r] = batch->groups[r];
    for (size_t p = 0; p < num_patches; p++)
        for (size_t s2 = 0; s2 < k; s2++) kv_ids[p * k + s2] = p;

    float *mask = (float *)malloc(S * S * sizeof(float));
    float *weights = (float *)malloc(S * S * sizeof(float));
    if (rc == ORC_OK) {
        blt_block_diffusion_config mc;
        memset(&mc, 0, sizeof(mc));
        mc.mode = BLT_BDM_INFER, mc.seq_len = S, mc.num_clean = N, mc.block_size = batch->block_size;
        mc.num_blocks = batch->num_blocks; /* the INFER rule reads neither block_starts nor block_size */
        rc = orc_build_block_diffusion_mask(&mc, mask);
    }

    const size_t hidden = L ? dec->layers[0].ffn_up_w.shape[1] : 0;
    float *normed = (float *)malloc(S * E * sizeof(float));
    float *mid = (float *)malloc(S * E * sizeof(float));
    float *qkv = (float *)malloc(S * 3 * E * sizeof(float));
    float *combined = (float *)malloc(S * E * sizeof(float));
    float *tmp = (float *)malloc(S * E * sizeof(float));
    float *resid1 = (float *)malloc(S * E * sizeof(float));
    float *up = (float *)malloc(S * (hidden ? hidden : 1) * sizeof(float));
    float *gate = (float *)malloc(S * (hidden ? hidden : 1) * sizeof(float));
    float *act = (float *)malloc(S * (hidden ? hidden : 1) * sizeof(float));

    for (size_t l = 0; l < L && rc == ORC_OK; l++) {
        const blt_local_layer_storage *s = &dec->layers[l];
        const float *b_in = cur;
        if (orc_local_cross_attn_fires(cfg->cross_attn_placement, cfg->cross_attn_all_layers, L, l)) {
            blt_mask_config xm;
            memset(&xm, 0, sizeof(xm));
            xm.seq_len_q = S, xm.seq_len_kv = num_patches * k;
            xm.query_group_ids = q_ids, xm.kv_group_ids = kv_ids;
            xm.bidirectional_within_group = true, xm.is_causal = false;
            orc_rmsnorm_forward(cur, (const float *)s->cross_norm_weight.data, normed, S, E);
            rc = orc_cross_attention_forward(normed, patch_in, (const float *)s->cross_weight_q.data,
                                             (const float *)s->cross_weight_k.data, (const float *)s->cross_weight_v.data,
                                             (const float *)s->cross_weight_proj.data, tmp, S, num_patches * k, E, XH, &xm);
            if (rc != ORC_OK) break;
            orc_add(cur, tmp, mid, S * E);
            b_in = mid;
        }
        orc_rmsnorm_forward(b_in, (const float *)s->norm1_weight.data, normed, S, E);
        orc_matmul(normed, (const float *)s->attn_qkv_w.data, qkv, S, E, 3 * E);
        for (size_t h = 0; h < H; h++) { /* rotate Q and K of every head in place, rows by their gathered tables */
            orc_rope_apply_packed(qkv, 3 * E, h * hd, S, hd, rope_c, rope_s);
            orc_rope_apply_packed(qkv, 3 * E, E + h * hd, S, hd, rope_c, rope_s);
        }
        memset(combined, 0, S * E * sizeof(float));
        for (size_t h = 0; h < H && rc == ORC_OK; h++) {
            blt_attention_head_args a;
            memset(&a, 0, sizeof(a));
            a.q = qkv + h * hd, a.k = qkv + E + h * hd, a.v = qkv + 2 * E + h * hd;
            a.q_stride = a.k_stride = a.v_stride = 3 * E;
            a.combined = combined, a.combined_stride = E, a.combined_col_offset = h * hd;
            a.weights_out = weights;
            a.mask = mask;
            a.nq = S, a.nk = S, a.head_dim = hd;
            a.is_causal = false;
            a.scale = 1.0f / sqrtf((float)hd);
            rc = orc_attention_head_core(&a);
        }
        if (rc != ORC_OK) break;
        orc_matmul(combined, (const float *)s->attn_proj_w.data, tmp, S, E, E);
        orc_add(b_in, tmp, resid1, S * E);
        orc_rmsnorm_forward(resid1, (const float *)s->norm2_weight.data, normed, S, E);
        const size_t hid = s->ffn_up_w.shape[1];
        orc_matmul(normed, (const float *)s->ffn_up_w.data, up, S, E, hid);
        orc_matmul(normed, (const float *)s->ffn_gate_w.data, gate, S, E, hid);
        orc_swiglu_forward(gate, up, act, S * hid);
        orc_matmul(act, (const float *)s->ffn_down_w.data, tmp, S, hid, E);
        orc_add(resid1, tmp, next, S * E);
        float *t = cur;
        cur = next, next = t;
    }
    if (rc == ORC_OK) orc_matmul(cur, (const float *)dec->lm_head_weight.data, logits_out, S, E, V);
    free(cur), free(next), free(positions), free(rope_c), free(rope_s), free(q_ids), free(kv_ids), free(mask);
    free(weights), free(normed), free(mid), free(qkv), free(combined), free(tmp), free(resid1), free(up), free(gate);
    free(act);
    return rc;
}

/* The block rows of the same forward over a cache that already holds the clean prefix (`base` =
 * num_clean valid rows of sequence b, tier 2 refreshed): the rows of
 * orc_local_decoder_forward_diffusion_infer's logits from num_clean on, computed without touching
 * the prefix -- a clean row never sees a block row (csrc/ops/mask_builder_cpu.c:128-131), so the
 * prefix's K and V are what the incremental step cached, and a block row sees all of them plus the
 * whole block (133-135).  Group of row r: batch->groups[r]; rotary row: batch->positions[r]; no
 * window (the INFER mask has none); nothing is committed.  logits_out is [n_block_rows, vocab]. */
int orc_kv_block_step(blt_kv_cache *cache, size_t b, size_t base, size_t num_patches, const blt_block_batch *batch,
                      int d0_mode, float *logits_out) {
    const blt_local_decoder *dec = cache->decoder;
    const blt_local_decoder_config *cfg = &dec->config;
    const size_t E = cache->embed_dim, L = cfg->num_layers, H = cfg->num_heads, XH = cfg->cross_attn_heads;
    const size_t n = batch->n_block_rows;
    if (n < 1 || num_patches < 1 || batch->num_clean != base) return ORC_ERR_ARG;
    if (base + n > cache->max_seq_len || num_patches * cache->k > cache->max_subtokens) return ORC_ERR_CAPACITY;
    float *cur = (float *)malloc(n * E * sizeof(float));
    float *mid = (float *)malloc(n * E * sizeof(float));
    int rc = orc_block_d0_rows(dec, batch, d0_mode, cur);
    for (size_t l = 0; l < L && rc == ORC_OK; l++) {
        const blt_local_layer_storage *s = &dec->layers[l];
        const float *in = cur;
        if (orc_local_cross_attn_fires(cfg->cross_attn_placement, cfg->cross_attn_all_layers, L, l)) {
            rc = orc_kv_cross_block((const float *)cache->cross_k[l].data, (const float *)cache->cross_v[l].data,
                                    cache->max_subtokens, E, XH, b, num_patches * cache->k, cache->k, batch->groups, n,
                                    (const float *)s->cross_norm_weight.data, (const float *)s->cross_weight_q.data,
                                    (const float *)s->cross_weight_proj.data, cur, mid);
            in = mid;
        }
        if (rc != ORC_OK) break;
        rc = orc_kv_decode_layer_kind((float *)cache->self_k[l].data, (float *)cache->self_v[l].data,
                                      cache->max_seq_len, E, H, b, base, n, 0, 1, batch->positions,
                                      (const float *)s->norm1_weight.data, (const float *)s->attn_qkv_w.data,
                                      (const float *)s->attn_proj_w.data, (const float *)s->norm2_weight.data,
                                      (const float *)s->ffn_up_w.data, (const float *)s->ffn_gate_w.data,
                                      (const float *)s->ffn_down_w.data, s->ffn_up_w.shape[1],
                                      (const float *)dec->rope_cos_cache.data, (const float *)dec->rope_sin_cache.data,
                                      dec->rope_cos_cache.shape[0], in, cur);
    }
    if (rc == ORC_OK) orc_matmul(cur, (const float *)dec->lm_head_weight.data, logits_out, n, E, cfg->vocab_size);
    free(cur), free(mid);
    return rc;
}

/* csrc/models/transformer.c:97-128 for an RMSNorm + SwiGLU block (what csrc/models/local_common.c:
 * 99-115 and csrc/models/transformer_stack.c configure): norm, attention block, residual, norm,
 * up / gate projections, SwiGLU, down projection, residual.  input / output are [seq_len, E]. */
int orc_transformer_forward(const float *input, const float *norm1_w, const float *qkv_w, const float *proj_w,
                            const float *norm2_w, const float *up_w, const float *gate_w, const float *down_w,
                            float *output, size_t seq_len, size_t embed_dim, size_t hidden_dim, size_t num_heads,
                            int is_causal, int use_rope, float rope_theta, const float *rope_cos_cache,
                            const float *rope_sin_cache, const blt_mask_config *mask_config) {
    const size_t T = seq_len, E = embed_dim, Hd = hidden_dim;
    float *normed = (float *)malloc(T * E * sizeof(float));
    float *attn = (float *)malloc(T * E * sizeof(float));
    float *resid = (float *)malloc(T * E * sizeof(float));
    float *up = (float *)malloc(T * Hd * sizeof(float));
    float *gate = (float *)malloc(T * Hd * sizeof(float));
    float *act = (float *)malloc(T * Hd * sizeof(float));
    orc_rmsnorm_forward(input, norm1_w, normed, T, E);
    int rc = orc_multihead_attention(normed, qkv_w, proj_w, attn, T, E, num_heads, is_causal, use_rope, rope_theta,
                                     rope_cos_cache, rope_sin_cache, mask_config);
    if (rc == ORC_OK) {
        orc_add(input, attn, resid, T * E);
        orc_rmsnorm_forward(resid, norm2_w, normed, T, E);
        orc_matmul(normed, up_w, up, T, E, Hd);
        orc_matmul(normed, gate_w, gate, T, E, Hd);
        orc_swiglu_forward(gate, up, act, T * Hd);
        orc_matmul(act, down_w, output, T, Hd, E);
        orc_add(resid, output, output, T * E);
    }
    free(normed), free(attn), free(resid), free(up), free(gate), free(act);
    return rc;
}

/* ------------------------------------------------------------------------- */
/* local encoder: embedding + hashed n-grams, patch pooling, layer loop        */
/* ------------------------------------------------------------------------- */

/* ops/gather_scatter_cpu.c:41-61 */
int orc_indexed_row_accumulate(const float *table, size_t vocab, const uint32_t *idx, float *io, size_t rows,
                               size_t embed_dim) {
    for (size_t i = 0; i < rows; i++) {
        if (idx[i] == BLT_IDX_SENTINEL) continue;
        if (idx[i] >= vocab) return ORC_ERR_ARG;
        const float *row = table + (size_t)idx[i] * embed_dim;
        float *dst = io + i * embed_dim;
        for (size_t d = 0; d < embed_dim; d++) dst[d] += row[d];
    }
    return ORC_OK;
}

/* ops/elementwise_cpu.c:31-40 */
void orc_scale(float *x, size_t n, float scalar) {
    for (size_t i = 0; i < n; i++) x[i] *= scalar;
}

/* ops/patch_pool_cpu.c:3-48 */
int orc_patch_pool_forward(const float *byte_hidden, size_t seq_len, size_t embed_dim, const blt_patch_info *patches,
                           size_t num_patches, int pool_type, float *out) {
    if (pool_type != BLT_POOL_MEAN && pool_type != BLT_POOL_MAX) return ORC_ERR_ARG;
    for (size_t j = 0; j < num_patches; j++) {
        const size_t start = patches[j].start_idx, len = patches[j].length;
        if (len < 1 || start + len > seq_len) return ORC_ERR_ARG;
        float *dst = out + j * embed_dim;
        const float *src0 = byte_hidden + start * embed_dim;
        if (pool_type == BLT_POOL_MEAN) {
            for (size_t d = 0; d < embed_dim; d++) dst[d] = 0.0f;
            for (size_t i = 0; i < len; i++)
                for (size_t d = 0; d < embed_dim; d++) dst[d] += src0[i * embed_dim + d];
            const float inv_len = 1.0f / (float)len;
            for (size_t d = 0; d < embed_dim; d++) dst[d] *= inv_len;
        } else {
            memcpy(dst, src0, embed_dim * sizeof(float));
            for (size_t i = 1; i < len; i++)
                for (size_t d = 0; d < embed_dim; d++)
                    if (src0[i * embed_dim + d] > dst[d]) dst[d] = src0[i * embed_dim + d];
        }
    }
    return ORC_OK;
}

/* models/hash_ngram.c:16-79 (state, first window, rolling update), 183-191 (the index list) */
int orc_ngram_indices(const uint8_t *bytes, size_t seq_len, size_t n, uint64_t prime, uint64_t modulus,
                      uint32_t *idx) {
    if (n == 0 || n > 8 || modulus <= 1 || prime == 0 || prime > (UINT64_MAX - 255) / modulus) return ORC_ERR_ARG;
    uint64_t pow_n = 1ULL % modulus;
    for (size_t i = 0; i < n; i++) pow_n = (pow_n * prime) % modulus;
    uint8_t window[8] = {0};
    size_t window_start = 0, seen = 0;
    uint64_t current = 0;
    for (size_t i = 0; i < seq_len; i++) {
        const uint8_t outgoing = window[window_start];
        window[window_start] = bytes[i];
        window_start = (window_start + 1) % n;
        seen++;
        if (seen < n) {
            idx[i] = BLT_IDX_SENTINEL;
            continue;
        }
        if (seen == n) {
            uint64_t hash = 0;
            size_t at = window_start;
            for (size_t t = 0; t < n; t++) {
                hash = (hash * prime + window[at]) % modulus;
                at = (at + 1) % n;
            }
            current = hash;
        } else {
            uint64_t updated = (current * prime + bytes[i]) % modulus;
            const uint64_t gone = ((uint64_t)outgoing * pow_n) % modulus;
            current = (updated + modulus - gone) % modulus;
        }
        idx[i] = (uint32_t)current;
    }
    return ORC_OK;
}

/* models/byte_embedding.c:16-53 then models/hash_ngram.c:142-207 */
int orc_embed_bytes(const float *byte_table, const blt_hash_ngram_config *config,
                    const blt_hash_ngram_weights *weights, const uint8_t *bytes, size_t seq_len, float *out) {
    const size_t E = config->embed_dim;
    if (config->num_ngram_sizes > BLT_MAX_NGRAM_SIZES) return ORC_ERR_ARG;
    for (size_t i = 0; i < seq_len; i++) memcpy(out + i * E, byte_table + (size_t)bytes[i] * E, E * sizeof(float));
    uint32_t *idx = (uint32_t *)malloc((seq_len ? seq_len : 1) * sizeof(uint32_t));
    int rc = ORC_OK;
    for (size_t t = 0; t < config->num_ngram_sizes && rc == ORC_OK; t++) {
        const size_t n = config->ngram_sizes[t];
        if (n == 0 || n > seq_len) continue;
        rc = orc_ngram_indices(bytes, seq_len, n, config->hash_prime, config->per_ngram_vocab, idx);
        if (rc == ORC_OK)
            rc = orc_indexed_row_accumulate((const float *)weights->tables[t].data, config->per_ngram_vocab, idx, out,
                                            seq_len, E);
    }
    free(idx);
    if (rc == ORC_OK && config->normalize) orc_scale(out, seq_len * E, 1.0f / (float)(config->num_ngram_sizes + 1));
    return rc;
}

/* models/local_encoder.c:193-281; masks and views as make_context / make_cross_attn_config /
 * setup_query_split_mask build them (52-113), layer configuration as local_common.c:99-115 */
int orc_local_encoder_forward(const blt_local_encoder *enc, const uint8_t *bytes, size_t seq_len,
                              const blt_patch_info *patches, size_t num_patches, const size_t *doc_boundaries,
                              size_t num_docs, float *patch_out, float *byte_hidden_out) {
    const blt_local_encoder_config *cfg = &enc->config;
    const size_t E = cfg->embed_dim, T = seq_len, P = num_patches;
    const size_t patch_dim = cfg->patch_dim == 0 ? E : cfg->patch_dim;
    if (E == 0 || patch_dim % E != 0 || P < 1 || T < 1 || T > cfg->max_seq_len) return ORC_ERR_ARG;
    const size_t k = patch_dim / E;

    size_t *q_groups = (size_t *)malloc(P * sizeof(size_t));
    size_t *kv_groups = (size_t *)malloc(T * sizeof(size_t));
    size_t *q_split = (size_t *)malloc(P * k * sizeof(size_t));
    float *h = (float *)malloc(T * E * sizeof(float));
    float *h_next = (float *)malloc(T * E * sizeof(float));
    float *pooled = (float *)malloc(P * E * sizeof(float));
    float *p = (float *)malloc(P * patch_dim * sizeof(float));
    float *query = (float *)malloc(P * patch_dim * sizeof(float));
    float *cross = (float *)malloc(P * patch_dim * sizeof(float));
    int rc = orc_patch_build_group_ids(patches, P, T, q_groups, kv_groups);

    blt_mask_config local_mask, cross_mask;
    memset(&local_mask, 0, sizeof(local_mask));
    memset(&cross_mask, 0, sizeof(cross_mask));
    local_mask.seq_len_q = local_mask.seq_len_kv = T;
    local_mask.sliding_window = cfg->local_window;
    local_mask.doc_boundaries = doc_boundaries;
    local_mask.num_docs = num_docs;
    local_mask.is_causal = true;
    cross_mask.seq_len_q = P * k;
    cross_mask.seq_len_kv = T;
    cross_mask.query_group_ids = q_groups;
    cross_mask.kv_group_ids = kv_groups;
    cross_mask.bidirectional_within_group = true;
    if (k > 1) {
        orc_patch_expand_group_ids(q_groups, P, k, q_split);
        cross_mask.query_group_ids = q_split;
    }

    if (rc == ORC_OK)
        rc = orc_embed_bytes((const float *)enc->byte_embedding_weight.data, &cfg->ngram_config, &enc->ngram_weights,
                             bytes, T, h);
    if (rc == ORC_OK) rc = orc_patch_pool_forward(h, T, E, patches, P, (int)cfg->pool_type, pooled);
    if (rc == ORC_OK)
        for (size_t sj = 0; sj < k; sj++) orc_strided_copy(p + sj * E, patch_dim, pooled, E, P, E);

    for (size_t l = 0; l < cfg->num_layers && rc == ORC_OK; l++) {
        const blt_local_layer_storage *s = &enc->layers[l];
        rc = orc_transformer_forward(h, (const float *)s->norm1_weight.data, (const float *)s->attn_qkv_w.data,
                                     (const float *)s->attn_proj_w.data, (const float *)s->norm2_weight.data,
                                     (const float *)s->ffn_up_w.data, (const float *)s->ffn_gate_w.data,
                                     (const float *)s->ffn_down_w.data, h_next, T, E, cfg->hidden_dim, cfg->num_heads, 1,
                                     1, cfg->rope_theta, (const float *)enc->rope_cos_cache.data,
                                     (const float *)enc->rope_sin_cache.data, &local_mask);
        if (rc != ORC_OK) break;
        float *swap = h;
        h = h_next, h_next = swap;
        if (!orc_local_cross_attn_fires((int)cfg->cross_attn_placement, cfg->cross_attn_all_layers, cfg->num_layers, l))
            continue;
        orc_rmsnorm_forward(p, (const float *)s->cross_norm_weight.data, query, P * k, E);
        rc = orc_cross_attention_forward(query, h, (const float *)s->cross_weight_q.data,
                                         (const float *)s->cross_weight_k.data, (const float *)s->cross_weight_v.data,
                                         (const float *)s->cross_weight_proj.data, cross, P * k, T, E,
                                         cfg->cross_attn_heads, &cross_mask);
        if (rc == ORC_OK) orc_add(p, cross, p, P * patch_dim);
    }
    if (rc == ORC_OK) {
        memcpy(patch_out, p, P * patch_dim * sizeof(float));
        memcpy(byte_hidden_out, h, T * E * sizeof(float));
    }
    free(q_groups), free(kv_groups), free(q_split), free(h), free(h_next), free(pooled), free(p), free(query), free(cross);
    return rc;
}

