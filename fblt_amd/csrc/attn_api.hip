/*
 * Entry points of the attention forward path: the per-head device twin the
 * reference's dispatcher binds, the whole-batch launch and the resident plan.
 * Host code only (argument checks, descriptor translation, kernel choice);
 * the kernels live in attn_rows.hip, attn_mfma.hip, attn_wide.hip, attn_fine.hip and attn_once.hip.
 */
#include "blt_hip.h"
#include "blt_fatal.h"
#include "hip_check.h"
#include "attn_launch.h"
#include "launch.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

namespace {

/* Kernel family a problem is routed to. */
enum Family : uint32_t { FAM_ROWS = 0, FAM_MFMA = 1, FAM_WIDE = 2, FAM_FINE = 3, FAM_ONCE = 4, FAM_COUNT = 5 };

struct Bucket {
    Family fam;
    uint32_t hd;      /* head_dim shared by the bucket */
    bool vec4;        /* every problem has ATTN_FLAG_VEC4 */
    bool dense;       /* every problem reads a dense mask */
    bool affine;      /* mfma: problems are one strided batch, see `aff` */
    AttnAffine aff;
    uint32_t base;    /* first descriptor in the sorted array */
    uint32_t count;
    uint32_t max_nq;
    uint32_t tiles;   /* mfma: number of work items; first item index in tile array = tile_base */
    uint32_t tile_base;
    uint32_t span;    /* fine: keys the longest 32-row tile needs; once: 16-key tiles the longest 16-row tile spans */
    bool tall;        /* fine: 16-row workgroups of sixteen waves */
    bool whole;       /* fine: one four-wave workgroup per whole problem (strided batches) */
};

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

/* Translate and check one problem.  `what` prefixes error messages. */
AttnProb translate(const blt_attention_problem &pr, bool need_score_buffer, const char *what) {
    const blt_attention_head_args &a = pr.head;
    BLT_REQUIRE(a.q != NULL && a.k != NULL && a.v != NULL && a.combined != NULL, "%s: buffers must not be NULL",
                what);
    if (need_score_buffer)
        BLT_REQUIRE(a.weights_out != NULL || a.scores_scratch != NULL || a.lse_out != NULL,
                    "%s: need weights_out, scores_scratch, or lse_out", what);
    BLT_REQUIRE(a.nq <= 0x7FFFFFFFu && a.nk <= 0x7FFFFFFFu, "%s: nq/nk exceed 2^31-1", what);
    BLT_REQUIRE(a.head_dim >= 1 && a.head_dim <= ATTN_ROWS_MAX_HEAD_DIM, "%s: head_dim must be in [1, %u]", what,
                ATTN_ROWS_MAX_HEAD_DIM);
    BLT_REQUIRE(a.q_stride <= 0xFFFFFFFFu && a.k_stride <= 0xFFFFFFFFu && a.v_stride <= 0xFFFFFFFFu &&
                    a.combined_stride <= 0xFFFFFFFFu,
                "%s: row strides exceed 2^32-1 elements", what);

    AttnProb d;
    std::memset(&d, 0, sizeof(d));
    d.q = a.q;
    d.k = a.k;
    d.v = a.v;
    d.out = a.combined + a.combined_col_offset;
    d.weights = a.weights_out;
    d.lse = a.lse_out;
    d.q_stride = (uint32_t)a.q_stride;
    d.k_stride = (uint32_t)a.k_stride;
    d.v_stride = (uint32_t)a.v_stride;
    d.out_stride = (uint32_t)a.combined_stride;
    d.nq = (uint32_t)a.nq;
    d.nk = (uint32_t)a.nk;
    d.hd = (uint32_t)a.head_dim;
    d.scale = a.scale;

    switch (pr.mask_kind) {
    case BLT_ATTN_MASK_FROM_HEAD:
        if (a.mask != NULL) {
            d.vis = ATTN_VIS_DENSE;
            d.mask = a.mask;
        } else if (a.is_causal) {
            d.vis = ATTN_VIS_CAUSAL;
        } else {
            d.vis = ATTN_VIS_ALL;
        }
        break;
    case BLT_ATTN_MASK_CAUSAL:
        BLT_REQUIRE(a.mask == NULL, "%s: a mask descriptor and a dense mask exclude each other", what);
        BLT_REQUIRE(pr.causal_offset <= 0x7FFFFFFFu && pr.window <= 0xFFFFFFFFu,
                    "%s: causal_offset/window out of range", what);
        d.vis = ATTN_VIS_CAUSAL;
        d.causal_off = (uint32_t)pr.causal_offset;
        d.window = (uint32_t)pr.window;
        break;
    case BLT_ATTN_MASK_ROW_RANGE:
        BLT_REQUIRE(a.mask == NULL, "%s: a mask descriptor and a dense mask exclude each other", what);
        BLT_REQUIRE(pr.row_lo != NULL && pr.row_hi != NULL, "%s: row ranges must not be NULL", what);
        d.vis = ATTN_VIS_RANGE;
        d.row_lo = pr.row_lo;
        d.row_hi = pr.row_hi;
        d.range_span = pr.row_span;
        break;
    default:
        BLT_FATAL("%s: unknown mask_kind %u", what, pr.mask_kind);
    }

    const bool vec = aligned16(d.q) && aligned16(d.k) && aligned16(d.v) && aligned16(d.out) && d.q_stride % 4 == 0 &&
                     d.k_stride % 4 == 0 && d.v_stride % 4 == 0 && d.out_stride % 4 == 0 && d.hd % 4 == 0;
    if (vec) d.flags |= ATTN_FLAG_VEC4;
    return d;
}

/* BLT_HIP_ATTN_FAMILY=rows|mfma|wide|fine|once pins the kernel family wherever the
 * shape allows it (tuning and test hook); unset or anything else = automatic. */
int family_override() {
    static const int cached = [] {
        const char *e = getenv("BLT_HIP_ATTN_FAMILY");
        if (e && std::strcmp(e, "rows") == 0) return 1;
        if (e && std::strcmp(e, "mfma") == 0) return 2;
        if (e && std::strcmp(e, "wide") == 0) return 3;
        if (e && std::strcmp(e, "fine") == 0) return 4;
        if (e && std::strcmp(e, "once") == 0) return 5;
        return 0;
    }();
    return cached;
}

Family choose_family(const AttnProb &d) {
    const int forced = family_override();
    if (forced == 1) return FAM_ROWS;
    if (forced == 5) return attn_once_can(d) || attn_mfma_takes(d) ? FAM_MFMA : FAM_ROWS;
    if (forced >= 2 && attn_mfma_can(d)) return FAM_MFMA;
    if (attn_mfma_takes(d)) return FAM_MFMA;
    return FAM_ROWS;
}

/* The wide kernel pays off once its 128-row work items give every compute
 * unit one (short rows: few key tiles per item) or two (long rows: the
 * latency-oriented mfma kernel, which splits the keys of a 32-row tile over
 * its waves, keeps the shorter serial chain for longer) -- measured
 * crossovers: 128..256 items at 128 keys, 256..512 items at 512 keys. */
uint32_t wide_min_groups(uint32_t max_nk) {
    return max_nk <= 256u ? 256u : 512u;
}

/* Do problems p[0..n), all routed to the mfma family, go to the wide kernel instead? */
bool choose_wide(const AttnProb *p, uint32_t n) {
    const int forced = family_override();
    if (forced == 1 || forced == 2 || forced == 4 || forced == 5) return false;
    uint64_t groups = 0;
    uint32_t max_nk = 0;
    for (uint32_t i = 0; i < n; i++) {
        if (!attn_wide_can(p[i])) return false;
        groups += attn_wide_groups(p[i]);
        max_nk = std::max(max_nk, p[i].nk);
    }
    return forced == 3 || groups >= wide_min_groups(max_nk);
}

/* Do problems p[0..n), all routed to the mfma family, go to the fine kernel, and in which workgroup
 * shape?  `span` gets the keys its longest 32-row tile needs.  Measured at both head widths (4 heads
 * of 32, 8 heads of 64), 1..128 sequences of 64..2048 rows, against the other two matrix-core
 * kernels:
 *   - few long problems (at most 128 tiles of 32 rows, rows of 256 keys and more): workgroups of 16
 *     rows and sixteen waves double the workgroups and halve the chain of matrix instructions on the
 *     busiest SIMD (512 rows x 4 heads: 8.9 -> 8.0 us; 1024 rows: 15.1 -> 11.7 us).  Only strided
 *     batches and single problems have this shape;
 *   - one LDS fill holds every key a tile needs (128 keys at width 64, 256 at 32): ahead unless the
 *     launch is tiny (up to one 4-wave workgroup per compute unit: the mfma kernel's shorter
 *     prologue wins from 128 keys on) or so large that workgroups queue up several deep (the wide
 *     kernel overlaps its fetches with its arithmetic, this one fetches, then computes);
 *   - longer rows when the launch is just what the chip holds at once, two 8-wave workgroups per
 *     compute unit (512 tiles: 10..25 % ahead of the mfma kernel, behind it at 256 and at 1024). */
bool choose_fine(const AttnProb *p, uint32_t n, bool strided, uint32_t &span, bool &tall) {
    /* BLT_HIP_FINE_ROWS=16|32 pins the workgroup shape (tuning and test hook) */
    static const int rows_pinned = [] {
        const char *e = getenv("BLT_HIP_FINE_ROWS");
        const int v = e ? std::atoi(e) : 0;
        return v == 16 || v == 32 ? v : 0;
    }();
    const int forced = family_override();
    tall = false;
    if (forced != 0 && forced != 4) return false;
    span = 0;
    uint64_t tiles = 0, groups = 0;
    uint32_t max_nk = 0;
    for (uint32_t i = 0; i < n; i++) {
        if (!attn_fine_can(p[i])) return false;
        span = std::max(span, attn_fine_span(p[i]));
        tiles += (p[i].nq + 31u) / 32u;
        groups += attn_wide_can(p[i]) ? attn_wide_groups(p[i]) : 0u;
        max_nk = std::max(max_nk, p[i].nk);
    }
    const bool tall_fits = strided && tiles <= 128u && span >= 256u;
    if (forced == 4) {
        tall = strided && (rows_pinned == 16 || (rows_pinned == 0 && tall_fits));
        return true;
    }
    if (rows_pinned != 32 && (tall_fits || (rows_pinned == 16 && strided))) {
        tall = true;
        return true;
    }
    if (span > attn_fine_fill_max(p[0].hd)) return tiles > 448u && tiles <= 512u;
    if (tiles <= 256u && span > 64u) return false;
    return groups < (max_nk <= 64u ? 640u : 448u);
}

/* Do problems p[0..n), all routed to the mfma family, go to the once kernel (16-row tiles whose keys
 * are all in flight at once)?  `span` gets the 16-key tiles its longest tile spans.  The kernel is
 * built for launches one trip to memory deep: it is chosen while the launch gives a compute unit
 * one workgroup, or two short ones. */
bool choose_once(const AttnProb *p, uint32_t n, uint32_t &span) {
    const int forced = family_override();
    if (forced != 0 && forced != 5) return false;
    uint64_t tiles = 0;
    uint32_t most = 0;
    for (uint32_t i = 0; i < n; i++) {
        if (!attn_once_can(p[i])) return false;
        most = std::max(most, attn_once_span_tiles(p[i]));
        tiles += (p[i].nq + 15u) / 16u;
    }
    /* measured against the other matrix-core kernels (4 heads of 32 over 256 ... 1024 rows, 8 heads of 64
     * over 128 rows, 1 ... 16 sequences): ahead up to 256 tiles whatever the rows' length (one workgroup
     * per compute unit), up to 512 tiles while a row has at most 128 keys, behind beyond */
    if (forced == 0 && tiles > (most <= 8u ? 512u : 256u)) return false;
    span = most;
    return true;
}

/* Does a strided batch of n problems like `d` go to the fine family's whole-problem shape (one
 * four-wave workgroup per problem of at most 128 rows whose keys fit one LDS fill)?  It fetches
 * K and V once per problem and balances the causal triangle inside the workgroup, which pays once
 * the batch is several workgroups deep on every compute unit.  BLT_HIP_FINE_ROWS=128 pins it
 * wherever the shape allows (tuning and test hook). */
bool choose_whole(const AttnProb &d, uint32_t n, bool strided) {
    static const int rows_pinned = [] {
        const char *e = getenv("BLT_HIP_FINE_ROWS");
        return e ? std::atoi(e) : 0;
    }();
    const int forced = family_override();
    if (!strided || (forced != 0 && forced != 4) || !attn_whole_can(d)) return false;
    if (rows_pinned != 0) return rows_pinned == 128;
    if (forced != 0 || d.nq < 48u) return false; /* three row halves and fewer leave most of the waves idle */
    /* measured against the family's other shapes and the wide kernel (8 heads of 64 and 4 heads
     * of 32): 128 rows ahead from 144 problems on (11.9 against 12.4 us; 12.5 against 15.6 at
     * 256, 38.7 against 45.5 at 1024, 72.5 against 86 at 2048), 64 rows from 768 on */
    return n >= (d.nq > 64u ? 144u : 640u);
}

/* Element distance between two float pointers (either both NULL or both set). */
bool elem_delta(const void *a, const void *b, int64_t &out) {
    if ((a == nullptr) != (b == nullptr)) return false;
    const int64_t bytes = (int64_t)(reinterpret_cast<intptr_t>(b) - reinterpret_cast<intptr_t>(a));
    if (bytes % 4 != 0) return false;
    out = bytes / 4;
    return true;
}

bool same_shape(const AttnProb &a, const AttnProb &b) {
    return a.q_stride == b.q_stride && a.k_stride == b.k_stride && a.v_stride == b.v_stride &&
           a.out_stride == b.out_stride && a.nq == b.nq && a.nk == b.nk && a.hd == b.hd && a.vis == b.vis &&
           a.causal_off == b.causal_off && a.window == b.window && a.scale == b.scale && a.flags == b.flags;
}

/* The nine pointers of a problem, in a fixed order. */
void pointers_of(const AttnProb &d, const void *(&out)[9]) {
    out[0] = d.q, out[1] = d.k, out[2] = d.v, out[3] = d.out, out[4] = d.weights, out[5] = d.lse, out[6] = d.mask;
    out[7] = d.row_lo, out[8] = d.row_hi;
}

/* Are problems p[0..n) one strided batch: p[i] = p[0] + (i / H) * seq + (i % H) * head
 * for every pointer, with a common shape?  Fills `out` for the first H that fits. */
bool detect_affine(const AttnProb *p, uint32_t n, AttnAffine &out) {
    if (n < 2) return false;
    for (uint32_t i = 1; i < n; i++)
        if (!same_shape(p[0], p[i])) return false;
    for (uint32_t H = 1; H <= n; H++) {
        if (n % H != 0) continue;
        int64_t head[9], seq[9];
        const void *p0[9], *pi[9];
        pointers_of(p[0], p0);
        bool ok = true;
        for (int f = 0; f < 9 && ok; f++) {
            head[f] = seq[f] = 0;
            if (H > 1) {
                pointers_of(p[1], pi);
                ok = elem_delta(p0[f], pi[f], head[f]);
            }
            if (ok && n > H) {
                pointers_of(p[H], pi);
                ok = elem_delta(p0[f], pi[f], seq[f]);
            }
        }
        for (uint32_t i = 0; i < n && ok; i++) {
            pointers_of(p[i], pi);
            for (int f = 0; f < 9 && ok; f++) {
                int64_t d;
                ok = elem_delta(p0[f], pi[f], d) &&
                     (p0[f] == nullptr || d == (int64_t)(i / H) * seq[f] + (int64_t)(i % H) * head[f]);
            }
        }
        if (!ok) continue;
        if (seq[7] != seq[8] || head[7] != head[8]) continue; /* row_lo and row_hi move together */
        std::memset(&out, 0, sizeof(out));
        out.first = p[0];
        out.q_seq = seq[0], out.q_head = head[0];
        out.k_seq = seq[1], out.k_head = head[1];
        out.v_seq = seq[2], out.v_head = head[2];
        out.o_seq = seq[3], out.o_head = head[3];
        out.w_seq = seq[4], out.w_head = head[4];
        out.lse_seq = seq[5], out.lse_head = head[5];
        out.mask_seq = seq[6], out.mask_head = head[6];
        out.range_seq = seq[7], out.range_head = head[7];
        out.count = n;
        out.heads = H;
        out.nqt = (p[0].nq + 31u) / 32u;
        return true;
    }
    return false;
}

} // namespace

struct blt_attention_plan {
    std::vector<AttnProb> host;   /* sorted by bucket */
    std::vector<Bucket> buckets;
    std::vector<AttnTile> tiles;  /* mfma work items, all buckets */
    AttnProb *dev = nullptr;      /* resident plans: descriptors in device memory */
    AttnTile *dev_tiles = nullptr;
    std::string kernel_name = "none";
};

namespace {

void plan_build(blt_attention_plan &pl, const blt_attention_problem *problems, size_t count, bool need_score_buffer,
                const char *what) {
    pl.host.clear();
    pl.buckets.clear();
    pl.tiles.clear();
    pl.host.reserve(count);
    std::vector<std::pair<uint64_t, AttnProb>> keyed;
    keyed.reserve(count);
    bool any_mfma = false;
    for (size_t t = 0; t < count; t++) {
        AttnProb d = translate(problems[t], need_score_buffer, what);
        if (d.nq == 0) continue; /* nothing to write */
        const Family f = choose_family(d);
        any_mfma = any_mfma || f == FAM_MFMA;
        const uint64_t vec4 = (d.flags & ATTN_FLAG_VEC4) ? 1u : 0u, dense = d.vis == ATTN_VIS_DENSE ? 1u : 0u;
        keyed.emplace_back(((uint64_t)f << 40) | ((uint64_t)d.hd << 8) | (vec4 << 1) | dense, d);
    }
    /* Problems that went to the rows family only for their few rows (the short documents of a
     * document-causal batch) join the matrix-core launch the batch has anyway rather than cost a
     * launch of their own. */
    if (any_mfma && family_override() == 0) {
        for (auto &kd : keyed) {
            const AttnProb &d = kd.second;
            if ((Family)(kd.first >> 40) == FAM_ROWS && d.vis != ATTN_VIS_RANGE && attn_mfma_can(d))
                kd.first = (kd.first & ((1ull << 40) - 1u)) | ((uint64_t)FAM_MFMA << 40);
        }
    }
    std::stable_sort(keyed.begin(), keyed.end(),
                     [](const std::pair<uint64_t, AttnProb> &x, const std::pair<uint64_t, AttnProb> &y) {
                         return x.first < y.first;
                     });
    for (size_t t = 0; t < keyed.size(); t++) {
        const AttnProb &d = keyed[t].second;
        const Family f = (Family)(keyed[t].first >> 40);
        if (t == 0 || keyed[t].first != keyed[t - 1].first) {
            Bucket b;
            std::memset(&b, 0, sizeof(b));
            b.fam = f;
            b.hd = d.hd;
            b.vec4 = (d.flags & ATTN_FLAG_VEC4) != 0;
            b.dense = d.vis == ATTN_VIS_DENSE;
            b.base = (uint32_t)t;
            b.count = 0;
            b.max_nq = 0;
            b.tiles = 0;
            b.tile_base = 0;
            pl.buckets.push_back(b);
        }
        Bucket &b = pl.buckets.back();
        b.count++;
        b.max_nq = std::max(b.max_nq, d.nq);
        pl.host.push_back(d);
    }
    for (Bucket &b : pl.buckets) {
        if (b.fam == FAM_ROWS) { /* strided batches need no descriptor memory in this family either */
            b.affine = detect_affine(pl.host.data() + b.base, b.count, b.aff);
            continue;
        }
        if (b.fam != FAM_MFMA) continue;
        b.affine = detect_affine(pl.host.data() + b.base, b.count, b.aff);
        b.whole = choose_whole(pl.host[b.base], b.count, b.affine);
        if (b.whole) b.fam = FAM_FINE;
        else if (choose_once(pl.host.data() + b.base, b.count, b.span)) b.fam = FAM_ONCE;
        else if (choose_fine(pl.host.data() + b.base, b.count, b.affine, b.span, b.tall)) b.fam = FAM_FINE;
        else if (choose_wide(pl.host.data() + b.base, b.count)) b.fam = FAM_WIDE;
        if (b.affine) continue; /* no descriptor or tile memory needed */
        b.tile_base = (uint32_t)pl.tiles.size();
        if (b.fam == FAM_WIDE) attn_wide_make_tiles(pl.host.data(), b.base, b.count, pl.tiles);
        else if (b.fam == FAM_FINE) attn_fine_make_tiles(pl.host.data(), b.base, b.count, pl.tiles);
        else if (b.fam == FAM_ONCE) attn_once_make_tiles(pl.host.data(), b.base, b.count, pl.tiles);
        else attn_mfma_make_tiles(pl.host.data(), b.base, b.count, pl.tiles);
        b.tiles = (uint32_t)pl.tiles.size() - b.tile_base;
    }
    bool any[FAM_COUNT] = {false, false, false, false, false};
    for (const Bucket &b : pl.buckets) any[b.fam] = true;
    /* the families the plan launches, joined by '+': "fine", "mfma+rows", ... */
    static const char *const names[FAM_COUNT] = {"rows", "mfma", "wide", "fine", "once"};
    pl.kernel_name.clear();
    for (int f = FAM_COUNT - 1; f >= 0; f--) {
        if (!any[f]) continue;
        if (!pl.kernel_name.empty()) pl.kernel_name += "+";
        pl.kernel_name += names[f];
    }
    if (pl.kernel_name.empty()) pl.kernel_name = "none";
}

void plan_launch(const blt_attention_plan &pl, const AttnProb *dev, const AttnTile *dev_tiles) {
    for (const Bucket &b : pl.buckets) {
        if (b.fam == FAM_ONCE && b.affine)
            attn_once_launch_affine(b.aff, 0);
        else if (b.fam == FAM_ONCE)
            attn_once_launch(dev, dev_tiles + b.tile_base, b.tiles, b.hd, b.span, b.dense, 0);
        else if (b.fam == FAM_WIDE && b.affine)
            attn_wide_launch_affine(b.aff, 0);
        else if (b.fam == FAM_WIDE)
            attn_wide_launch(dev, dev_tiles + b.tile_base, b.tiles, b.hd, b.dense, 0);
        else if (b.fam == FAM_FINE && b.whole)
            attn_whole_launch_affine(b.aff, 0);
        else if (b.fam == FAM_FINE && b.affine)
            attn_fine_launch_affine(b.aff, b.tall, 0);
        else if (b.fam == FAM_FINE)
            attn_fine_launch(dev, dev_tiles + b.tile_base, b.tiles, b.hd, b.span, 0);
        else if (b.fam == FAM_MFMA && b.affine)
            attn_mfma_launch_affine(b.aff, 0);
        else if (b.fam == FAM_MFMA)
            attn_mfma_launch(dev, dev_tiles + b.tile_base, b.tiles, b.hd, b.vec4, b.dense, 0);
        else if (b.affine)
            attn_rows_launch_affine(b.aff, 0);
        else
            attn_rows_launch(dev, b.base, b.count, b.hd, b.max_nq, 0);
    }
    HIP_CHECK_LAUNCH("attention forward");
}

/* Staging for one-shot batches: descriptors go host vector -> pinned buffer ->
 * device buffer with a truly asynchronous copy on the library's stream.  The
 * device buffer can be reused by the next call because that call's copy is
 * ordered behind this call's kernels -- which holds per stream, so there is
 * one staging buffer per (host thread, stream); the pinned side is the calling
 * thread's ring of buffers (blt_upload_staged). */
struct Staging {
    blt_attention_plan plan;
    void *device = nullptr;
    size_t capacity = 0;

    void run() {
        const size_t pbytes = plan.host.size() * sizeof(AttnProb);
        const size_t tbytes = plan.tiles.size() * sizeof(AttnTile);
        const size_t need = pbytes + tbytes;
        if (need == 0) return;
        bool strided = true; /* every bucket travels in kernel arguments: nothing to stage */
        for (const Bucket &b : plan.buckets) strided = strided && b.affine;
        if (strided) {
            plan_launch(plan, nullptr, nullptr);
            return;
        }
        BLT_REQUIRE(!blt_stream_capturing(),
                    "blt_attention_batch: this batch stages its descriptors through host memory, which a graph "
                    "cannot replay; use a resident plan (blt_attention_plan_*) or a strided batch under capture");
        if (need > capacity) {
            if (device) {
                HIP_CHECK(hipDeviceSynchronize());
                HIP_CHECK(hipFree(device));
            }
            capacity = std::max<size_t>(2 * need, 64 * 1024);
            HIP_CHECK(hipMalloc(&device, capacity));
        }
        /* the device copy is rewritten in stream order, behind the kernels of the previous call that
         * read it; the host side goes through the ring of pinned buffers, so consecutive calls do
         * not wait for each other */
        blt_upload_staged(device, plan.host.data(), pbytes);
        if (tbytes) blt_upload_staged(static_cast<char *>(device) + pbytes, plan.tiles.data(), tbytes);
        plan_launch(plan, static_cast<const AttnProb *>(device),
                    reinterpret_cast<const AttnTile *>(static_cast<const char *>(device) + pbytes));
    }
};

Staging &staging() {
    static thread_local std::map<hipStream_t, Staging> by_stream;
    return by_stream[blt_stream_key()];
}

} // namespace

extern "C" void blt_attention_head_core_hip(blt_backend backend, const blt_attention_head_args *a) {
    BLT_REQUIRE(backend == BLT_BACKEND_HIP, "blt_attention_head_core: HIP implementation called with non-HIP backend");
    BLT_REQUIRE(a != NULL, "blt_attention_head_core: buffers must not be NULL");
    blt_attention_problem pr;
    std::memset(&pr, 0, sizeof(pr));
    pr.head = *a;
    pr.mask_kind = BLT_ATTN_MASK_FROM_HEAD;
    /* one problem: the descriptor travels as a kernel argument, nothing is staged */
    const AttnProb d = translate(pr, true, "blt_attention_head_core");
    if (d.nq == 0) return;
    const Family f = choose_family(d);
    uint32_t span = 0;
    bool tall = false;
    if (f == FAM_MFMA && choose_once(&d, 1, span)) attn_once_launch_single(d, 0);
    else if (f == FAM_MFMA && choose_fine(&d, 1, true, span, tall)) attn_fine_launch_single(d, tall, 0);
    else if (f == FAM_MFMA && choose_wide(&d, 1)) attn_wide_launch_single(d, 0);
    else if (f == FAM_MFMA) attn_mfma_launch_single(d, 0);
    else attn_rows_launch_single(d, 0);
    HIP_CHECK_LAUNCH("blt_attention_head_core");
}

extern "C" void blt_attention_batch_hip(const blt_attention_problem *problems, size_t count) {
    if (count == 0) return;
    BLT_REQUIRE(problems != NULL, "blt_attention_batch: problems must not be NULL");
    Staging &st = staging();
    plan_build(st.plan, problems, count, false, "blt_attention_batch");
    st.run();
}

extern "C" blt_attention_plan *blt_attention_plan_create_hip(const blt_attention_problem *problems, size_t count) {
    BLT_REQUIRE(problems != NULL || count == 0, "blt_attention_plan_create: problems must not be NULL");
    blt_attention_plan *pl = new blt_attention_plan();
    plan_build(*pl, problems, count, false, "blt_attention_plan_create");
    if (!pl->host.empty()) {
        HIP_CHECK(hipMalloc((void **)&pl->dev, pl->host.size() * sizeof(AttnProb)));
        HIP_CHECK(hipMemcpy(pl->dev, pl->host.data(), pl->host.size() * sizeof(AttnProb), hipMemcpyHostToDevice));
    }
    if (!pl->tiles.empty()) {
        HIP_CHECK(hipMalloc((void **)&pl->dev_tiles, pl->tiles.size() * sizeof(AttnTile)));
        HIP_CHECK(hipMemcpy(pl->dev_tiles, pl->tiles.data(), pl->tiles.size() * sizeof(AttnTile),
                            hipMemcpyHostToDevice));
    }
    return pl;
}

extern "C" void blt_attention_plan_run_hip(const blt_attention_plan *plan) {
    BLT_REQUIRE(plan != NULL, "blt_attention_plan_run: plan must not be NULL");
    plan_launch(*plan, plan->dev, plan->dev_tiles);
}

extern "C" void blt_attention_plan_destroy_hip(blt_attention_plan *plan) {
    if (!plan) return;
    HIP_CHECK(hipDeviceSynchronize());
    if (plan->dev) HIP_CHECK(hipFree(plan->dev));
    if (plan->dev_tiles) HIP_CHECK(hipFree(plan->dev_tiles));
    delete plan;
}

extern "C" const char *blt_attention_plan_kernel_hip(const blt_attention_plan *plan) {
    return plan ? plan->kernel_name.c_str() : "none";
}
