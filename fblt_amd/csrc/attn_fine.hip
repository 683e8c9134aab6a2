/*
 * "fine" kernel family: fused QK^T -> online softmax -> PV for prefill shapes
 * whose launches hold about as many 32-row query tiles as the chip has
 * compute-unit slots (a patch transformer over 128 patches, a few heads of a
 * short byte window).  There a workgroup's time is the matrix-core time of its
 * busiest SIMD, so the work is cut finer than a 32x32 score tile:
 *
 *   unit          = 16 query rows x 16 keys on v_mfma_f32_16x16x4_f32
 *                   (HD/4 instructions for S^T, HD/4 for O^T);
 *   workgroup     = one tile of 32 query rows, eight waves: waves 0..3 own rows
 *                   0..15 of the tile, waves 4..7 rows 16..31;
 *   unit -> wave  : the units of the tile are numbered row half by row half,
 *                   key tile by key tile, and unit u goes to wave u % 4 of its
 *                   row half, so the four SIMDs of the compute unit differ by at
 *                   most one unit whatever the causal triangle leaves of each
 *                   row half, and fully masked 16x16 corners are never computed.
 *
 * Every K and V row a tile needs is used by both row halves, so the workgroup
 * fetches them once, with consecutive lanes on consecutive 16-byte pieces of a
 * row, into LDS (rows padded by four floats: fragment reads of sixteen lanes
 * fall on distinct banks); the waves read their fragments from there.  Keys
 * beyond what one fill holds are walked in further fills.
 *
 * Both contractions are computed transposed, as in the other matrix-core
 * kernels, so that a lane's scores, weights and output accumulators all
 * belong to one query (column c = lane % 16):
 *
 *   S^T[key, query] = sum_d K[key, d] Q[query, d]        A = K,   B = Q^T
 *   O^T[d,   query] = sum_key V[key, d] P^T[key, query]   A = V^T, B = P^T
 *
 * register r of lane (g = lane / 16, c) of an accumulator is row 4 g + r,
 * column c.  Row i of the e-th O^T tile stands for column (HD/16) i + e of the
 * head, so that a lane's V operands of one key are consecutive floats in LDS.
 * The eight partial (max, sum, O) of a tile meet once in LDS.
 *
 * A second shape of the same kernel serves launches with few, long problems (a
 * byte window of 512 rows over 4 heads: 64 tiles of 32 rows on 256 compute
 * units): the workgroup is one tile of 16 query rows and all of its sixteen
 * waves take key tiles of those rows, so the launch has twice the workgroups,
 * each with half the matrix-core work and four waves per SIMD to hide a unit's
 * latency chain; the next fill is requested before the units of the current one
 * start.
 *
 * A third shape (attn_whole_kernel) serves strided batches of many short problems
 * (at most 128 rows, keys within one fill), where the launch is several workgroups
 * deep on every compute unit and the time is the bytes moved: one four-wave
 * workgroup per problem fetches K and V once for all of its rows.
 *
 * Takes closed-form visibility (all keys, causal with optional window), head
 * widths 32 and 64 with 16-byte aligned rows, no weights output.
 */
#include "attn_device.h"
#include "attn_launch.h"
#include "attn_tile.h"
#include "hip_check.h"
#include "lane_ops.h"
#include "launch.h"
#include <algorithm>
#include <cstdlib>

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

/* HALVES row halves of 16 query rows per workgroup, WAVES waves in all (WAVES / HALVES per half). */
template <int HD, int HALVES, int WAVES>
struct FineShape {
    static constexpr uint32_t THREADS = 64u * WAVES;
    static constexpr int ROW = HD + 4;  /* floats per parked row  */
    static constexpr int LPR4 = HD / 4; /* 16-byte pieces per row */
    /* keys one LDS fill holds at most (K and V together: 68 KB at 64 columns, 72 KB at 32) */
    static constexpr uint32_t KC_MAX = HD == 64 ? 128u : 256u;
    static constexpr int PIECES = (int)(KC_MAX * LPR4 / THREADS); /* 16-byte pieces per thread and matrix */
    static constexpr uint32_t RPP = THREADS / LPR4;               /* rows per piece                      */
    /* a fill is parked and worked on in two stages where each wave finds a unit in either (eight
     * waves, two halves); with sixteen waves on one half a stage would leave half of them idle */
    static constexpr int STAGES = WAVES == 8 ? 2 : 1;
    static constexpr int MERGE_FLOATS = WAVES * 16 * ROW; /* one partial tile of 16 rows per wave */
    /* keys a fill holds at least: the merge overlays it */
    static constexpr uint32_t MIN_FILL = (MERGE_FLOATS + 2 * ROW - 1) / (2 * ROW);
    static_assert(PIECES * THREADS == KC_MAX * LPR4 && PIECES % STAGES == 0, "pieces tile the fill");
    static_assert(MIN_FILL % 16 == 0 && MIN_FILL <= KC_MAX, "the merge fits the smallest fill");
};

/* Query tile of the o-th workgroup of a problem with nqt tiles: the long tiles of a causal problem
 * first, and tile t at the same distance from the start of its half of the order as tile
 * nqt - 1 - t, so that workgroups dispatched half a launch apart add up to the same work. */
__device__ __forceinline__ uint32_t fine_tile_order(uint32_t o, uint32_t nqt) {
    const uint32_t first_half = (nqt + 1u) / 2u;
    return o < first_half ? nqt - 1u - o : o - first_half;
}

/* Keys row i sees, [lo, hi), for the two visibility kinds the kernel takes; selects only. */
__device__ __forceinline__ void fine_row_range(const AttnProb &p, uint32_t i, uint32_t &lo, uint32_t &hi) {
    const bool causal = p.vis == ATTN_VIS_CAUSAL;
    const uint32_t diag1 = i + p.causal_off + 1u; /* below 2^32: both terms are below 2^31 */
    hi = causal ? min(p.nk, diag1) : p.nk;
    lo = causal && p.window > 0u && diag1 > p.window ? min(diag1 - p.window, p.nk) : 0u;
    lo = min(lo, hi);
}

/* Key span of rows [first, last]: keys any of them sees [tlo, thi) (thi <= tlo: none) and keys all of
 * them see [flo, fhi); both ends of a row's range grow with the row. */
__device__ __forceinline__ void fine_span(const AttnProb &p, uint32_t first, uint32_t last, uint32_t &tlo, uint32_t &thi,
                                          uint32_t &flo, uint32_t &fhi) {
    uint32_t lo_a, hi_a, lo_b, hi_b;
    fine_row_range(p, first, lo_a, hi_a);
    fine_row_range(p, last, lo_b, hi_b);
    const bool any = hi_a > lo_a;
    tlo = any ? lo_a : 0xFFFFFFFFu, thi = any ? hi_b : 0u;
    flo = lo_b, fhi = hi_a;
}

/* The V operands of one key for this lane: row i of tile e of O^T is column DT i + e of the head,
 * so the lane's DT operands are consecutive floats, one 8- or 16-byte LDS read (vrow points at
 * column DT c of the key's row). */
template <int DT>
__device__ __forceinline__ void fine_v_operands(const float *vrow, float (&vf)[DT][4], const int r) {
    if constexpr (DT == 2) {
        const float2 t = *reinterpret_cast<const float2 *>(vrow);
        vf[0][r] = t.x, vf[1][r] = t.y;
    } else {
        static_assert(DT == 4, "head widths 32 and 64");
        const float4 t = *reinterpret_cast<const float4 *>(vrow);
        vf[0][r] = t.x, vf[1][r] = t.y, vf[2][r] = t.z, vf[3][r] = t.w;
    }
}

/* The finished columns DT (4 g + r) + e of a query row, from accumulators oacc[e][r] scaled by f:
 * the 4 DT consecutive floats from column 4 DT g on, written to dst (which points there). */
template <int DT>
__device__ __forceinline__ void fine_store_columns(float *dst, const floatx4 (&oacc)[DT], const float f) {
    if constexpr (DT == 2) {
#pragma unroll
        for (int r = 0; r < 4; r += 2)
            *reinterpret_cast<float4 *>(dst + 2 * r) =
                make_float4(oacc[0][r] * f, oacc[1][r] * f, oacc[0][r + 1] * f, oacc[1][r + 1] * f);
    } else {
#pragma unroll
        for (int r = 0; r < 4; r++)
            *reinterpret_cast<float4 *>(dst + 4 * r) =
                make_float4(oacc[0][r] * f, oacc[1][r] * f, oacc[2][r] * f, oacc[3][r] * f);
    }
}

/* One unit: 16 query rows (fragment qf, pre-loaded) against the 16 keys whose K rows start at
 * krow (this lane: row c, columns g*HD/4 ...) and whose V rows start at vrow (this lane: rows 4 g + r, columns HD/16 c ...,
 * column c) in LDS, rows ROW = HD + 4 floats apart.  Register r of the lane's scores is key
 * 4 g + r of the tile; that key is visible iff rel + r < len (unsigned: rel = the key's offset
 * into the row's range).  Running maximum m (log2 units), sum l and O^T accumulators are updated. */
template <int HD>
__device__ __forceinline__ void fine_unit(const float *krow, const float *vrow, const float (&qf)[HD / 4],
                                          floatx4 (&oacc)[HD / 16], float &m, float &l, const uint32_t rel,
                                          const uint32_t len, const float scale2) {
    constexpr int QD = HD / 4, DT = HD / 16, ROW = HD + 4;
    float kf[QD];
#pragma unroll
    for (int s = 0; s < QD; s += 4) {
        const float4 t = *reinterpret_cast<const float4 *>(krow + s);
        kf[s + 0] = t.x, kf[s + 1] = t.y, kf[s + 2] = t.z, kf[s + 3] = t.w;
    }
    float vf[DT][4];
#pragma unroll
    for (int r = 0; r < 4; r++) fine_v_operands<DT>(vrow + r * ROW, vf, r);

    /* S^T on two accumulators: neither chain waits for its own previous result */
    floatx4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < QD; s += 2) {
        s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[s], qf[s], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[s + 1], qf[s + 1], s1, 0, 0, 0);
    }

    float x[4];
    float mt = neg_inf();
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const float t = (s0[r] + s1[r]) * scale2;
        const bool vis = ((rel + r) < len) & isfinite(t);
        x[r] = vis ? t : neg_inf();
        mt = fmaxf(mt, x[r]);
    }
    mt = swap32(swap16(mt, OpMax()), OpMax());
    const float mn = fmaxf(m, mt);
    const float ms = mn == neg_inf() ? 0.f : mn;
    const float alpha = fast_exp2(m - ms);
    float ps = 0.f;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        x[r] = fast_exp2(x[r] - ms);
        ps += x[r];
    }
    l = l * alpha + ps;
    m = mn;
#pragma unroll
    for (int d = 0; d < DT; d++)
#pragma unroll
        for (int r = 0; r < 4; r++) oacc[d][r] *= alpha;
#pragma unroll
    for (int r = 0; r < 4; r++)
#pragma unroll
        for (int d = 0; d < DT; d++) oacc[d] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[d][r], x[r], oacc[d], 0, 0, 0);
}

/* Two units of the same query rows side by side -- key tiles at (krow0, vrow0) and (krow1, vrow1),
 * each with a running state of its own -- written out interleaved, so that one unit's softmax
 * arithmetic fills the time the other's matrix instructions take.  The two states are merged by
 * the caller (fine_merge_states). */
template <int HD>
__device__ __forceinline__ void fine_unit2(const float *krow0, const float *vrow0, const float *krow1, const float *vrow1,
                                           const float (&qf)[HD / 4], floatx4 (&oa)[HD / 16], float &ma, float &la,
                                           floatx4 (&ob)[HD / 16], float &mb, float &lb, const uint32_t rel0,
                                           const uint32_t rel1, const uint32_t len, const float scale2) {
    constexpr int QD = HD / 4, DT = HD / 16, ROW = HD + 4;
    float ka[QD], kb[QD];
#pragma unroll
    for (int s = 0; s < QD; s += 4) {
        const float4 t = *reinterpret_cast<const float4 *>(krow0 + s);
        const float4 u = *reinterpret_cast<const float4 *>(krow1 + s);
        ka[s + 0] = t.x, ka[s + 1] = t.y, ka[s + 2] = t.z, ka[s + 3] = t.w;
        kb[s + 0] = u.x, kb[s + 1] = u.y, kb[s + 2] = u.z, kb[s + 3] = u.w;
    }
    float va[DT][4], vb[DT][4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        fine_v_operands<DT>(vrow0 + r * ROW, va, r);
        fine_v_operands<DT>(vrow1 + r * ROW, vb, r);
    }

    floatx4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < QD; s++) {
        sa = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[s], qf[s], sa, 0, 0, 0);
        sb = __builtin_amdgcn_mfma_f32_16x16x4f32(kb[s], qf[s], sb, 0, 0, 0);
    }

    float xa[4], xb[4];
    float ta = neg_inf(), tb = neg_inf();
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const float a = sa[r] * scale2, b = sb[r] * scale2;
        xa[r] = (((rel0 + r) < len) & isfinite(a)) ? a : neg_inf();
        xb[r] = (((rel1 + r) < len) & isfinite(b)) ? b : neg_inf();
        ta = fmaxf(ta, xa[r]), tb = fmaxf(tb, xb[r]);
    }
    ta = swap32(swap16(ta, OpMax()), OpMax());
    tb = swap32(swap16(tb, OpMax()), OpMax());
    const float na = fmaxf(ma, ta), nb = fmaxf(mb, tb);
    const float za = na == neg_inf() ? 0.f : na, zb = nb == neg_inf() ? 0.f : nb;
    const float fa = fast_exp2(ma - za), fb = fast_exp2(mb - zb);
    float pa = 0.f, pb = 0.f;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        xa[r] = fast_exp2(xa[r] - za), xb[r] = fast_exp2(xb[r] - zb);
        pa += xa[r], pb += xb[r];
    }
    la = la * fa + pa, lb = lb * fb + pb;
    ma = na, mb = nb;
#pragma unroll
    for (int d = 0; d < DT; d++)
#pragma unroll
        for (int r = 0; r < 4; r++) oa[d][r] *= fa, ob[d][r] *= fb;
#pragma unroll
    for (int r = 0; r < 4; r++)
#pragma unroll
        for (int d = 0; d < DT; d++) {
            oa[d] = __builtin_amdgcn_mfma_f32_16x16x4f32(va[d][r], xa[r], oa[d], 0, 0, 0);
            ob[d] = __builtin_amdgcn_mfma_f32_16x16x4f32(vb[d][r], xb[r], ob[d], 0, 0, 0);
        }
}

/* state b folded into state a (log2-unit maxima) */
template <int DT>
__device__ __forceinline__ void fine_merge_states(floatx4 (&oa)[DT], float &ma, float &la, const floatx4 (&ob)[DT],
                                                  const float mb, const float lb) {
    const float mn = fmaxf(ma, mb);
    const float ms = mn == neg_inf() ? 0.f : mn;
    const float fa = fast_exp2(ma - ms), fb = fast_exp2(mb - ms);
    la = la * fa + lb * fb;
    ma = mn;
#pragma unroll
    for (int d = 0; d < DT; d++)
#pragma unroll
        for (int r = 0; r < 4; r++) oa[d][r] = oa[d][r] * fa + ob[d][r] * fb;
}

template <int HD, int SRC, int HALVES, int WAVES>
__global__ __launch_bounds__(64 * WAVES, 4) void attn_fine_kernel(const AttnProb *__restrict__ probs,
                                                                  const AttnTile *__restrict__ tiles, AttnAffine aff,
                                                                  uint32_t kc) {
    using Shape = FineShape<HD, HALVES, WAVES>;
    constexpr uint32_t FINE_THREADS = Shape::THREADS;
    constexpr uint32_t ROWS = 16u * HALVES; /* query rows of a workgroup            */
    constexpr uint32_t WPH = WAVES / HALVES; /* waves of a row half (a power of two) */
    constexpr int ROW = Shape::ROW;
    constexpr int LPR4 = Shape::LPR4;
    constexpr int QD = HD / 4;  /* columns of the head one lane group contracts */
    constexpr int DT = HD / 16; /* 16-row tiles of O^T */

    extern __shared__ __attribute__((aligned(16))) float sm[];
    float *const sm_k = sm;
    float *const sm_v = sm + (size_t)kc * ROW;
    float *const sm_q = sm + (size_t)2 * kc * ROW; /* the tile's query rows, ROWS x ROW */

    if (SRC != SRC_TILES) {
        /* every kernel argument the workgroup will read is asked for here, in one go: left to
         * itself the compiler fetches them group by group where they are first needed, and each
         * group is a round trip through a cold scalar cache */
        asm volatile("" ::"s"(aff.first.q), "s"(aff.first.k), "s"(aff.first.v), "s"(aff.first.out), "s"(aff.first.lse));
        asm volatile("" ::"s"(aff.first.q_stride), "s"(aff.first.k_stride), "s"(aff.first.v_stride),
                     "s"(aff.first.out_stride), "s"(aff.first.nq), "s"(aff.first.nk), "s"(aff.first.vis),
                     "s"(aff.first.causal_off), "s"(aff.first.window), "s"(aff.first.scale));
        asm volatile("" ::"s"(aff.q_seq), "s"(aff.q_head), "s"(aff.k_seq), "s"(aff.k_head), "s"(aff.v_seq),
                     "s"(aff.v_head), "s"(aff.o_seq), "s"(aff.o_head), "s"(aff.lse_seq), "s"(aff.lse_head));
        asm volatile("" ::"s"(aff.count), "s"(aff.heads), "s"(aff.nqt), "s"(kc));
    }
    uint32_t qtile;
    AttnProb p;
    if (SRC == SRC_TILES) {
        qtile = tiles[blockIdx.x].qtile;
        p = probs[tiles[blockIdx.x].prob];
    } else if (SRC == SRC_SINGLE) {
        qtile = fine_tile_order(blockIdx.x, gridDim.x);
        p = aff.first;
    } else {
        const uint32_t prob = blockIdx.x % aff.count;
        qtile = fine_tile_order(blockIdx.x / aff.count, (aff.first.nq + ROWS - 1u) / ROWS);
        affine_problem(p, aff, prob, false);
    }

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t half = HALVES == 1 ? 0u : wave / WPH; /* row half of the tile */
    const uint32_t wi = wave & (WPH - 1u);               /* wave of the row half */
    const uint32_t g = lane >> 4;
    const uint32_t c = lane & 15u;

    const uint32_t q0 = qtile * ROWS;
    const uint32_t last_row = min(q0 + ROWS - 1u, p.nq - 1u);

    /* keys the tile needs, as 16-key tiles [t0, t1) */
    uint32_t tlo, thi, flo, fhi;
    fine_span(p, q0, last_row, tlo, thi, flo, fhi);
    const uint32_t t0 = thi > tlo ? tlo / 16u : 0u;
    const uint32_t t1 = thi > tlo ? (thi + 15u) / 16u : 0u;

    /* this wave's row half: its own key tiles [my0, my1) */
    uint32_t my0 = 0, my1 = 0;
    {
        const uint32_t first = q0 + 16u * half;
        uint32_t lo_a, hi_a, f0, f1;
        fine_span(p, min(first, p.nq - 1u), min(first + 15u, p.nq - 1u), lo_a, hi_a, f0, f1);
        if (first < p.nq && hi_a > lo_a) my0 = lo_a / 16u, my1 = (hi_a + 15u) / 16u;
    }
    /* this wave's key tiles: kt = wi - 2 half (mod WPH), one in every WPH; with two halves of four
     * waves the units a stage of 32 keys completes (two key tiles, two row halves) fall on four
     * different SIMDs */
    uint32_t kt = my0 + ((wi - 2u * half - my0) & (WPH - 1u));

    /* this lane's query row and what it sees */
    const uint32_t row = q0 + 16u * half + c;
    const bool live = row < p.nq;
    const uint32_t qi = live ? row : p.nq - 1u;
    uint32_t lo, hi;
    fine_row_range(p, qi, lo, hi);
    if (!live) hi = lo;
    /* keys every row of the half sees whole: no per-key test on those tiles */
    uint32_t half_flo, half_fhi;
    {
        const uint32_t first = min(q0 + 16u * half, p.nq - 1u);
        uint32_t a_, b_;
        fine_span(p, first, min(first + 15u, p.nq - 1u), a_, b_, half_flo, half_fhi);
        if (q0 + 16u * half + 15u >= p.nq) half_fhi = half_flo; /* padding rows see nothing */
    }
    const float scale2 = p.scale * LOG2E;

    floatx4 oacc[DT];
#pragma unroll
    for (int d = 0; d < DT; d++)
#pragma unroll
        for (int r = 0; r < 4; r++) oacc[d][r] = 0.f;
    float m = neg_inf(), l = 0.f;

    /* The tile's query rows: one 16-byte piece per thread, consecutive lanes on consecutive pieces of
     * a row (a load whose lanes each touch another row is served at a quarter of the rate, and a
     * fragment read straight from global memory is such a load), parked with the first stage's
     * rows and read back as fragments -- row c of the half, columns [g*QD, (g+1)*QD) -- after the
     * barrier that stage has anyway.  Threads past the tile's pieces repeat one (no branch around
     * the request) and park nothing. */
    constexpr uint32_t QPIECES = ROWS * (uint32_t)LPR4;
    static_assert(QPIECES <= FINE_THREADS, "one query piece per thread at most");
    float qf[QD];
    const uint32_t qe = tid % QPIECES;
    const floatx4 q_piece = *reinterpret_cast<const floatx4 *>(
        p.q + (size_t)min(q0 + qe / LPR4, p.nq - 1u) * p.q_stride + 4u * (qe % LPR4));
    bool q_ready = false; /* uniform: the fragment has been read */

    /* ---- fill: rows [c0, c0 + kc) of K and V, clamped to the last row the tile needs; the first
     * fill is requested here, the later ones at the end of the loop's body, so that nothing at the
     * head of the loop waits for what the previous round left in flight ---- */
    const uint32_t key_end = t1 * 16u;
    const uint32_t last_key = min(max(key_end, 1u), p.nk) - 1u; /* row 0 when the tile sees nothing */
    float4 kp[Shape::PIECES], vp[Shape::PIECES];
    auto request = [&](uint32_t c0) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < Shape::PIECES; t++) {
            const uint32_t e = tid + FINE_THREADS * t;
            const uint32_t r = e / LPR4, f = e % LPR4;
            const uint32_t j = min(c0 + r, last_key);
            kp[t] = *reinterpret_cast<const float4 *>(p.k + (size_t)j * p.k_stride + 4u * f);
            vp[t] = *reinterpret_cast<const float4 *>(p.v + (size_t)j * p.v_stride + 4u * f);
        }
    };
    uint32_t c0 = t0 * 16u;
    request(c0); /* unconditionally: a branch here would make the code after it wait for every request */
    /* the query piece is parked here, where the compiler still counts the requests in flight one by
     * one: inside the loops below a use of a value that is still on its way makes it wait for every
     * request, the later pieces of the fill included */
    if (tid < QPIECES) *reinterpret_cast<floatx4 *>(sm_q + (qe / LPR4) * ROW + 4u * (qe % LPR4)) = q_piece;
    while (c0 < key_end) {
        /* ---- the pieces land in the order they were requested: piece by piece, park it and work
         * on the key tiles it completes while the later pieces are still on their way ---- */
        const uint32_t fill_end = min(c0 + kc, key_end);
        constexpr uint32_t RPP = Shape::RPP; /* rows per piece */
        auto park = [&](const uint32_t pc, const float4 k_piece, const float4 v_piece) __attribute__((always_inline)) {
            const uint32_t e = tid + FINE_THREADS * pc;
            const uint32_t r = e / LPR4, f = e % LPR4;
            /* no test (and nothing for the compiler to sink the piece's loads behind) on the pieces
             * below what every fill holds */
            if (RPP * (pc + 1u) <= Shape::MIN_FILL || r < kc) {
                *reinterpret_cast<float4 *>(sm_k + r * ROW + 4u * f) = k_piece;
                *reinterpret_cast<float4 *>(sm_v + r * ROW + 4u * f) = v_piece;
            }
        };
        /* one stage = the units of the key tiles that pieces [0, pieces_done) complete */
        auto stage = [&](const uint32_t pieces_done) __attribute__((always_inline)) {
            __syncthreads();
            if (!q_ready) { /* first barrier of the workgroup: the query rows are parked */
                const float *qrow = sm_q + (16u * half + c) * ROW + g * QD;
#pragma unroll
                for (int s = 0; s < QD; s += 4) {
                    const float4 t = *reinterpret_cast<const float4 *>(qrow + s);
                    qf[s + 0] = t.x, qf[s + 1] = t.y, qf[s + 2] = t.z, qf[s + 3] = t.w;
                }
                q_ready = true;
            }
            const uint32_t stage_end = min(c0 + RPP * pieces_done, fill_end);
            while (kt < my1 && kt * 16u < stage_end) {
                const uint32_t k0 = kt * 16u;
                const float *krow = sm_k + (k0 - c0 + c) * ROW + g * QD;
                const float *vrow = sm_v + (k0 - c0 + 4u * g) * ROW + DT * c;
                const bool all_seen = k0 >= half_flo && k0 + 16u <= half_fhi; /* uniform over the wave */
                fine_unit<HD>(krow, vrow, qf, oacc, m, l, k0 + 4u * g - (all_seen ? 0u : lo),
                              all_seen ? 0xFFFFFFFFu : (hi > lo ? hi - lo : 0u), scale2);
                kt += WPH;
            }
            return c0 + RPP * pieces_done < fill_end; /* more keys to come: uniform over the workgroup */
        };
        /* The next fill is requested as soon as this one has left the registers, before the last
         * stage's units start (past the end of the keys the requests repeat the last row: no branch
         * around them).  The two fills' requests never overlap in the registers. */
        constexpr int PPS = Shape::PIECES / Shape::STAGES;
#pragma unroll
        for (int t = 0; t < PPS; t++) park(t, kp[t], vp[t]);
        if (Shape::STAGES == 1) {
            request(c0 + kc);
            stage(Shape::PIECES);
        } else if (stage(PPS)) {
#pragma unroll
            for (int t = PPS; t < Shape::PIECES; t++) park(t, kp[t], vp[t]);
            request(c0 + kc);
            stage(Shape::PIECES);
        }
        __syncthreads(); /* the fill is consumed: the next fill, or the merge, may overwrite it */
        c0 += kc;
    }

    /* the four lane groups of a column carry the same m, their sums add */
    l = swap32(swap16(l, OpSum()), OpSum());

    /* ---- merge: every wave parks [16 queries][HD columns, max, sum] ---- */
    float *mine = sm + wave * (16 * ROW);
    fine_store_columns<DT>(mine + c * ROW + 4 * DT * g, oacc, 1.0f);
    if (g == 0) *reinterpret_cast<float2 *>(mine + c * ROW + HD) = make_float2(m, l);
    __syncthreads();

    /* the threads of a row half: thread = (row, 16-byte piece of the row) */
    constexpr uint32_t TPH = FINE_THREADS / HALVES;
    const uint32_t mh = HALVES == 1 ? 0u : tid / TPH, idx = tid % TPH;
    const uint32_t mr = idx / LPR4, mf = idx % LPR4;
    if (mr < 16u) {
        const float *part = sm + (WPH * mh) * (16 * ROW) + mr * ROW;
        float pm[WPH], pl[WPH];
        float M = neg_inf();
#pragma unroll
        for (int w = 0; w < (int)WPH; w++) {
            const float2 t = *reinterpret_cast<const float2 *>(part + w * (16 * ROW) + HD);
            pm[w] = t.x, pl[w] = t.y;
            M = fmaxf(M, pm[w]);
        }
        const float Ms = M == neg_inf() ? 0.f : M;
        float L = 0.f;
        float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int w = 0; w < (int)WPH; w++) {
            const float f = fast_exp2(pm[w] - Ms);
            const float4 t = *reinterpret_cast<const float4 *>(part + w * (16 * ROW) + 4u * mf);
            L += pl[w] * f;
            o.x += t.x * f, o.y += t.y * f, o.z += t.z * f, o.w += t.w * f;
        }
        const float inv = L > 0.f ? 1.0f / L : 0.f;
        const uint32_t orow = q0 + 16u * mh + mr;
        if (orow < p.nq) {
            *reinterpret_cast<float4 *>(p.out + (size_t)orow * p.out_stride + 4u * mf) =
                make_float4(o.x * inv, o.y * inv, o.z * inv, o.w * inv);
            if (mf == 0 && p.lse) {
                p.lse[2 * (size_t)orow + 0] = M * LN2; /* back to natural units */
                p.lse[2 * (size_t)orow + 1] = L;
            }
        }
    }
}

/* Whole short problems (at most 128 query rows, keys that fit one fill), for strided batches of
 * so many of them that throughput matters and the launch floor does not: the workgroup -- eight
 * waves -- fetches the problem's K and V rows ONCE into LDS, meets once, and from there on its
 * waves run on their own.  A wave takes one row half (of 16 rows): wave w the half n-1-w, wave
 * w + 4, which shares its SIMD, the half w -- under a causal mask the two add up to the same
 * number of units on every SIMD, and a half's keys are all the wave's own, so nothing is merged;
 * the finished rows go to global memory straight from the accumulators.  Two workgroups fit a
 * compute unit (LDS), four waves on every SIMD: a wave's softmax and LDS waits are another's
 * matrix instructions (four waves of two halves each, one after the other: 22.5 / 36.3 / 72.5 us
 * at 512 / 1024 / 2048 problems of 128 rows x 64 columns against 20.4 / 35.2 / 62.0 now). */
template <int HD>
struct WholeShape {
    static constexpr uint32_t THREADS = 512;
    static constexpr uint32_t MAX_ROWS = 128;
    static constexpr uint32_t KC_MAX = FineShape<HD, 2, 8>::KC_MAX;
    static constexpr int ROW = HD + 4, LPR4 = HD / 4;
    static constexpr int PIECES = (int)(KC_MAX * LPR4 / THREADS);
};

template <int HD>
__global__ __launch_bounds__(512, 2) void attn_whole_kernel(AttnAffine aff, uint32_t kc) {
    using Shape = WholeShape<HD>;
    constexpr int ROW = Shape::ROW, LPR4 = Shape::LPR4, QD = HD / 4, DT = HD / 16;
    extern __shared__ __attribute__((aligned(16))) float sm[];
    float *const sm_k = sm;
    float *const sm_v = sm + (size_t)kc * ROW;

    asm volatile("" ::"s"(aff.first.q), "s"(aff.first.k), "s"(aff.first.v), "s"(aff.first.out), "s"(aff.first.lse));
    asm volatile("" ::"s"(aff.first.q_stride), "s"(aff.first.k_stride), "s"(aff.first.v_stride),
                 "s"(aff.first.out_stride), "s"(aff.first.nq), "s"(aff.first.nk), "s"(aff.first.vis),
                 "s"(aff.first.causal_off), "s"(aff.first.window), "s"(aff.first.scale));
    asm volatile("" ::"s"(aff.q_seq), "s"(aff.q_head), "s"(aff.k_seq), "s"(aff.k_head), "s"(aff.v_seq), "s"(aff.v_head),
                 "s"(aff.o_seq), "s"(aff.o_head), "s"(aff.lse_seq), "s"(aff.lse_head));
    asm volatile("" ::"s"(aff.count), "s"(aff.heads), "s"(kc));
    AttnProb p;
    affine_problem(p, aff, blockIdx.x, false);

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t g = lane >> 4, c = lane & 15u;
    const uint32_t halves = (p.nq + 15u) / 16u; /* at most 8 */

    /* keys the problem needs: rows [c0, key_end), at most kc of them */
    uint32_t tlo, thi, flo, fhi;
    fine_span(p, 0u, p.nq - 1u, tlo, thi, flo, fhi);
    const uint32_t c0 = thi > tlo ? tlo / 16u * 16u : 0u;
    const uint32_t key_end = thi > tlo ? (thi + 15u) / 16u * 16u : 0u;
    const uint32_t last_key = min(max(key_end, 1u), p.nk) - 1u;

    /* The wave's row half, NONE: nothing.  Waves w and w + 4 sit on one SIMD: w takes half n-1-w, w + 4
     * takes half w, which under a causal mask add up to the same number of units on every SIMD. */
    constexpr uint32_t NONE = 0xFFFFFFFFu;
    const uint32_t pw = wave & 3u;
    const uint32_t far = pw < halves && halves - 1u - pw >= pw ? halves - 1u - pw : NONE;
    const uint32_t ha = wave < 4u ? far : (far != NONE && far > pw ? pw : NONE);

    auto load_q = [&](float (&qf)[QD], const uint32_t half) __attribute__((always_inline)) {
        const uint32_t row = min(16u * (half == NONE ? 0u : half) + c, p.nq - 1u);
        const float *qrow = p.q + (size_t)row * p.q_stride + g * QD;
#pragma unroll
        for (int s = 0; s < QD; s += 4) {
            const float4 t = *reinterpret_cast<const float4 *>(qrow + s);
            qf[s + 0] = t.x, qf[s + 1] = t.y, qf[s + 2] = t.z, qf[s + 3] = t.w;
        }
    };
    float qa[QD];
    load_q(qa, ha);

    /* ---- the fill: every piece is requested, then parked in the order it was requested ---- */
    float4 kp[Shape::PIECES], vp[Shape::PIECES];
#pragma unroll
    for (int t = 0; t < Shape::PIECES; t++) {
        const uint32_t e = tid + Shape::THREADS * t;
        const uint32_t r = e / LPR4, f = e % LPR4;
        const uint32_t j = min(c0 + r, last_key);
        kp[t] = *reinterpret_cast<const float4 *>(p.k + (size_t)j * p.k_stride + 4u * f);
        vp[t] = *reinterpret_cast<const float4 *>(p.v + (size_t)j * p.v_stride + 4u * f);
    }
#pragma unroll
    for (int s = 0; s < QD; s++) asm volatile("" : "+v"(qa[s]));
    /* the pieces go to the lambda by value: indexed inside it, the arrays would live in scratch memory */
    auto park = [&](const uint32_t pc, const float4 k_piece, const float4 v_piece) __attribute__((always_inline)) {
        const uint32_t e = tid + Shape::THREADS * pc;
        const uint32_t r = e / LPR4, f = e % LPR4;
        if (r < kc) {
            *reinterpret_cast<float4 *>(sm_k + r * ROW + 4u * f) = k_piece;
            *reinterpret_cast<float4 *>(sm_v + r * ROW + 4u * f) = v_piece;
        }
    };
#pragma unroll
    for (int t = 0; t < Shape::PIECES; t++) park(t, kp[t], vp[t]);
    __syncthreads(); /* the only one: from here on no wave waits for another */

    const float scale2 = p.scale * LOG2E;
    auto run_half = [&](const float (&qf)[QD], const uint32_t half) __attribute__((always_inline)) {
        const uint32_t first = 16u * half;
        const uint32_t row = first + c;
        const bool live = row < p.nq;
        uint32_t lo, hi;
        fine_row_range(p, live ? row : p.nq - 1u, lo, hi);
        if (!live) hi = lo;
        /* key tiles of the half: [my0, my1) */
        uint32_t lo_a, hi_a, all_lo, all_hi;
        fine_span(p, first, min(first + 15u, p.nq - 1u), lo_a, hi_a, all_lo, all_hi);
        (void)all_lo, (void)all_hi;
        const uint32_t my0 = hi_a > lo_a ? lo_a / 16u : 0u, my1 = hi_a > lo_a ? (hi_a + 15u) / 16u : 0u;

        floatx4 oacc[DT];
#pragma unroll
        for (int d = 0; d < DT; d++)
#pragma unroll
            for (int r = 0; r < 4; r++) oacc[d][r] = 0.f;
        float m = neg_inf(), l = 0.f;
        /* key tiles two at a time on two running states, folded together at the end */
        floatx4 oodd[DT];
#pragma unroll
        for (int d = 0; d < DT; d++)
#pragma unroll
            for (int r = 0; r < 4; r++) oodd[d][r] = 0.f;
        float modd = neg_inf(), lodd = 0.f;
        const uint32_t vlen = hi > lo ? hi - lo : 0u;
        uint32_t kt = my0;
        for (; kt + 1u < my1; kt += 2u) {
            const uint32_t k0 = kt * 16u;
            const float *krow = sm_k + (k0 - c0 + c) * ROW + g * QD;
            const float *vrow = sm_v + (k0 - c0 + 4u * g) * ROW + DT * c;
            fine_unit2<HD>(krow, vrow, krow + 16 * ROW, vrow + 16 * ROW, qf, oacc, m, l, oodd, modd, lodd,
                           k0 + 4u * g - lo, k0 + 16u + 4u * g - lo, vlen, scale2);
        }
        if (kt < my1) {
            const uint32_t k0 = kt * 16u;
            const float *krow = sm_k + (k0 - c0 + c) * ROW + g * QD;
            const float *vrow = sm_v + (k0 - c0 + 4u * g) * ROW + DT * c;
            fine_unit<HD>(krow, vrow, qf, oacc, m, l, k0 + 4u * g - lo, vlen, scale2);
        }
        fine_merge_states<DT>(oacc, m, l, oodd, modd, lodd);
        /* the four lane groups of a column carry the same m, their sums add; lane (g, c) holds
         * the HD/4 consecutive columns from (HD/4) g on of query row c */
        l = swap32(swap16(l, OpSum()), OpSum());
        if (!live) return;
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        fine_store_columns<DT>(p.out + (size_t)row * p.out_stride + 4u * DT * g, oacc, inv);
        if (g == 0 && p.lse) {
            p.lse[2 * (size_t)row + 0] = m * LN2; /* back to natural units */
            p.lse[2 * (size_t)row + 1] = l;
        }
    };
    if (ha != NONE) run_half(qa, ha);
}

/* keys per fill for a launch whose longest tile needs `span` keys */
template <typename Shape>
uint32_t fine_fill_keys(uint32_t span) {
    const uint32_t want = std::max<uint32_t>(16u, (span + 15u) / 16u * 16u + 16u); /* a span may straddle a tile */
    return std::min<uint32_t>(Shape::KC_MAX, std::max<uint32_t>(Shape::MIN_FILL, want));
}

template <int HD, int SRC, int HALVES, int WAVES>
void fine_launch_as(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t nblocks, const AttnAffine &aff,
                    uint32_t span, hipStream_t s) {
    using Shape = FineShape<HD, HALVES, WAVES>;
    const uint32_t kc = fine_fill_keys<Shape>(span);
    /* K and V rows of a fill, then the tile's query rows */
    const size_t lds = ((size_t)2 * kc + 16u * HALVES) * Shape::ROW * sizeof(float);
    static const bool raised = [] { /* more than the 64 KB a kernel may use without asking */
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_fine_kernel<HD, SRC, HALVES, WAVES>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize,
                                      (2 * (int)Shape::KC_MAX + 16 * HALVES) * Shape::ROW * (int)sizeof(float)));
        return true;
    }();
    (void)raised;
    blt_launch("attn_fine", attn_fine_kernel<HD, SRC, HALVES, WAVES>, dim3(nblocks), dim3(Shape::THREADS), lds, s,
               dprobs, dtiles, aff, kc);
}

/* tall: workgroups of one 16-row tile and sixteen waves (strided batches and single problems) */
template <int SRC>
void fine_launch_hd(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t nblocks, const AttnAffine &aff,
                    uint32_t hd, uint32_t span, bool tall, hipStream_t s) {
    if constexpr (SRC != SRC_TILES) {
        if (tall) {
            if (hd == 32u) fine_launch_as<32, SRC, 1, 16>(dprobs, dtiles, nblocks, aff, span, s);
            else fine_launch_as<64, SRC, 1, 16>(dprobs, dtiles, nblocks, aff, span, s);
            return;
        }
    }
    if (hd == 32u) fine_launch_as<32, SRC, 2, 8>(dprobs, dtiles, nblocks, aff, span, s);
    else fine_launch_as<64, SRC, 2, 8>(dprobs, dtiles, nblocks, aff, span, s);
}

} // namespace

/* Keys the longest 32-row tile of the problem needs. */
uint32_t attn_fine_span(const AttnProb &d) {
    if (d.vis != ATTN_VIS_CAUSAL) return d.nk;
    if (d.window > 0) return std::min<uint64_t>(d.nk, (uint64_t)d.window + 31u);
    return (uint32_t)std::min<uint64_t>(d.nk, (uint64_t)d.nq + d.causal_off);
}

/* keys one LDS fill holds at head width hd */
uint32_t attn_fine_fill_max(uint32_t hd) { return hd == 32u ? FineShape<32, 2, 8>::KC_MAX : FineShape<64, 2, 8>::KC_MAX; }

/* shapes the kernel is able to run */
bool attn_fine_can(const AttnProb &d) {
    return (d.hd == 32u || d.hd == 64u) && (d.flags & ATTN_FLAG_VEC4) != 0 && d.weights == nullptr &&
           (d.vis == ATTN_VIS_ALL || d.vis == ATTN_VIS_CAUSAL) && d.nq >= 1u && d.nk >= 1u;
}

/* Work items for problems [base, base+count), longest first. */
void attn_fine_make_tiles(const AttnProb *host, uint32_t base, uint32_t count, std::vector<AttnTile> &tiles) {
    attn_mfma_make_tiles(host, base, count, tiles);
}

void attn_fine_launch(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t ntiles, uint32_t hd, uint32_t span,
                      hipStream_t s) {
    if (ntiles == 0) return;
    AttnAffine none;
    __builtin_memset(&none, 0, sizeof(none));
    fine_launch_hd<SRC_TILES>(dprobs, dtiles, ntiles, none, hd, span, false, s);
}

void attn_fine_launch_single(const AttnProb &single, bool tall, hipStream_t s) {
    const uint32_t rows = tall ? 16u : 32u;
    const uint32_t ntiles = (single.nq + rows - 1u) / rows;
    if (ntiles == 0) return;
    AttnAffine a;
    __builtin_memset(&a, 0, sizeof(a));
    a.first = single;
    fine_launch_hd<SRC_SINGLE>(nullptr, nullptr, ntiles, a, single.hd, attn_fine_span(single), tall, s);
}

/* the whole-problem kernel takes strided batches of problems like this one */
bool attn_whole_can(const AttnProb &d) {
    if (!attn_fine_can(d) || d.nq > WholeShape<64>::MAX_ROWS) return false;
    /* keys the rows see, from the first row's first to the last row's last, in 16-key tiles */
    uint64_t lo = 0, hi = d.nk;
    if (d.vis == ATTN_VIS_CAUSAL) {
        hi = std::min<uint64_t>(d.nk, (uint64_t)d.nq + d.causal_off);
        if (d.window > 0 && (uint64_t)d.causal_off + 1u > d.window) lo = std::min<uint64_t>((uint64_t)d.causal_off + 1u - d.window, hi);
    }
    const uint64_t span = (hi + 15u) / 16u * 16u - lo / 16u * 16u;
    return span <= attn_fine_fill_max(d.hd);
}

void attn_whole_launch_affine(const AttnAffine &aff, hipStream_t s) {
    if (aff.count == 0) return;
    const AttnProb &d = aff.first;
    BLT_REQUIRE(attn_whole_can(d), "attention: internal: the whole-problem kernel was given a shape it does not take");
    uint64_t lo = 0, hi = d.nk;
    if (d.vis == ATTN_VIS_CAUSAL) {
        hi = std::min<uint64_t>(d.nk, (uint64_t)d.nq + d.causal_off);
        if (d.window > 0 && (uint64_t)d.causal_off + 1u > d.window) lo = std::min<uint64_t>((uint64_t)d.causal_off + 1u - d.window, hi);
    }
    const uint32_t kc = std::max<uint32_t>(16u, (uint32_t)((hi + 15u) / 16u * 16u - lo / 16u * 16u));
    if (d.hd == 32u) {
        const size_t lds = (size_t)2 * kc * WholeShape<32>::ROW * sizeof(float);
        static const bool raised = [] {
            HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_whole_kernel<32>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize,
                                          2 * (int)WholeShape<32>::KC_MAX * WholeShape<32>::ROW * (int)sizeof(float)));
            return true;
        }();
        (void)raised;
        blt_launch("attn_whole", attn_whole_kernel<32>, dim3(aff.count), dim3(WholeShape<32>::THREADS), lds, s, aff, kc);
    } else {
        const size_t lds = (size_t)2 * kc * WholeShape<64>::ROW * sizeof(float);
        static const bool raised = [] {
            HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_whole_kernel<64>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize,
                                          2 * (int)WholeShape<64>::KC_MAX * WholeShape<64>::ROW * (int)sizeof(float)));
            return true;
        }();
        (void)raised;
        blt_launch("attn_whole", attn_whole_kernel<64>, dim3(aff.count), dim3(WholeShape<64>::THREADS), lds, s, aff, kc);
    }
}

void attn_fine_launch_affine(const AttnAffine &aff, bool tall, hipStream_t s) {
    const uint32_t rows = tall ? 16u : 32u;
    const uint32_t blocks = aff.count * ((aff.first.nq + rows - 1u) / rows);
    if (blocks == 0) return;
    fine_launch_hd<SRC_AFFINE>(nullptr, nullptr, blocks, aff, aff.first.hd, attn_fine_span(aff.first), tall, s);
}
