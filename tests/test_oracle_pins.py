"""Pins the CPU checker WITHOUT the reference build: reference-held vectors,
closed forms, float64 brute force and structural invariants, each chosen so
that a plausible slip (dropped scale, wrong sign, transposed operand, off-by-one
in a mask) fails at least one of them."""
import ctypes as C

import numpy as np
import pytest

from fblt_amd import abi
from oracle import binding


def core(orc, q, k, v, scale, mask=None, causal=False, hd=None, nq=None, nk=None):
    nq = nq or q.shape[0]
    nk = nk or k.shape[0]
    hd = hd or q.shape[1]
    out = np.full((nq, hd), 3.0, dtype=np.float32)
    w = np.full((nq, nk), 3.0, dtype=np.float32)
    a = binding.head_args(q.reshape(-1), k.reshape(-1), v.reshape(-1), out.reshape(-1), nq, nk, hd, scale,
                          q.shape[1], k.shape[1], v.shape[1], hd, 0, weights=w.reshape(-1),
                          mask=None if mask is None else mask.reshape(-1), causal=causal)
    assert orc.orc_attention_head_core(C.byref(a)) == 0
    return out, w


def test_reference_inline_vector(oracle):
    # tests/unit/models/unit_attention.c:24-88 (identity projections => Q=K=V=input slices)
    x = np.array([[1, 0], [0, 1]], dtype=np.float32)
    scale = float(np.float32(1.0) / np.sqrt(np.float32(2.0)))
    out, w = core(oracle, x, x, x, scale)
    assert np.allclose(out, [[0.6697615, 0.3302385], [0.3302385, 0.6697615]], atol=1e-7)
    # causal variants, unit_attention.c:160-184: row 0 is one-hot; mask form == flag form
    out_c, w_c = core(oracle, x, x, x, scale, causal=True)
    assert np.allclose(out_c, [[1, 0], [0.3302385, 0.6697615]], atol=1e-7)
    m = np.array([[0, -np.inf], [0, 0]], dtype=np.float32)
    out_m, w_m = core(oracle, x, x, x, scale, mask=m)
    assert np.array_equal(out_m, out_c) and np.array_equal(w_m, w_c)


def test_two_key_softmax_is_a_sigmoid(oracle):
    rs = np.random.RandomState(0)
    for _ in range(50):
        hd = rs.randint(1, 40)
        q = rs.randn(1, hd).astype(np.float32)
        k = rs.randn(2, hd).astype(np.float32)
        v = np.array([[1.0], [0.0]], dtype=np.float32)
        vv = np.zeros((2, hd), dtype=np.float32)
        vv[:, :1] = v
        scale = float(rs.rand() + 0.1)
        out, w = core(oracle, q, k, vv, scale)
        d = (q.astype(np.float64) @ (k[0] - k[1]).astype(np.float64))[0] * scale
        sig = 1.0 / (1.0 + np.exp(-d))
        assert abs(w[0, 0] - sig) < 2e-6 and abs(out[0, 0] - sig) < 2e-6   # wrong sign => 1 - sig
        assert abs(w.sum() - 1) < 1e-6


def test_uniform_and_single_key_and_dead_rows(oracle):
    rs = np.random.RandomState(1)
    nq, nk, hd = 6, 9, 5
    k = rs.randn(nk, hd).astype(np.float32)
    v = rs.randn(nk, hd).astype(np.float32)
    zero_q = np.zeros((nq, hd), dtype=np.float32)
    out, w = core(oracle, zero_q, k, v, 0.7, causal=True)
    for i in range(nq):  # equal scores: mean of the visible V rows, keys j <= i only
        assert np.allclose(out[i], v[:i + 1].astype(np.float64).mean(0), atol=1e-6)
        assert np.allclose(w[i, :i + 1], 1.0 / (i + 1), atol=1e-7) and (w[i, i + 1:] == 0).all()
    q = rs.randn(nq, hd).astype(np.float32)
    mask = np.full((nq, nk), -np.inf, dtype=np.float32)
    for i in range(nq - 1):
        mask[i, (3 * i) % nk] = 0.0           # exactly one visible key
    out, w = core(oracle, q, k, v, 0.3, mask=mask)
    for i in range(nq - 1):
        assert np.array_equal(out[i], v[(3 * i) % nk])      # weight exactly 1.0 => exact copy
    assert (out[nq - 1] == 0).all() and (w[nq - 1] == 0).all()   # all-masked row: zeros


def test_float64_brute_force(oracle):
    rs = np.random.RandomState(2)
    for trial in range(30):
        nq, nk, hd = rs.randint(1, 9), rs.randint(1, 12), rs.randint(1, 10)
        qs, ks, vs = hd + rs.randint(0, 3), hd + rs.randint(0, 3), hd + rs.randint(0, 3)
        q = rs.randn(nq, qs).astype(np.float32)
        k = rs.randn(nk, ks).astype(np.float32)
        v = rs.randn(nk, vs).astype(np.float32)
        scale = float(rs.rand() * 2)
        mask = np.where(rs.rand(nq, nk) < 0.3, -np.inf, rs.randn(nq, nk)).astype(np.float32)
        out, w = core(oracle, q, k, v, scale, mask=mask, hd=hd)
        s = q[:, :hd].astype(np.float64) @ k[:, :hd].astype(np.float64).T * scale + mask
        for i in range(nq):
            fin = np.isfinite(s[i])
            ref = np.zeros(nk)
            if fin.any():
                e = np.exp(s[i, fin] - s[i, fin].max())
                ref[fin] = e / e.sum()
            assert np.allclose(w[i], ref, atol=2e-6)
            assert np.allclose(out[i], ref @ v[:, :hd].astype(np.float64), atol=5e-6)


def test_nonfinite_scores_are_dropped(oracle):
    # csrc/ops/vecmath_cpu.c:33-46: only finite entries enter the max and the sum
    q = np.array([[1.0, 0.0]], dtype=np.float32)
    k = np.array([[np.inf, 0.0], [1.0, 0.0], [2.0, 0.0]], dtype=np.float32)
    v = np.eye(3, 2, dtype=np.float32)
    out, w = core(oracle, q, k, v, 1.0)
    assert w[0, 0] == 0.0 and abs(w[0, 1] + w[0, 2] - 1) < 1e-6 and w[0, 2] > w[0, 1]


def mask_of(orc, **kw):
    cfg = abi.BltMaskConfig()
    keep = []
    for name, val in kw.items():
        if name in ("doc_boundaries", "query_group_ids", "kv_group_ids"):
            arr = abi.size_array(val)
            keep.append(arr)
            setattr(cfg, name, arr)
        else:
            setattr(cfg, name, val)
    out = np.empty(cfg.seq_len_q * cfg.seq_len_kv, dtype=np.float32)
    rc = orc.orc_build_attention_mask(C.byref(cfg), binding.fptr(out))
    return rc, out.reshape(cfg.seq_len_q, cfg.seq_len_kv) == 0.0, out


def test_mask_builder_reference_cases(oracle):
    # tests/unit/backend/unit_mask.c:14-192
    rc, ok, raw = mask_of(oracle, seq_len_q=4, seq_len_kv=4, is_causal=True)
    assert rc == 0 and (ok == np.tril(np.ones((4, 4), bool))).all()
    assert set(np.unique(raw)) == {0.0, -np.inf}
    rc, ok, _ = mask_of(oracle, seq_len_q=6, seq_len_kv=6, is_causal=True, sliding_window=3)
    assert list(ok[5]) == [False, False, False, True, True, True]
    rc, ok, _ = mask_of(oracle, seq_len_q=6, seq_len_kv=6, doc_boundaries=[3], num_docs=2)
    assert ok[1, 2] and ok[4, 5] and not ok[2, 3] and not ok[5, 0]
    rc, ok, _ = mask_of(oracle, seq_len_q=4, seq_len_kv=4, query_group_ids=[0, 0, 1, 1], kv_group_ids=[0, 0, 1, 1])
    assert not ok[0, 2] and not ok[3, 1] and ok[1, 0] and not ok[0, 1]
    # a row without any key is the reference's abort (mask_builder_cpu.c:93)
    rc, _, _ = mask_of(oracle, seq_len_q=2, seq_len_kv=2, query_group_ids=[0, 5], kv_group_ids=[0, 0],
                       bidirectional_within_group=True)
    assert rc == 4


def test_mask_builder_randomised_predicate(oracle):
    # independent statement of the rule (tests/unit/models/unit_global_transformer.c:121+ style fuzz)
    rs = np.random.RandomState(3)
    for _ in range(60):
        nq, nk = rs.randint(1, 20), rs.randint(1, 20)
        causal, W, off = bool(rs.randint(2)), int(rs.choice([0, 0, 1, 3, 7])), int(rs.choice([0, 0, 2, 5]))
        bounds = sorted(rs.randint(0, max(nq, nk) + 1, size=rs.randint(0, 4)).tolist())
        use_g, bidir = bool(rs.randint(2)), bool(rs.randint(2))
        qg, kg = rs.randint(0, 3, nq).tolist(), rs.randint(0, 3, nk).tolist()
        kw = dict(seq_len_q=nq, seq_len_kv=nk, is_causal=causal, sliding_window=W, causal_offset=off)
        if bounds:
            kw.update(doc_boundaries=bounds, num_docs=len(bounds) + 1)
        if use_g:
            kw.update(query_group_ids=qg, kv_group_ids=kg, bidirectional_within_group=bidir)
        rc, ok, _ = mask_of(oracle, **kw)
        doc = lambda p: sum(1 for b in bounds if p >= b)
        dead = False
        for i in range(nq):
            row_any = False
            for j in range(nk):
                want = True
                if causal and j > i + off:
                    want = False
                if W > 0 and abs((i + off if causal else i) - j) >= W:
                    want = False
                if bounds and doc(i) != doc(j):
                    want = False
                if use_g and (qg[i] != kg[j] or (not bidir and j > i)):
                    want = False
                assert ok[i, j] == want, (kw, i, j)
                row_any |= want
            if not row_any:
                dead = True
                break          # rows after the first dead one are unspecified
        assert (rc == 4) == dead


def test_block_diffusion_fixture(oracle):
    # tests/unit/models/unit_block_diffusion.c:115-172
    want = ["10000000000000", "11000000000000", "11100000000000", "11110000000000", "11111000000000",
            "11111100000000", "11000011110000", "11000011110000", "11000011110000", "11000011110000",
            "11110000001111", "11110000001111", "11110000001111", "11110000001111"]
    cfg = abi.BltBlockDiffusionConfig()
    starts = abi.size_array([2, 4])
    cfg.mode, cfg.seq_len, cfg.num_clean, cfg.block_size = abi.BLT_BDM_TRAIN, 14, 6, 4
    cfg.block_starts, cfg.num_blocks = starts, 2
    out = np.empty(14 * 14, dtype=np.float32)
    assert oracle.orc_build_block_diffusion_mask(C.byref(cfg), binding.fptr(out)) == 0
    got = ["".join("1" if x == 0 else "0" for x in row) for row in out.reshape(14, 14)]
    assert got == want
    assert np.isneginf(out[out != 0]).all()
    cfg = abi.BltBlockDiffusionConfig()
    cfg.mode, cfg.seq_len, cfg.num_clean = abi.BLT_BDM_INFER, 7, 3
    out = np.empty(49, dtype=np.float32)
    assert oracle.orc_build_block_diffusion_mask(C.byref(cfg), binding.fptr(out)) == 0
    ok = out.reshape(7, 7) == 0
    for i in range(7):
        for j in range(7):
            assert ok[i, j] == ((j <= i) if i < 3 else True)
    # bad configurations are the reference's aborts (mask_builder_cpu.c:103-119)
    cfg.num_clean = 0
    assert oracle.orc_build_block_diffusion_mask(C.byref(cfg), binding.fptr(out)) == 5


def test_block_diffusion_no_leak(oracle):
    # tests/unit/models/unit_block_diffusion.c:186-238
    N, B, starts = 9, 3, [1, 3, 5, 8]
    S = N + B * len(starts)
    cfg = abi.BltBlockDiffusionConfig()
    arr = abi.size_array(starts)
    cfg.mode, cfg.seq_len, cfg.num_clean, cfg.block_size = abi.BLT_BDM_TRAIN, S, N, B
    cfg.block_starts, cfg.num_blocks = arr, len(starts)
    out = np.empty(S * S, dtype=np.float32)
    assert oracle.orc_build_block_diffusion_mask(C.byref(cfg), binding.fptr(out)) == 0
    ok = out.reshape(S, S) == 0
    for i in range(S):
        for j in range(S):
            if i < N:
                assert ok[i, j] == (j < N and j <= i)
            else:
                blk = (i - N) // B
                own = j >= N and (j - N) // B == blk
                assert ok[i, j] == (j < starts[blk] or own)


def test_patch_index_reference_vectors(oracle):
    # tests/unit/models/unit_local_decoder.c:94-113
    p = abi.patch_array([0, 3, 7, 8, 15], [3, 4, 1, 7, 1])
    got = [oracle.orc_patch_decoder_latent_at(p, 5, pos) for pos in range(16)]
    assert got == [0, 0, 0, 0, 0, 0, 1, 2, 2, 2, 2, 2, 2, 2, 3, 3]
    assert oracle.orc_patch_decoder_latent_at(p, 5, 16) == 4 and oracle.orc_patch_decoder_latent_at(p, 5, 100) == 4
    # tests/unit/backend/unit_mask.c:116-127
    src, dst = abi.size_array([0, 1]), abi.size_array([9] * 6)
    oracle.orc_patch_expand_group_ids(src, 2, 3, dst)
    assert list(dst) == [0, 0, 0, 1, 1, 1]
    # group ids: patch p is query group p, its bytes carry p; bad tilings are rejected
    q, kv = abi.size_array([9] * 5), abi.size_array([9] * 16)
    assert oracle.orc_patch_build_group_ids(p, 5, 16, q, kv) == 0
    assert list(q) == [0, 1, 2, 3, 4]
    assert list(kv) == [0] * 3 + [1] * 4 + [2] + [3] * 7 + [4]
    assert oracle.orc_patch_build_group_ids(p, 5, 17, q, kv) == 6
    gap = abi.patch_array([0, 4], [3, 2])
    assert oracle.orc_patch_build_group_ids(gap, 2, 6, q, kv) == 6
    # one-hot cross mask rows (unit_local_decoder.c:34-87)
    rc, ok, _ = mask_of(oracle, seq_len_q=16, seq_len_kv=5, query_group_ids=list(kv), kv_group_ids=list(q),
                        bidirectional_within_group=True)
    assert rc == 0 and (ok.sum(1) == 1).all() and (ok.argmax(1) == np.array(list(kv))).all()


def test_kv_slab_indexing(oracle):
    # [batch*max_seq_len, E] row-major, row == absolute position (kv_cache.c:56-60, kv_cache.h:17-18)
    assert oracle.orc_kv_row(0, 0, 768) == 0 and oracle.orc_kv_row(3, 5, 768) == 3 * 768 + 5
    assert oracle.orc_kv_slot(2, 7, 3, 9, 768, 128, 32) == ((2 * 768 + 7) * 128 + 3 * 32 + 9)
    m = np.empty(3 * 8, dtype=np.float32)
    oracle.orc_kv_self_mask(binding.fptr(m), 3, 5, 0)
    ok = m.reshape(3, 8) == 0
    for r in range(3):
        assert list(ok[r]) == [j <= 5 + r for j in range(8)]
    oracle.orc_kv_self_mask(binding.fptr(m), 3, 5, 4)
    ok = m.reshape(3, 8) == 0
    for r in range(3):
        assert list(ok[r]) == [j <= 5 + r and 5 + r - j < 4 for j in range(8)]


@pytest.mark.parametrize("chunks", [[1] * 12, [5, 1, 1, 5], [12], [3, 4, 5]])
@pytest.mark.parametrize("window", [0, 5])
def test_kv_cached_equals_dense(chunks, window, oracle):
    """The reference's invariant (tests/unit/infer/unit_kv_cache.c:136-151): stepping through the
    cache in any chunking gives bit-identical rows to one dense causal pass."""
    rs = np.random.RandomState(11)
    T, H, hd = sum(chunks), 2, 6
    E = H * hd
    q, k, v = (rs.randn(T, E).astype(np.float32) for _ in range(3))
    # dense: one causal(+window) pass over all T rows
    cfg = abi.BltMaskConfig()
    cfg.seq_len_q = cfg.seq_len_kv = T
    cfg.is_causal, cfg.sliding_window = True, window
    mask = np.empty(T * T, dtype=np.float32)
    assert oracle.orc_build_attention_mask(C.byref(cfg), binding.fptr(mask)) == 0
    dense = np.zeros((T, E), dtype=np.float32)
    scratch = np.empty(T * T, dtype=np.float32)
    for h in range(H):
        a = binding.head_args(q.reshape(-1), k.reshape(-1), v.reshape(-1), dense.reshape(-1), T, T, hd,
                              float(np.float32(1) / np.sqrt(np.float32(hd))), E, E, E, E, h * hd, q_off=h * hd,
                              k_off=h * hd, v_off=h * hd, scratch=scratch, mask=mask)
        assert oracle.orc_attention_head_core(C.byref(a)) == 0
    # cached: sequence 1 of a 2-sequence slab, chunk by chunk
    max_len = T + 3
    ck = np.full((2 * max_len, E), 99.0, dtype=np.float32)
    cv = np.full((2 * max_len, E), 99.0, dtype=np.float32)
    got = np.zeros((T, E), dtype=np.float32)
    base = 0
    for n in chunks:
        rows = slice(base, base + n)
        comb = np.zeros((n, E), dtype=np.float32)
        rc = oracle.orc_kv_attend_step(binding.fptr(ck.reshape(-1)), binding.fptr(cv.reshape(-1)), max_len, E, H, 1,
                                       base, n, window, binding.fptr(np.ascontiguousarray(q[rows])),
                                       binding.fptr(np.ascontiguousarray(k[rows])),
                                       binding.fptr(np.ascontiguousarray(v[rows])), binding.fptr(comb.reshape(-1)))
        assert rc == 0
        got[rows] = comb
        base += n
    assert got.tobytes() == dense.tobytes()
    assert (ck[:max_len] == 99.0).all() and np.array_equal(ck[max_len:max_len + T], k)  # only slab 1 rows touched
    assert oracle.orc_kv_attend_step(binding.fptr(ck.reshape(-1)), binding.fptr(cv.reshape(-1)), max_len, E, H, 1,
                                     T, 4, 0, binding.fptr(q), binding.fptr(k), binding.fptr(v),
                                     binding.fptr(got.reshape(-1))) == 7   # over capacity


# ---------------------------------------------------------------------------
# RoPE (csrc/ops/reductions_cpu.c:179-229, csrc/infer/rope_gather.c)
# ---------------------------------------------------------------------------
def _rope_apply(oracle, x, c, s):
    rows, heads, hd = x.shape
    out = np.empty_like(x)
    oracle.orc_rope_apply(binding.fptr(x.reshape(-1)), rows, heads, hd, binding.fptr(c.reshape(-1)),
                          binding.fptr(s.reshape(-1)), binding.fptr(out.reshape(-1)))
    return out


def test_rope_tables_against_float64(oracle):
    """angle = pos / theta^(2i/hd): position 0 is (1, 0), band 0 turns by one radian per position,
    every entry within float rounding of the float64 value."""
    for hd, theta, n in ((32, 500000.0, 300), (64, 10000.0, 50), (2, 500000.0, 9)):
        half = hd // 2
        c, s = np.empty(n * half, dtype=np.float32), np.empty(n * half, dtype=np.float32)
        assert oracle.orc_rope_precompute(n, theta, hd, binding.fptr(c), binding.fptr(s)) == 0
        c, s = c.reshape(n, half), s.reshape(n, half)
        assert (c[0] == 1.0).all() and (s[0] == 0.0).all()
        assert abs(c[1, 0] - np.cos(1.0)) < 1e-7 and abs(s[1, 0] - np.sin(1.0)) < 1e-7
        i = np.arange(half, dtype=np.float64)
        ang = np.arange(n, dtype=np.float64)[:, None] / np.power(theta, 2.0 * i / hd)[None, :]
        # the float angle carries a relative error of ~2^-23, i.e. up to pos * 2^-23 absolute
        tol = 4e-7 + np.arange(n)[:, None] * 3e-7
        assert (np.abs(c - np.cos(ang)) < tol).all() and (np.abs(s - np.sin(ang)) < tol).all()
    assert oracle.orc_rope_precompute(4, 500000.0, 3, binding.fptr(c.reshape(-1)), binding.fptr(s.reshape(-1))) != 0


def test_rope_apply_closed_forms(oracle):
    rs = np.random.RandomState(3)
    x = rs.randn(5, 3, 8).astype(np.float32)
    one, zero = np.ones((5, 4), dtype=np.float32), np.zeros((5, 4), dtype=np.float32)
    # angle 0: identity, bit for bit
    assert _rope_apply(oracle, x, one, zero).tobytes() == x.tobytes()
    # quarter turn (cos, sin) = (0, 1): (x0, x1) -> (-x1, x0); the forward twin of the reference's
    # backward vector (tests/unit/backend/unit_reductions_cpu.c:133-157: grad (1, 0) -> (0, -1))
    q = _rope_apply(oracle, x, zero, one)
    assert (q[..., 0::2] == -x[..., 1::2]).all() and (q[..., 1::2] == x[..., 0::2]).all()
    back = _rope_apply(oracle, np.array([[[0.0, -1.0]]], dtype=np.float32), zero[:1, :1], one[:1, :1])
    assert back.reshape(-1).tolist() == [1.0, 0.0]
    # general angle against float64, pair norms preserved, rows use their own table row
    ang = rs.rand(5, 4) * 6.0
    c, s = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    y = _rope_apply(oracle, x, c, s).astype(np.float64)
    x64, c64, s64 = x.astype(np.float64), c.astype(np.float64)[:, None, :], s.astype(np.float64)[:, None, :]
    want0 = x64[..., 0::2] * c64 - x64[..., 1::2] * s64
    want1 = x64[..., 1::2] * c64 + x64[..., 0::2] * s64
    assert np.abs(y[..., 0::2] - want0).max() < 1e-6 and np.abs(y[..., 1::2] - want1).max() < 1e-6
    n_in = x64[..., 0::2] ** 2 + x64[..., 1::2] ** 2
    n_out = y[..., 0::2] ** 2 + y[..., 1::2] ** 2
    assert np.abs(n_in - n_out).max() < 1e-5


def test_rope_scores_depend_on_position_difference(oracle):
    """q.k after rotating q at position p+d and k at position p equals the same for (d, 0)."""
    hd, n = 16, 64
    half = hd // 2
    c, s = np.empty(n * half, dtype=np.float32), np.empty(n * half, dtype=np.float32)
    oracle.orc_rope_precompute(n, 100.0, hd, binding.fptr(c), binding.fptr(s))
    c, s = c.reshape(n, half), s.reshape(n, half)
    rs = np.random.RandomState(4)
    q, k = rs.randn(1, 1, hd).astype(np.float32), rs.randn(1, 1, hd).astype(np.float32)
    def score(pq, pk):
        a = _rope_apply(oracle, q, c[pq:pq + 1], s[pq:pq + 1]).astype(np.float64)
        b = _rope_apply(oracle, k, c[pk:pk + 1], s[pk:pk + 1]).astype(np.float64)
        return float((a * b).sum())
    for d in (0, 1, 7):
        base = score(d, 0)
        for p in (3, 20, 50):
            assert abs(score(p + d, p) - base) < 2e-4, (d, p)


def test_rope_gather_and_step_composition(oracle):
    """The gather copies table rows; the rotating step equals rotating by hand and calling the plain step."""
    rs = np.random.RandomState(6)
    H, hd, max_len, batch = 2, 8, 30, 2
    E, half = H * hd, hd // 2
    c, s = np.empty(max_len * half, dtype=np.float32), np.empty(max_len * half, dtype=np.float32)
    oracle.orc_rope_precompute(max_len, 500000.0, hd, binding.fptr(c), binding.fptr(s))
    pos = abi.size_array([7, 0, 29])
    gc, gs = np.empty(3 * half, dtype=np.float32), np.empty(3 * half, dtype=np.float32)
    assert oracle.orc_rope_position_gather(binding.fptr(c), binding.fptr(s), max_len, half, pos, 3, binding.fptr(gc),
                                           binding.fptr(gs)) == 0
    assert (gc.reshape(3, half) == c.reshape(max_len, half)[[7, 0, 29]]).all()
    assert (gs.reshape(3, half) == s.reshape(max_len, half)[[7, 0, 29]]).all()
    assert oracle.orc_rope_position_gather(binding.fptr(c), binding.fptr(s), max_len, half, abi.size_array([30]), 1,
                                           binding.fptr(gc), binding.fptr(gs)) != 0
    ck1 = rs.randn(batch * max_len, E).astype(np.float32)
    cv1 = rs.randn(batch * max_len, E).astype(np.float32)
    ck2, cv2 = ck1.copy(), cv1.copy()
    for b, base, n, window in ((0, 4, 1, 0), (1, 9, 5, 0), (0, 5, 3, 4)):
        qkv = rs.randn(n, 3 * E).astype(np.float32)   # packed rows: strides 3E
        mine = np.zeros((n, E), dtype=np.float32)
        f = qkv.reshape(-1)
        rc = oracle.orc_kv_rope_attend_step(
            binding.fptr(ck1.reshape(-1)), binding.fptr(cv1.reshape(-1)), max_len, E, H, b, base, n, window,
            binding.fptr(f), 3 * E, C.cast(f.ctypes.data + 4 * E, binding._fp), 3 * E,
            C.cast(f.ctypes.data + 8 * E, binding._fp), 3 * E, binding.fptr(c), binding.fptr(s), max_len,
            binding.fptr(mine.reshape(-1)))
        assert rc == 0
        tc, ts = c.reshape(max_len, half)[base:base + n].copy(), s.reshape(max_len, half)[base:base + n].copy()
        q = _rope_apply(oracle, np.ascontiguousarray(qkv[:, :E]).reshape(n, H, hd), tc, ts).reshape(n, E)
        k = _rope_apply(oracle, np.ascontiguousarray(qkv[:, E:2 * E]).reshape(n, H, hd), tc, ts).reshape(n, E)
        v = np.ascontiguousarray(qkv[:, 2 * E:])
        theirs = np.zeros((n, E), dtype=np.float32)
        assert oracle.orc_kv_attend_step(binding.fptr(ck2.reshape(-1)), binding.fptr(cv2.reshape(-1)), max_len, E, H,
                                         b, base, n, window, binding.fptr(q), binding.fptr(k), binding.fptr(v),
                                         binding.fptr(theirs.reshape(-1))) == 0
        assert mine.tobytes() == theirs.tobytes()
        assert ck1.tobytes() == ck2.tobytes() and cv1.tobytes() == cv2.tobytes()


# ---------------------------------------------------------------------------
# projections and the attention block (csrc/ops/linalg_cpu.c:8-18, csrc/models/attention.c:130-207)
# ---------------------------------------------------------------------------
def test_matmul_reference_vector_and_float64(oracle):
    a = np.array([1, 2, 3, 4], dtype=np.float32)
    b = np.array([5, 6, 7, 8], dtype=np.float32)
    out = np.zeros(4, dtype=np.float32)
    oracle.orc_matmul(binding.fptr(a), binding.fptr(b), binding.fptr(out), 2, 2, 2)
    assert out.tolist() == [19.0, 22.0, 43.0, 50.0]   # tests/unit/backend/unit_linalg_cpu.c:10-48
    rs = np.random.RandomState(8)
    for m, k, n in ((1, 7, 5), (9, 33, 17), (40, 128, 24)):
        a, b = rs.randn(m, k).astype(np.float32), rs.randn(k, n).astype(np.float32)
        out = np.zeros((m, n), dtype=np.float32)
        oracle.orc_matmul(binding.fptr(a.reshape(-1)), binding.fptr(b.reshape(-1)), binding.fptr(out.reshape(-1)), m,
                          k, n)
        want = a.astype(np.float64) @ b.astype(np.float64)
        assert np.abs(out - want).max() < 2e-5
        # not a transposed operand: a non-square case fails if either were
        assert np.abs(out - (b.T.astype(np.float64) @ a.T.astype(np.float64)).T).max() < 2e-5
    # the sum runs over k in ascending order with separate rounding: a case where the order shows
    a = np.array([[1e8, 1.0, -1e8]], dtype=np.float32)
    b = np.ones((3, 1), dtype=np.float32)
    out = np.zeros((1, 1), dtype=np.float32)
    oracle.orc_matmul(binding.fptr(a.reshape(-1)), binding.fptr(b.reshape(-1)), binding.fptr(out.reshape(-1)), 1, 3, 1)
    assert out[0, 0] == 0.0   # (1e8 + 1) rounds to 1e8, then - 1e8


def _mha(oracle, x, wqkv, wproj, H, causal=False, rope=False, theta=10000.0, mask_cfg=None, caches=None):
    T, E = x.shape
    out = np.full((T, E), 3.0, dtype=np.float32)
    c = binding.fptr(caches[0].reshape(-1)) if caches else None
    s = binding.fptr(caches[1].reshape(-1)) if caches else None
    rc = oracle.orc_multihead_attention(binding.fptr(x.reshape(-1)), binding.fptr(wqkv.reshape(-1)),
                                        binding.fptr(wproj.reshape(-1)), binding.fptr(out.reshape(-1)), T, E, H,
                                        int(causal), int(rope), theta, c, s,
                                        C.byref(mask_cfg) if mask_cfg is not None else None)
    assert rc == 0, rc
    return out


def _identity_block():
    x = np.array([[1, 0, 1, 0], [0, 1, 0, 1]], dtype=np.float32)
    wqkv = np.zeros((4, 12), dtype=np.float32)
    for i in range(4):
        wqkv[i, i] = wqkv[i, 4 + i] = wqkv[i, 8 + i] = 1.0
    return x, wqkv, np.eye(4, dtype=np.float32)


def test_attention_block_reference_vectors(oracle):
    """tests/unit/models/unit_attention.c:30-88 (identity weights, two tokens, two heads) and
    160-171 (causal: row 0 sees only itself)."""
    x, wqkv, wproj = _identity_block()
    out = _mha(oracle, x, wqkv, wproj, 2)
    want = np.array([[0.6697615, 0.3302385, 0.6697615, 0.3302385], [0.3302385, 0.6697615, 0.3302385, 0.6697615]])
    assert np.abs(out - want).max() < 1e-6
    out_c = _mha(oracle, x, wqkv, wproj, 2, causal=True)
    assert np.abs(out_c[0] - np.array([1, 0, 1, 0])).max() < 1e-6
    assert np.abs(out_c[1] - want[1]).max() < 1e-6
    # mask_config causal == is_causal (unit_attention.c:184)
    cfg = abi.BltMaskConfig()
    cfg.seq_len_q = cfg.seq_len_kv = 2
    cfg.is_causal = True
    assert _mha(oracle, x, wqkv, wproj, 2, mask_cfg=cfg).tobytes() == out_c.tobytes()
    # with rotation: position 0 is not rotated, and running it twice gives the same bits (unit_attention.c:66-79)
    r1 = _mha(oracle, x, wqkv, wproj, 2, rope=True)
    r2 = _mha(oracle, x, wqkv, wproj, 2, rope=True)
    assert r1.tobytes() == r2.tobytes() and np.isfinite(r1).all()


def test_attention_block_equals_its_parts(oracle):
    rs = np.random.RandomState(21)
    T, E, H = 19, 24, 3
    hd, half = E // H, E // H // 2
    x = rs.randn(T, E).astype(np.float32)
    wqkv = (rs.randn(E, 3 * E) / np.sqrt(E)).astype(np.float32)
    wproj = (rs.randn(E, E) / np.sqrt(E)).astype(np.float32)
    cos, sin = np.empty(T * half, dtype=np.float32), np.empty(T * half, dtype=np.float32)
    assert oracle.orc_rope_precompute(T, 500000.0, hd, binding.fptr(cos), binding.fptr(sin)) == 0
    got = _mha(oracle, x, wqkv, wproj, H, causal=True, rope=True, theta=500000.0)
    got_cached = _mha(oracle, x, wqkv, wproj, H, causal=True, rope=True, theta=1.0, caches=(cos, sin))
    assert got.tobytes() == got_cached.tobytes()   # caches win over theta
    qkv = np.zeros((T, 3 * E), dtype=np.float32)
    oracle.orc_matmul(binding.fptr(x.reshape(-1)), binding.fptr(wqkv.reshape(-1)), binding.fptr(qkv.reshape(-1)), T, E,
                      3 * E)
    # packed rotation == copy out, orc_rope_apply, copy back
    q_heads = np.ascontiguousarray(qkv[:, :E]).reshape(T, H, hd)
    rot = np.empty_like(q_heads)
    oracle.orc_rope_apply(binding.fptr(q_heads.reshape(-1)), T, H, hd, binding.fptr(cos), binding.fptr(sin),
                          binding.fptr(rot.reshape(-1)))
    for h in range(H):
        oracle.orc_rope_apply_packed(binding.fptr(qkv.reshape(-1)), 3 * E, h * hd, T, hd, binding.fptr(cos),
                                     binding.fptr(sin))
        oracle.orc_rope_apply_packed(binding.fptr(qkv.reshape(-1)), 3 * E, E + h * hd, T, hd, binding.fptr(cos),
                                     binding.fptr(sin))
    assert qkv[:, :E].reshape(T, H, hd).tobytes() == rot.tobytes()
    comb = np.zeros((T, E), dtype=np.float32)
    w = np.zeros(T * T, dtype=np.float32)
    flat = qkv.reshape(-1)
    for h in range(H):
        a = binding.head_args(flat, flat, flat, comb.reshape(-1), T, T, hd, float(np.float32(1) / np.sqrt(np.float32(hd))),
                              3 * E, 3 * E, 3 * E, E, h * hd, q_off=h * hd, k_off=E + h * hd, v_off=2 * E + h * hd,
                              weights=w, causal=True)
        assert oracle.orc_attention_head_core(C.byref(a)) == 0
    want = np.zeros((T, E), dtype=np.float32)
    oracle.orc_matmul(binding.fptr(comb.reshape(-1)), binding.fptr(wproj.reshape(-1)), binding.fptr(want.reshape(-1)), T,
                      E, E)
    assert got.tobytes() == want.tobytes()


def _group_cfg(P, T, q_groups, kv_groups):
    cfg = abi.BltMaskConfig()
    cfg.seq_len_q, cfg.seq_len_kv = P, T
    keep = (abi.size_array(q_groups), abi.size_array(kv_groups))
    cfg.query_group_ids, cfg.kv_group_ids = keep
    cfg.bidirectional_within_group = True
    return cfg, keep


def _xattn(oracle, xq, xkv, wq, wk, wv, wp, H, cfg):
    P, E = xq.shape
    out = np.full((P, E), 3.0, dtype=np.float32)
    rc = oracle.orc_cross_attention_forward(*(binding.fptr(a.reshape(-1)) for a in (xq, xkv, wq, wk, wv, wp, out)), P,
                                            xkv.shape[0], E, H, C.byref(cfg) if cfg is not None else None)
    return rc, out


def test_cross_attention_reference_vectors(oracle):
    """tests/unit/models/unit_cross_attention.c:24-117 (identity weights, two patches over two bytes
    each) and 124-246 (bytes of patch 1 never reach patch 0)."""
    xq = np.array([[1, 0, 1, 0], [0, 1, 0, 1]], dtype=np.float32)
    xkv = np.array([[1, 0, 1, 0], [0, 1, 0, 1], [1, 0, 1, 0], [0, 1, 0, 1]], dtype=np.float32)
    eye = np.eye(4, dtype=np.float32)
    cfg, _keep = _group_cfg(2, 4, [0, 1], [0, 0, 1, 1])
    rc, out = _xattn(oracle, xq, xkv, eye, eye, eye, eye, 2, cfg)
    want = np.array([[0.6697615, 0.3302385, 0.6697615, 0.3302385], [0.3302385, 0.6697615, 0.3302385, 0.6697615]])
    assert rc == 0 and np.abs(out - want).max() < 1e-6
    xkv_b = xkv.copy()
    xkv_b[2] = [500, -500, 250, -250]
    xkv_b[3] = [-500, 500, -250, 250]
    rc, out_b = _xattn(oracle, xq, xkv_b, eye, eye, eye, eye, 2, cfg)
    assert rc == 0 and out_b[0].tobytes() == out[0].tobytes() and np.abs(out_b[1] - out[1]).max() > 1e-3
    # the mask is required, and its lengths must be the call's (cross_attention.c:23-24, 58-60)
    assert _xattn(oracle, xq, xkv, eye, eye, eye, eye, 2, None)[0] == 8
    bad, _k2 = _group_cfg(2, 3, [0, 1], [0, 0, 1])
    assert _xattn(oracle, xq, xkv, eye, eye, eye, eye, 2, bad)[0] == 8


def test_cross_attention_equals_its_parts_and_float64(oracle):
    rs = np.random.RandomState(77)
    P, T, E, H = 5, 23, 24, 3
    hd = E // H
    xq, xkv = rs.randn(P, E).astype(np.float32), rs.randn(T, E).astype(np.float32)
    wq, wk, wv, wp = ((rs.randn(E, E) / np.sqrt(E)).astype(np.float32) for _ in range(4))
    kv_groups = np.sort(np.concatenate([np.arange(P), rs.randint(0, P, size=T - P)]))
    cfg, _keep = _group_cfg(P, T, list(range(P)), kv_groups.tolist())
    rc, got = _xattn(oracle, xq, xkv, wq, wk, wv, wp, H, cfg)
    assert rc == 0
    # a patch that owns no byte is refused by the mask builder (mask_builder_cpu.c:93)
    holed = kv_groups.copy()
    holed[holed == 2] = 3
    cfg_h, _keep_h = _group_cfg(P, T, list(range(P)), holed.tolist())
    assert _xattn(oracle, xq, xkv, wq, wk, wv, wp, H, cfg_h)[0] == 4
    # composition of the pinned parts, bit for bit
    def mm(a, b):
        o = np.zeros((a.shape[0], b.shape[1]), dtype=np.float32)
        oracle.orc_matmul(binding.fptr(a.reshape(-1)), binding.fptr(b.reshape(-1)), binding.fptr(o.reshape(-1)),
                          a.shape[0], a.shape[1], b.shape[1])
        return o
    q, k, v = mm(xq, wq), mm(xkv, wk), mm(xkv, wv)
    mask = np.empty(P * T, dtype=np.float32)
    assert oracle.orc_build_attention_mask(C.byref(cfg), binding.fptr(mask)) == 0
    comb = np.zeros((P, E), dtype=np.float32)
    w = np.zeros(P * T, dtype=np.float32)
    for h in range(H):
        a = binding.head_args(q.reshape(-1), k.reshape(-1), v.reshape(-1), comb.reshape(-1), P, T, hd,
                              float(np.float32(1) / np.sqrt(np.float32(hd))), E, E, E, E, h * hd, q_off=h * hd,
                              k_off=h * hd, v_off=h * hd, weights=w, mask=mask)
        assert oracle.orc_attention_head_core(C.byref(a)) == 0
    assert got.tobytes() == mm(comb, wp).tobytes()
    # float64 restatement from the definition (different operand for K/V than for Q shows a swapped input)
    q64, k64, v64 = xq.astype(np.float64) @ wq, xkv.astype(np.float64) @ wk, xkv.astype(np.float64) @ wv
    comb64 = np.zeros((P, E))
    for h in range(H):
        sl = slice(h * hd, (h + 1) * hd)
        sc = q64[:, sl] @ k64[:, sl].T / np.sqrt(hd)
        for i in range(P):
            keys = np.nonzero(kv_groups == i)[0]
            e = np.exp(sc[i, keys] - sc[i, keys].max())
            comb64[i, sl] = (e / e.sum()) @ v64[keys, sl]
    want = comb64 @ wp.astype(np.float64)
    assert np.abs(got - want).max() < 2e-5


# ---------------------------------------------------------------------------
# row ops of the decoder layer (reductions_cpu.c:325-352, elementwise_cpu.c:9-18, 86-99)
# ---------------------------------------------------------------------------
def test_rmsnorm_add_swiglu_closed_forms(oracle):
    rs = np.random.RandomState(41)
    # a constant row c normalises to sign(c) * weight (up to the eps in the root)
    x = np.full((2, 16), 3.0, dtype=np.float32)
    x[1] = -0.5
    w = rs.randn(16).astype(np.float32)
    out = np.zeros_like(x)
    oracle.orc_rmsnorm_forward(binding.fptr(x.reshape(-1)), binding.fptr(w), binding.fptr(out.reshape(-1)), 2, 16)
    assert np.abs(out[0] - w).max() < 1e-6 and np.abs(out[1] + w).max() < 1e-5
    # unit weight: the output's mean square is 1; each row uses its own statistics
    x = (rs.randn(7, 33) * np.arange(1, 8)[:, None]).astype(np.float32)
    out = np.zeros_like(x)
    oracle.orc_rmsnorm_forward(binding.fptr(x.reshape(-1)), binding.fptr(np.ones(33, dtype=np.float32)),
                               binding.fptr(out.reshape(-1)), 7, 33)
    assert np.abs((out.astype(np.float64) ** 2).mean(axis=1) - 1.0).max() < 1e-5
    want = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + 1e-6)
    assert np.abs(out - want).max() < 1e-5
    # add
    a, b = rs.randn(50).astype(np.float32), rs.randn(50).astype(np.float32)
    out = np.zeros(50, dtype=np.float32)
    oracle.orc_add(binding.fptr(a), binding.fptr(b), binding.fptr(out), 50)
    assert (out == a + b).all()
    oracle.orc_add(binding.fptr(a), binding.fptr(np.zeros(50, dtype=np.float32)), binding.fptr(out), 50)
    assert out.tobytes() == a.tobytes()
    # swiglu: silu(g) * u, silu(0) = 0, large negative gate -> 0, large positive gate -> g * u
    g = np.array([0.0, 1.0, -1.0, 30.0, -30.0, 2.5], dtype=np.float32)
    u = np.array([5.0, 2.0, 2.0, 0.5, 3.0, -1.5], dtype=np.float32)
    out = np.zeros(6, dtype=np.float32)
    oracle.orc_swiglu_forward(binding.fptr(g), binding.fptr(u), binding.fptr(out), 6)
    want = g.astype(np.float64) / (1.0 + np.exp(-g.astype(np.float64))) * u
    assert out[0] == 0.0 and abs(out[3] - 15.0) < 1e-5 and abs(out[4]) < 1e-10
    assert np.abs(out - want).max() < 1e-6


def test_decode_layer_equals_its_parts(oracle):
    rs = np.random.RandomState(43)
    H, hd, max_len, batch, hidden = 2, 8, 24, 2, 40
    E, half = H * hd, hd // 2
    cos, sin = np.empty(max_len * half, dtype=np.float32), np.empty(max_len * half, dtype=np.float32)
    oracle.orc_rope_precompute(max_len, 500000.0, hd, binding.fptr(cos), binding.fptr(sin))
    ck1, cv1 = rs.randn(batch * max_len, E).astype(np.float32), rs.randn(batch * max_len, E).astype(np.float32)
    ck2, cv2 = ck1.copy(), cv1.copy()
    W = {k: (rs.randn(*shape) / np.sqrt(shape[0])).astype(np.float32)
         for k, shape in dict(qkv=(E, 3 * E), proj=(E, E), up=(E, hidden), gate=(E, hidden), down=(hidden, E)).items()}
    n1, n2 = (1.0 + 0.1 * rs.randn(E)).astype(np.float32), (1.0 + 0.1 * rs.randn(E)).astype(np.float32)
    fp = lambda a: binding.fptr(a.reshape(-1))
    for b, base, n in ((0, 3, 1), (1, 7, 4)):
        x = rs.randn(n, E).astype(np.float32)
        mine = np.zeros((n, E), dtype=np.float32)
        assert oracle.orc_kv_decode_layer(fp(ck1), fp(cv1), max_len, E, H, b, base, n, 0, fp(n1), fp(W["qkv"]),
                                          fp(W["proj"]), fp(n2), fp(W["up"]), fp(W["gate"]), fp(W["down"]), hidden,
                                          fp(cos), fp(sin), max_len, fp(x), fp(mine)) == 0
        normed, qkv, comb = np.zeros((n, E), np.float32), np.zeros((n, 3 * E), np.float32), np.zeros((n, E), np.float32)
        oracle.orc_rmsnorm_forward(fp(x), fp(n1), fp(normed), n, E)
        oracle.orc_matmul(fp(normed), fp(W["qkv"]), fp(qkv), n, E, 3 * E)
        f = qkv.reshape(-1)
        fpo = lambda off: C.cast(f.ctypes.data + 4 * off, binding._fp)
        assert oracle.orc_kv_rope_attend_step(fp(ck2), fp(cv2), max_len, E, H, b, base, n, 0, fpo(0), 3 * E, fpo(E),
                                              3 * E, fpo(2 * E), 3 * E, fp(cos), fp(sin), max_len, fp(comb)) == 0
        attn, resid = np.zeros((n, E), np.float32), np.zeros((n, E), np.float32)
        oracle.orc_matmul(fp(comb), fp(W["proj"]), fp(attn), n, E, E)
        oracle.orc_add(fp(x), fp(attn), fp(resid), n * E)
        oracle.orc_rmsnorm_forward(fp(resid), fp(n2), fp(normed), n, E)
        up, gate, act = (np.zeros((n, hidden), np.float32) for _ in range(3))
        oracle.orc_matmul(fp(normed), fp(W["up"]), fp(up), n, E, hidden)
        oracle.orc_matmul(fp(normed), fp(W["gate"]), fp(gate), n, E, hidden)
        oracle.orc_swiglu_forward(fp(gate), fp(up), fp(act), n * hidden)
        oracle.orc_matmul(fp(act), fp(W["down"]), fp(attn), n, hidden, E)
        want = np.zeros((n, E), np.float32)
        oracle.orc_add(fp(resid), fp(attn), fp(want), n * E)
        assert mine.tobytes() == want.tobytes()
        assert ck1.tobytes() == ck2.tobytes() and cv1.tobytes() == cv2.tobytes()
