"""Bit-for-bit comparison of the CPU checker with the reference's own CPU ops
(oracle/_ref/libblt_ref.so, compiled from the reference's sources by
`make -C oracle ref`).  Skipped on machines without that build; the committed
fixtures under tests/golden/ carry the same evidence there."""
import ctypes as C

import numpy as np
import pytest

from fblt_amd import abi, decoder
from oracle import binding

CPU = abi.BLT_BACKEND_CPU


def _both_core(orc, ref, q, k, v, nq, nk, hd, scale, qs, ks, vs, mask, causal, use_weights):
    res = []
    for lib in (orc, ref):
        out = np.full((nq, hd + 2), 4.0, dtype=np.float32)
        w = np.full(nq * nk, 4.0, dtype=np.float32)
        a = binding.head_args(q, k, v, out.reshape(-1), nq, nk, hd, scale, qs, ks, vs, hd + 2, 1,
                              weights=w if use_weights else None, scratch=None if use_weights else w, mask=mask,
                              causal=causal)
        if lib is orc:
            assert lib.orc_attention_head_core(C.byref(a)) == 0
        else:
            lib.blt_attention_head_core(CPU, C.byref(a))
        res.append((out, w))
    return res


def test_attention_core_bit_exact(oracle, ref):
    rs = np.random.RandomState(5)
    for trial in range(120):
        nq, nk, hd = rs.randint(1, 40), rs.randint(1, 60), int(rs.choice([1, 2, 7, 16, 32, 64]))
        qs, ks, vs = hd + rs.randint(0, 5), hd + rs.randint(0, 5), hd + rs.randint(0, 5)
        q = (rs.randn(nq * qs) * rs.choice([0.1, 1, 5])).astype(np.float32)
        k = rs.randn(nk * ks).astype(np.float32)
        v = rs.randn(nk * vs).astype(np.float32)
        kind = trial % 4
        mask, causal = None, False
        if kind == 1:
            causal = True
        elif kind == 2:
            mask = np.where(rs.rand(nq * nk) < 0.5, -np.inf, 0.0).astype(np.float32)
        elif kind == 3:
            mask = (rs.randn(nq * nk) * 3).astype(np.float32)
            mask[rs.rand(nq * nk) < 0.1] = np.inf
        scale = float(np.float32(1) / np.sqrt(np.float32(hd)))
        (o1, w1), (o2, w2) = _both_core(oracle, ref, q, k, v, nq, nk, hd, scale, qs, ks, vs, mask, causal,
                                        trial % 2 == 0)
        assert o1.tobytes() == o2.tobytes(), trial
        assert w1.tobytes() == w2.tobytes(), trial


def test_softmax_dot_copy_bit_exact(oracle, ref):
    rs = np.random.RandomState(6)
    for trial in range(60):
        n = rs.randint(1, 200)
        row = (rs.randn(n) * 4).astype(np.float32)
        if trial % 5 == 0:
            row[rs.randint(n)] = np.inf
        mask = np.where(rs.rand(n) < 0.4, -np.inf, 0).astype(np.float32) if trial % 3 == 0 else None
        a, b = row.copy(), row.copy()
        idx, causal, scale = rs.randint(n), trial % 2 == 1, float(rs.rand() + 0.05)
        oracle.orc_softmax_masked_row_inplace(binding.fptr(a), n, idx, causal, binding.fptr(mask), scale)
        ref.blt_softmax_masked_row_inplace(CPU, binding.fptr(b), n, idx, causal, binding.fptr(mask), scale)
        assert a.tobytes() == b.tobytes()
        x, y = rs.randn(n).astype(np.float32), rs.randn(n).astype(np.float32)
        d1 = oracle.orc_vec_dot(binding.fptr(x), binding.fptr(y), n)
        d2 = ref.blt_vec_dot(CPU, binding.fptr(x), binding.fptr(y), n)
        assert np.float32(d1).tobytes() == np.float32(d2).tobytes()
    src = rs.randn(7, 20).astype(np.float32)
    d1, d2 = np.zeros((7, 11), np.float32), np.zeros((7, 11), np.float32)
    oracle.orc_strided_copy(binding.fptr(d1.reshape(-1)), 11, binding.fptr(src.reshape(-1)), 20, 7, 9)
    ref.blt_strided_copy(CPU, binding.fptr(d2.reshape(-1)), 11, binding.fptr(src.reshape(-1)), 20, 7, 9)
    assert d1.tobytes() == d2.tobytes()


def _ref_mask(ref, cfg, builder):
    arena = ref.blt_arena_create(16 << 20, CPU)
    t = abi.BltTensor()
    getattr(ref, builder)(C.byref(cfg), C.byref(t), arena)
    n = t.numel
    out = np.ctypeslib.as_array(C.cast(t.data, C.POINTER(C.c_float)), shape=(n,)).copy()
    ref.blt_arena_destroy(arena)
    return out, tuple(t.shape[:2])


def test_mask_builders_bit_exact(oracle, ref):
    rs = np.random.RandomState(8)
    done = 0
    for trial in range(400):
        nq, nk = rs.randint(1, 40), rs.randint(1, 40)
        cfg = abi.BltMaskConfig()
        cfg.seq_len_q, cfg.seq_len_kv = nq, nk
        cfg.is_causal = bool(rs.randint(2))
        cfg.sliding_window = int(rs.choice([0, 0, 2, 9]))
        cfg.causal_offset = int(rs.choice([0, 0, 3, 17]))
        keep = []
        if rs.randint(2):
            b = sorted(rs.randint(0, 45, size=rs.randint(1, 4)).tolist())
            arr = abi.size_array(b)
            keep.append(arr)
            cfg.doc_boundaries, cfg.num_docs = arr, len(b) + 1
        if rs.randint(2):
            qa = abi.size_array(np.sort(rs.randint(0, 4, nq)) if rs.randint(2) else rs.randint(0, 3, nq))
            ka = abi.size_array(np.sort(rs.randint(0, 4, nk)) if rs.randint(2) else rs.randint(0, 3, nk))
            keep += [qa, ka]
            cfg.query_group_ids, cfg.kv_group_ids = qa, ka
            cfg.bidirectional_within_group = bool(rs.randint(2))
        mine = np.empty(nq * nk, dtype=np.float32)
        rc = oracle.orc_build_attention_mask(C.byref(cfg), binding.fptr(mine))
        if rc != 0:
            continue  # the reference would exit the process on this recipe
        theirs, shape = _ref_mask(ref, cfg, "blt_build_attention_mask")
        assert shape == (nq, nk) and mine.tobytes() == theirs.tobytes(), trial
        done += 1
    assert done > 100
    for trial in range(40):
        N, B, NB = rs.randint(1, 20), rs.randint(1, 5), rs.randint(0, 5)
        cfg = abi.BltBlockDiffusionConfig()
        train = trial % 2 == 0
        starts = abi.size_array(rs.randint(0, N, size=max(NB, 1)))
        cfg.mode = abi.BLT_BDM_TRAIN if train else abi.BLT_BDM_INFER
        cfg.seq_len, cfg.num_clean, cfg.block_size = N + B * NB, N, B
        cfg.block_starts, cfg.num_blocks = starts, NB
        S = N + B * NB
        mine = np.empty(S * S, dtype=np.float32)
        assert oracle.orc_build_block_diffusion_mask(C.byref(cfg), binding.fptr(mine)) == 0
        theirs, _ = _ref_mask(ref, cfg, "blt_build_block_diffusion_mask")
        assert mine.tobytes() == theirs.tobytes()


def test_patch_helpers_equal(oracle, ref):
    rs = np.random.RandomState(9)
    for _ in range(50):
        P = rs.randint(1, 12)
        lens = rs.randint(1, 9, size=P)
        starts = np.concatenate(([0], np.cumsum(lens)[:-1]))
        if rs.randint(3) == 0:
            starts = starts + rs.randint(1, 4)  # uncovered head: latent rule still defined
        p = abi.patch_array(starts, lens)
        T = int(starts[-1] + lens[-1])
        for pos in range(T + 3):
            assert oracle.orc_patch_decoder_latent_at(p, P, pos) == ref.blt_patch_decoder_latent_at(p, P, pos)
        if starts[0] == 0:
            q1, k1, q2, k2 = (abi.size_array([0] * max(P, T)) for _ in range(4))
            assert oracle.orc_patch_build_group_ids(p, P, T, q1, k1) == 0
            ref.blt_patch_build_group_ids(p, P, T, q2, k2)
            assert list(q1)[:P] == list(q2)[:P] and list(k1)[:T] == list(k2)[:T]


def test_kv_step_against_reference_op_sequence(oracle, ref):
    """orc_kv_attend_step against the reference's ops issued in the order of
    csrc/infer/kv_cache.c:363-390 (strided copies into the slab, then one core
    call per head with the dense step mask and a scratch score buffer)."""
    rs = np.random.RandomState(10)
    H, hd, max_len, batch = 4, 8, 40, 3
    E = H * hd
    ck1 = rs.randn(batch * max_len, E).astype(np.float32)
    cv1 = rs.randn(batch * max_len, E).astype(np.float32)
    ck2, cv2 = ck1.copy(), cv1.copy()
    for b, base, n, window in [(0, 0, 1, 0), (1, 5, 1, 0), (2, 7, 6, 0), (1, 6, 3, 4), (0, 1, 30, 9)]:
        q, k, v = (rs.randn(n, E).astype(np.float32) for _ in range(3))
        mine = np.zeros((n, E), dtype=np.float32)
        assert oracle.orc_kv_attend_step(binding.fptr(ck1.reshape(-1)), binding.fptr(cv1.reshape(-1)), max_len, E, H,
                                         b, base, n, window, binding.fptr(q), binding.fptr(k), binding.fptr(v),
                                         binding.fptr(mine.reshape(-1))) == 0
        total = base + n
        kd, vd = ck2.reshape(-1), cv2.reshape(-1)
        slab = b * max_len * E
        for h in range(H):
            for dst, src in ((kd, k), (vd, v)):
                ref.blt_strided_copy(CPU, C.cast(dst.ctypes.data + 4 * (slab + base * E + h * hd), C.POINTER(C.c_float)),
                                     E, C.cast(src.ctypes.data + 4 * h * hd, C.POINTER(C.c_float)), E, n, hd)
        mask = np.empty(n * total, dtype=np.float32)   # kv_cache.c:229-236, restated in numpy
        for r in range(n):
            p = base + r
            for j in range(total):
                ok = j <= p and not (window > 0 and p - j >= window)
                mask[r * total + j] = 0.0 if ok else -np.inf
        theirs = np.zeros((n, E), dtype=np.float32)
        scratch = np.empty(n * total, dtype=np.float32)
        for h in range(H):
            a = binding.head_args(q.reshape(-1), kd, vd, theirs.reshape(-1), n, total, hd,
                                  float(np.float32(1) / np.sqrt(np.float32(hd))), E, E, E, E, h * hd, q_off=h * hd,
                                  k_off=slab + h * hd, v_off=slab + h * hd, scratch=scratch, mask=mask)
            ref.blt_attention_head_core(CPU, C.byref(a))
        assert mine.tobytes() == theirs.tobytes()
        assert ck1.tobytes() == ck2.tobytes() and cv1.tobytes() == cv2.tobytes()


def test_rope_bit_exact(oracle, ref):
    """orc_rope_precompute / orc_rope_apply against blt_rope_precompute / blt_rope_apply of the
    reference (csrc/ops/reductions_cpu.c:179-229)."""
    for hd, theta, n in ((32, 500000.0, 700), (64, 500000.0, 300), (8, 10000.0, 40)):
        half = hd // 2
        c1, s1 = np.empty(n * half, dtype=np.float32), np.empty(n * half, dtype=np.float32)
        assert oracle.orc_rope_precompute(n, theta, hd, binding.fptr(c1), binding.fptr(s1)) == 0
        c2, s2 = np.empty(n * half, dtype=np.float32), np.empty(n * half, dtype=np.float32)
        tc, ts = abi.BltTensor(), abi.BltTensor()
        ref.blt_tensor_view_2d(C.byref(tc), c2.ctypes.data, n, half, CPU)
        ref.blt_tensor_view_2d(C.byref(ts), s2.ctypes.data, n, half, CPU)
        cfg = binding.BltRopeConfig(theta, hd)
        ref.blt_rope_precompute(n, C.byref(cfg), C.byref(tc), C.byref(ts))
        assert c1.tobytes() == c2.tobytes() and s1.tobytes() == s2.tobytes()
        rs = np.random.RandomState(hd)
        x = rs.randn(n, 3, hd).astype(np.float32)
        mine = np.empty_like(x)
        oracle.orc_rope_apply(binding.fptr(x.reshape(-1)), n, 3, hd, binding.fptr(c1), binding.fptr(s1),
                              binding.fptr(mine.reshape(-1)))
        theirs = binding.ref_rope_apply(ref, x, c2.reshape(n, half), s2.reshape(n, half))
        assert mine.tobytes() == theirs.tobytes()


def test_kv_rope_step_against_reference_op_sequence(oracle, ref):
    """orc_kv_rope_attend_step against the reference's ops in the order of kv_cache.c:343-366:
    per head copy Q and K out of the packed rows, blt_rope_apply both at positions base..base+n-1,
    copy rotated Q into q_full and rotated K / plain V into the slab; then the (separately pinned)
    attention of the plain step."""
    rs = np.random.RandomState(12)
    H, hd, max_len, batch = 4, 8, 40, 2
    E, half = H * hd, hd // 2
    cos, sin = np.empty(max_len * half, dtype=np.float32), np.empty(max_len * half, dtype=np.float32)
    oracle.orc_rope_precompute(max_len, 500000.0, hd, binding.fptr(cos), binding.fptr(sin))
    ck1 = rs.randn(batch * max_len, E).astype(np.float32)
    cv1 = rs.randn(batch * max_len, E).astype(np.float32)
    ck2, cv2 = ck1.copy(), cv1.copy()
    fp = C.POINTER(C.c_float)
    for b, base, n, window in [(0, 0, 1, 0), (1, 5, 1, 0), (0, 7, 6, 0), (1, 6, 3, 4)]:
        qkv = rs.randn(n, 3 * E).astype(np.float32)
        f = qkv.reshape(-1)
        mine = np.zeros((n, E), dtype=np.float32)
        assert oracle.orc_kv_rope_attend_step(
            binding.fptr(ck1.reshape(-1)), binding.fptr(cv1.reshape(-1)), max_len, E, H, b, base, n, window,
            binding.fptr(f), 3 * E, C.cast(f.ctypes.data + 4 * E, fp), 3 * E, C.cast(f.ctypes.data + 8 * E, fp), 3 * E,
            binding.fptr(cos), binding.fptr(sin), max_len, binding.fptr(mine.reshape(-1))) == 0
        rc = cos.reshape(max_len, half)[base:base + n].copy()
        rsn = sin.reshape(max_len, half)[base:base + n].copy()
        q_full = np.zeros((n, E), dtype=np.float32)
        kd, vd = ck2.reshape(-1), cv2.reshape(-1)
        slab = b * max_len * E
        for h in range(H):
            q_head, k_head = np.empty((n, hd), dtype=np.float32), np.empty((n, hd), dtype=np.float32)
            ref.blt_strided_copy(CPU, binding.fptr(q_head.reshape(-1)), hd, C.cast(f.ctypes.data + 4 * h * hd, fp),
                                 3 * E, n, hd)
            ref.blt_strided_copy(CPU, binding.fptr(k_head.reshape(-1)), hd,
                                 C.cast(f.ctypes.data + 4 * (E + h * hd), fp), 3 * E, n, hd)
            q_rot = binding.ref_rope_apply(ref, q_head.reshape(n, 1, hd), rc, rsn).reshape(n, hd)
            k_rot = binding.ref_rope_apply(ref, k_head.reshape(n, 1, hd), rc, rsn).reshape(n, hd)
            ref.blt_strided_copy(CPU, C.cast(q_full.ctypes.data + 4 * h * hd, fp), E, binding.fptr(q_rot.reshape(-1)),
                                 hd, n, hd)
            ref.blt_strided_copy(CPU, C.cast(kd.ctypes.data + 4 * (slab + base * E + h * hd), fp), E,
                                 binding.fptr(k_rot.reshape(-1)), hd, n, hd)
            ref.blt_strided_copy(CPU, C.cast(vd.ctypes.data + 4 * (slab + base * E + h * hd), fp), E,
                                 C.cast(f.ctypes.data + 4 * (2 * E + h * hd), fp), 3 * E, n, hd)
        assert ck1.tobytes() == ck2.tobytes() and cv1.tobytes() == cv2.tobytes()
        # attention over the slab with the rotated Q: rows already in place, so re-writing them is a no-op
        k_rows = np.ascontiguousarray(ck2.reshape(batch, max_len, E)[b, base:base + n])
        v_rows = np.ascontiguousarray(cv2.reshape(batch, max_len, E)[b, base:base + n])
        theirs = np.zeros((n, E), dtype=np.float32)
        assert oracle.orc_kv_attend_step(binding.fptr(ck2.reshape(-1)), binding.fptr(cv2.reshape(-1)), max_len, E, H,
                                         b, base, n, window, binding.fptr(q_full.reshape(-1)),
                                         binding.fptr(k_rows.reshape(-1)), binding.fptr(v_rows.reshape(-1)),
                                         binding.fptr(theirs.reshape(-1))) == 0
        assert mine.tobytes() == theirs.tobytes()


def test_matmul_and_attention_block_bit_exact(oracle, ref):
    """orc_matmul and orc_multihead_attention against blt_matmul / blt_multihead_attention compiled
    from the reference (csrc/ops/linalg_cpu.c, csrc/models/attention.c:130-207)."""
    rs = np.random.RandomState(31)
    for m, k, n in ((1, 16, 48), (7, 33, 5), (64, 128, 96)):
        a, b = rs.randn(m, k).astype(np.float32), rs.randn(k, n).astype(np.float32)
        mine, theirs = np.zeros((m, n), dtype=np.float32), np.zeros((m, n), dtype=np.float32)
        oracle.orc_matmul(binding.fptr(a.reshape(-1)), binding.fptr(b.reshape(-1)), binding.fptr(mine.reshape(-1)), m,
                          k, n)
        ta, tb, to = (abi.tensor_view(x.ctypes.data, x.shape, CPU) for x in (a, b, theirs))
        ref.blt_matmul(C.byref(ta), C.byref(tb), C.byref(to))
        assert mine.tobytes() == theirs.tobytes()
    arena = ref.blt_arena_create(32 << 20, CPU)
    try:
        for T, E, H, causal, rope, mask in ((2, 4, 2, False, False, None), (37, 32, 4, True, True, None),
                                            (50, 64, 2, False, True, "window"), (33, 24, 3, False, False, "docs"),
                                            (40, 32, 2, True, True, "causal_cfg")):
            x = rs.randn(T, E).astype(np.float32)
            wqkv = (rs.randn(E, 3 * E) / np.sqrt(E)).astype(np.float32)
            wproj = (rs.randn(E, E) / np.sqrt(E)).astype(np.float32)
            cfg, keep = None, None
            if mask is not None:
                cfg = abi.BltMaskConfig()
                cfg.seq_len_q = cfg.seq_len_kv = T
                if mask == "window":
                    cfg.is_causal, cfg.sliding_window = True, 9
                elif mask == "docs":
                    keep = abi.size_array([11, 20])
                    cfg.doc_boundaries, cfg.num_docs = keep, 3
                else:
                    cfg.is_causal = True
            mine = np.zeros((T, E), dtype=np.float32)
            assert oracle.orc_multihead_attention(
                binding.fptr(x.reshape(-1)), binding.fptr(wqkv.reshape(-1)), binding.fptr(wproj.reshape(-1)),
                binding.fptr(mine.reshape(-1)), T, E, H, int(causal), int(rope), 500000.0, None, None,
                C.byref(cfg) if cfg is not None else None) == 0
            theirs = np.zeros((T, E), dtype=np.float32)
            ac = abi.BltAttentionConfig()
            ac.embed_dim, ac.num_heads, ac.head_dim = E, H, E // H
            ac.is_causal, ac.use_rope, ac.rope_theta = causal, rope, 500000.0
            if cfg is not None:
                ac.mask_config = C.pointer(cfg)
            tx, tq, tp, to = (abi.tensor_view(v.ctypes.data, v.shape, CPU) for v in (x, wqkv, wproj, theirs))
            arena.contents.offset = 0
            ref.blt_multihead_attention(C.byref(tx), C.byref(tq), C.byref(tp), C.byref(to), C.byref(ac), arena)
            assert mine.tobytes() == theirs.tobytes(), (T, E, H, causal, rope, mask)
    finally:
        ref.blt_arena_destroy(arena)


def test_cross_attention_block_bit_exact(oracle, ref):
    """orc_cross_attention_forward against blt_cross_attention_forward compiled from the reference
    (csrc/models/cross_attention.c:101-157)."""
    rs = np.random.RandomState(53)
    arena = ref.blt_arena_create(32 << 20, CPU)
    try:
        for P, T, E, H, kind in ((2, 4, 4, 2, "groups"), (9, 70, 32, 4, "groups"), (16, 64, 64, 2, "uneven"),
                                 (12, 40, 24, 3, "window")):
            xq, xkv = rs.randn(P, E).astype(np.float32), rs.randn(T, E).astype(np.float32)
            ws = [(rs.randn(E, E) / np.sqrt(E)).astype(np.float32) for _ in range(4)]
            cfg = abi.BltMaskConfig()
            cfg.seq_len_q, cfg.seq_len_kv = P, T
            keep = None
            if kind == "window":
                cfg.sliding_window = 7
            else:
                # every patch owns at least one byte (a patch without one is fatal: mask_builder_cpu.c:93)
                extra = rs.randint(0, P, size=T - P) if kind == "groups" else rs.randint(0, 3, size=T - P)
                groups = np.sort(np.concatenate([np.arange(P), extra]))
                keep = (abi.size_array(list(range(P))), abi.size_array(groups.tolist()))
                cfg.query_group_ids, cfg.kv_group_ids = keep
                cfg.bidirectional_within_group = True
            mine = np.zeros((P, E), dtype=np.float32)
            assert oracle.orc_cross_attention_forward(
                *(binding.fptr(a.reshape(-1)) for a in (xq, xkv, *ws, mine)), P, T, E, H, C.byref(cfg)) == 0
            theirs = np.zeros((P, E), dtype=np.float32)
            tq, tkv, tw0, tw1, tw2, tw3, to = (abi.tensor_view(a.ctypes.data, a.shape, CPU)
                                               for a in (xq, xkv, *ws, theirs))
            wts = abi.BltCrossAttentionWeights(C.pointer(tw0), C.pointer(tw1), C.pointer(tw2), C.pointer(tw3))
            cc = abi.BltCrossAttentionConfig()
            cc.embed_dim, cc.num_heads, cc.head_dim = E, H, E // H
            cc.mask_config = C.pointer(cfg)
            arena.contents.offset = 0
            ref.blt_cross_attention_forward(C.byref(tq), C.byref(tkv), C.byref(wts), C.byref(to), C.byref(cc), arena)
            assert mine.tobytes() == theirs.tobytes(), (P, T, E, H, kind)
    finally:
        ref.blt_arena_destroy(arena)


def test_row_ops_bit_exact(oracle, ref):
    """orc_rmsnorm_forward / orc_add / orc_swiglu_forward against the reference's ops
    (csrc/ops/reductions_cpu.c:327-352, elementwise_cpu.c:9-18, 86-99)."""
    rs = np.random.RandomState(51)
    for rows, dim in ((1, 8), (13, 128), (64, 512), (5, 33)):
        x = (rs.randn(rows, dim) * 3).astype(np.float32)
        w = rs.randn(dim).astype(np.float32)
        mine, theirs = np.zeros_like(x), np.zeros_like(x)
        oracle.orc_rmsnorm_forward(binding.fptr(x.reshape(-1)), binding.fptr(w), binding.fptr(mine.reshape(-1)), rows,
                                   dim)
        tx, tw, to = abi.tensor_view(x.ctypes.data, x.shape, CPU), abi.tensor_view(w.ctypes.data, w.shape, CPU), \
            abi.tensor_view(theirs.ctypes.data, theirs.shape, CPU)
        ref.blt_rmsnorm_forward(C.byref(tx), C.byref(tw), C.byref(to))
        assert mine.tobytes() == theirs.tobytes()
        y = rs.randn(rows, dim).astype(np.float32)
        for mine_fn, ref_fn in ((oracle.orc_add, ref.blt_add), (oracle.orc_swiglu_forward, ref.blt_swiglu_forward)):
            mine, theirs = np.zeros_like(x), np.zeros_like(x)
            mine_fn(binding.fptr(x.reshape(-1)), binding.fptr(y.reshape(-1)), binding.fptr(mine.reshape(-1)),
                    rows * dim)
            ty, to = abi.tensor_view(y.ctypes.data, y.shape, CPU), abi.tensor_view(theirs.ctypes.data, theirs.shape, CPU)
            ref_fn(C.byref(tx), C.byref(ty), C.byref(to))
            assert mine.tobytes() == theirs.tobytes()


# ---------------------------------------------------------------------------
# the whole incremental decoder step (csrc/infer/kv_cache.c:112-416)
# ---------------------------------------------------------------------------
DECODER_CASES = [
    # E, H, XH, L, hidden, V, max_len, k_split, window, all_layers, placement
    dict(E=16, H=2, XH=2, L=2, hidden=24, V=19, max_len=40, k=1, window=0, all_layers=True, placement=0),
    dict(E=24, H=3, XH=2, L=3, hidden=40, V=256, max_len=48, k=2, window=7, all_layers=False, placement=0),
    dict(E=16, H=4, XH=1, L=2, hidden=16, V=11, max_len=32, k=1, window=0, all_layers=False, placement=4),  # FIRST
    dict(E=16, H=2, XH=4, L=2, hidden=16, V=11, max_len=32, k=3, window=5, all_layers=True, placement=1),   # NONE
]


def _host_decoder(oracle, c, seed):
    from fblt_amd import decoder
    hd, half = c["E"] // c["H"], c["E"] // c["H"] // 2
    cos, sin = (np.empty(c["max_len"] * half, dtype=np.float32) for _ in range(2))
    assert oracle.orc_rope_precompute(c["max_len"], 500000.0, hd, binding.fptr(cos), binding.fptr(sin)) == 0
    w = decoder.random_weights(c["E"], c["hidden"], c["L"], c["V"], seed)
    bound = decoder.bind(w, cos.reshape(c["max_len"], half), sin.reshape(c["max_len"], half), CPU, decoder.host_place,
                         c["E"], c["H"], c["XH"], c["hidden"], c["V"], c["max_len"], patch_dim=c["k"] * c["E"],
                         window=c["window"], all_layers=c["all_layers"], placement=c["placement"])
    return bound


@pytest.mark.parametrize("case", range(len(DECODER_CASES)))
def test_kv_decode_step_bit_exact(case, oracle, ref):
    """orc_kv_cache_refresh_cross + orc_kv_decode_step against blt_kv_cache_refresh_cross +
    blt_kv_decode_step compiled from the reference, over a prefill chunk, single-row steps and a
    re-segmentation (truncate to the common patches, refresh, decode again): logits and all four
    cache tiers bit for bit; then the reference's own invariant -- the cached steps give the dense
    decoder forward's logits (tests/unit/infer/unit_kv_cache.c:136-151)."""
    from fblt_amd import decoder
    c = DECODER_CASES[case]
    E, V, k = c["E"], c["V"], c["k"]
    rs = np.random.RandomState(100 + case)
    bound = _host_decoder(oracle, c, 200 + case)
    assert all(bool(ref.blt_local_cross_attn_fires(c["placement"], c["all_layers"], c["L"], l)) ==
               bool(oracle.orc_local_cross_attn_fires(c["placement"], int(c["all_layers"]), c["L"], l))
               for l in range(c["L"]))
    mine = decoder.HostCache(bound, c["max_len"])
    arena = ref.blt_arena_create(64 << 20, CPU)
    try:
        theirs = ref.blt_kv_cache_create_batched(arena, bound.ptr, c["max_len"], 1)
        mark = arena.contents.offset
        total_bytes = 21
        d0_all = rs.randn(total_bytes, E).astype(np.float32)
        # (patch lengths so far, from_patch for the refresh, rows to decode, trailing_closed)
        script = [([3, 4], 0, 7, 0), ([3, 4, 1], 2, 1, 0), ([3, 4, 2], 2, 1, 1), ([3, 4, 2, 5], 3, 5, 0),
                  ([3, 4, 2, 5, 1], 4, 1, 0), ([3, 4, 2, 5, 4], 4, 3, 1), ([3, 4, 2, 5, 4, 3], 5, 3, 0)]
        done = 0
        all_logits = []
        for lengths, from_patch, n, closed in script:
            P = len(lengths)
            patches = decoder.patch_table(lengths)
            patch_in = rs.randn(P, k * E).astype(np.float32)
            if from_patch:   # rows of completed patches do not change (append-only tier 2)
                patch_in[:from_patch] = prev_patch_in[:from_patch]
            prev_patch_in = patch_in
            tp = abi.tensor_view(patch_in.ctypes.data, patch_in.shape, CPU)
            same = ref.blt_kv_cache_common_patches(theirs, patches, P)
            assert same >= min(from_patch, theirs.contents.cross_num_patches)
            ref.blt_kv_cache_truncate(theirs, theirs.contents.self_len, min(from_patch, theirs.contents.cross_num_patches))
            ref.blt_kv_cache_refresh_cross(theirs, C.byref(tp), patches, P, from_patch, arena)
            assert oracle.orc_kv_cache_refresh_cross(mine.ptr, 0, binding.fptr(patch_in.reshape(-1)), P,
                                                     from_patch) == 0
            rows = np.ascontiguousarray(d0_all[done:done + n])
            got, want = np.zeros((n, V), dtype=np.float32), np.zeros((n, V), dtype=np.float32)
            td, tl = abi.tensor_view(rows.ctypes.data, rows.shape, CPU), abi.tensor_view(want.ctypes.data, want.shape, CPU)
            arena.contents.offset = mark
            ref.blt_kv_decode_step(theirs, C.byref(tp), patches, P, C.byref(td), closed, C.byref(tl), arena)
            assert oracle.orc_kv_decode_step(mine.ptr, 0, done, patches, P, binding.fptr(rows.reshape(-1)), n, closed,
                                             binding.fptr(got.reshape(-1))) == 0
            assert got.tobytes() == want.tobytes(), (case, lengths, n)
            done += n
            assert theirs.contents.self_len == done
            for name in ("self_k", "self_v", "cross_k", "cross_v"):
                for l in range(c["L"]):
                    t = getattr(theirs.contents, name)[l]
                    view = np.ctypeslib.as_array(C.cast(t.data, C.POINTER(C.c_float)), shape=(c["max_len"], E))
                    assert view.tobytes() == mine.tiers[name][l].tobytes(), (name, l, lengths)
            all_logits.append((done - n, closed, got))
        assert done == total_bytes
        ref.blt_kv_cache_destroy(theirs)
        # the reference's invariant: with the segmentation known up front, decoding in chunks gives
        # the dense forward's logits bit for bit, whatever the chunking
        lengths = script[-1][0]
        P = len(lengths)
        patches = decoder.patch_table(lengths)
        th = abi.tensor_view(d0_all.ctypes.data, d0_all.shape, CPU)
        tp = abi.tensor_view(prev_patch_in.ctypes.data, prev_patch_in.shape, CPU)
        for closed, chunks in ((0, (4, 1, 1, 6, 9)), (1, (21,)), (1, (1,) * 21), (0, (10, 11))):
            dense = np.zeros((total_bytes, V), dtype=np.float32)
            tl = abi.tensor_view(dense.ctypes.data, dense.shape, CPU)
            arena.contents.offset = mark
            ref.blt_local_decoder_forward_ext(bound.ptr, C.byref(th), C.byref(tp), patches, P, None, None, None, 0,
                                              None, closed, C.byref(tl), None, arena)
            fresh = decoder.HostCache(bound, c["max_len"])
            assert oracle.orc_kv_cache_refresh_cross(fresh.ptr, 0, binding.fptr(prev_patch_in.reshape(-1)), P, 0) == 0
            at = 0
            for n in chunks:
                rows = np.ascontiguousarray(d0_all[at:at + n])
                got = np.zeros((n, V), dtype=np.float32)
                last = at + n == total_bytes
                assert oracle.orc_kv_decode_step(fresh.ptr, 0, at, patches, P, binding.fptr(rows.reshape(-1)), n,
                                                 closed if last else 0, binding.fptr(got.reshape(-1))) == 0
                assert got.tobytes() == dense[at:at + n].tobytes(), (case, closed, chunks, at)
                at += n
    finally:
        ref.blt_arena_destroy(arena)


# ---------------------------------------------------------------------------
# inference-mode diffusion forward (csrc/models/block_diffusion.c:776-795)
# ---------------------------------------------------------------------------
# (patch lengths of the clean prefix, block rows, trailing_closed, d0 mode, how the block is filled)
DIFFUSION_SCRIPTS = [
    ([3, 4, 2], 4, 1, abi.BLT_D0_ZEROS, "draft"),      # blt_draft_block's batch: all [MASK], positions N + r, o_M
    ([3, 4, 2, 5], 8, 1, abi.BLT_D0_LEARNED, "draft"),
    ([5, 1, 6], 3, 0, abi.BLT_D0_LEARNED, "mixed"),    # some cells unmasked, groups and positions of the caller's
    ([2, 2, 2, 2, 3], 16, 1, abi.BLT_D0_ZEROS, "mixed"),
    ([7], 1, 1, abi.BLT_D0_LEARNED, "draft"),
]


def _block_batch(decoder, rs, N, R, P, fill, closed, max_len):
    if fill == "draft":
        return decoder.BlockBatch(N, R, P, trailing_closed=closed)
    tokens = [int(rs.randint(0, 256)) if rs.rand() < 0.5 else abi.BLT_MASK_TOKEN_ID for _ in range(R)]
    positions = [int(x) for x in np.sort(rs.randint(0, max_len, size=R))]
    groups = [int(rs.randint(0, P)) for _ in range(R)]
    return decoder.BlockBatch(N, R, P, tokens=tokens, positions=positions, groups=groups, trailing_closed=closed)


@pytest.mark.parametrize("script", range(len(DIFFUSION_SCRIPTS)))
@pytest.mark.parametrize("case", range(len(DECODER_CASES)))
def test_diffusion_infer_bit_exact(case, script, oracle, ref):
    """orc_local_decoder_forward_diffusion_infer against blt_local_decoder_forward_diffusion_infer
    compiled from the reference: logits of all N + R rows bit for bit, for four decoder
    configurations (sub-token split, cross-attention placements, window set -- which this forward
    ignores) and block sections as the draft loop builds them and as a caller may.  Then the
    cached form: the prefix through orc_kv_decode_step, the block rows through orc_kv_block_step
    -- the dense forward's block rows bit for bit (a clean row never sees a block row)."""
    from fblt_amd import decoder
    c = dict(DECODER_CASES[case])
    lengths, R, closed, d0_mode, fill = DIFFUSION_SCRIPTS[script]
    E, V, k = c["E"], c["V"], c["k"]
    N, P = sum(lengths), len(lengths)
    if N + R > c["max_len"]:
        pytest.skip("sequence longer than this decoder's tables")
    rs = np.random.RandomState(7000 + 10 * case + script)
    bound = _host_decoder(oracle, c, 300 + case)
    patches = decoder.patch_table(lengths)
    hidden = rs.randn(N, E).astype(np.float32)
    patch_in = rs.randn(P, k * E).astype(np.float32)
    batch = _block_batch(decoder, rs, N, R, P, fill, closed, c["max_len"])
    got = np.zeros((N + R, V), dtype=np.float32)
    assert oracle.orc_local_decoder_forward_diffusion_infer(
        bound.ptr, binding.fptr(hidden.reshape(-1)), binding.fptr(patch_in.reshape(-1)), patches, P, batch.ptr,
        d0_mode, binding.fptr(got.reshape(-1))) == 0
    want = np.zeros((N + R, V), dtype=np.float32)
    arena = ref.blt_arena_create(64 << 20, CPU)
    try:
        th = abi.tensor_view(hidden.ctypes.data, hidden.shape, CPU)
        tp = abi.tensor_view(patch_in.ctypes.data, patch_in.shape, CPU)
        tl = abi.tensor_view(want.ctypes.data, want.shape, CPU)
        ref.blt_local_decoder_forward_diffusion_infer(bound.ptr, C.byref(th), C.byref(tp), patches, P, batch.ptr,
                                                      d0_mode, C.byref(tl), arena)
    finally:
        ref.blt_arena_destroy(arena)
    assert np.isfinite(want).all()
    assert got.tobytes() == want.tobytes(), (case, script)

    # cached form; the dense forward has no window, so the prefix is cached without one
    bound.struct.config.local_window = 0
    cache = decoder.HostCache(bound, c["max_len"])
    assert oracle.orc_kv_cache_refresh_cross(cache.ptr, 0, binding.fptr(patch_in.reshape(-1)), P, 0) == 0
    clean = np.zeros((N, V), dtype=np.float32)
    assert oracle.orc_kv_decode_step(cache.ptr, 0, 0, patches, P, binding.fptr(hidden.reshape(-1)), N, closed,
                                     binding.fptr(clean.reshape(-1))) == 0
    assert clean.tobytes() == want[:N].tobytes(), (case, script, "clean rows")
    block = np.zeros((R, V), dtype=np.float32)
    assert oracle.orc_kv_block_step(cache.ptr, 0, N, P, batch.ptr, d0_mode, binding.fptr(block.reshape(-1))) == 0
    assert block.tobytes() == want[N:].tobytes(), (case, script, "block rows")


# ---------------------------------------------------------------------------
# the transformer block (csrc/models/transformer.c:97-128)
# ---------------------------------------------------------------------------
from tests.golden.block_cases import transformer_case  # noqa: E402


TRANSFORMER_SHAPES = [(2, 8, 2, 12, "causal"), (33, 32, 4, 48, "window"), (70, 48, 3, 64, "docs"),
                      (40, 64, 2, 96, "docs_window")]


@pytest.mark.parametrize("shape", TRANSFORMER_SHAPES)
def test_transformer_block_bit_exact(shape, oracle, ref):
    """orc_transformer_forward against blt_transformer_forward compiled from the reference."""
    T, E, H, hidden, mask = shape
    rs = np.random.RandomState(T * 131 + E)
    x, w, cfg, _keep = transformer_case(rs, T, E, H, hidden, mask)
    mine = np.zeros((T, E), dtype=np.float32)
    order = ("norm1", "qkv", "proj", "norm2", "up", "gate", "down")
    assert oracle.orc_transformer_forward(binding.fptr(x.reshape(-1)), *(binding.fptr(w[n].reshape(-1)) for n in order),
                                          binding.fptr(mine.reshape(-1)), T, E, hidden, H, 1, 1, 500000.0, None, None,
                                          C.byref(cfg)) == 0
    theirs = np.zeros((T, E), dtype=np.float32)
    tv = {n: abi.tensor_view(w[n].ctypes.data, w[n].shape, CPU) for n in order}
    wt = abi.BltTransformerWeights()
    wt.norm1_weight, wt.attn_qkv_w, wt.attn_proj_w = C.pointer(tv["norm1"]), C.pointer(tv["qkv"]), C.pointer(tv["proj"])
    wt.norm2_weight, wt.ffn_up_w, wt.ffn_gate_w = C.pointer(tv["norm2"]), C.pointer(tv["up"]), C.pointer(tv["gate"])
    wt.ffn_down_w = C.pointer(tv["down"])
    tc = abi.BltTransformerConfig()
    ac = tc.attn_config
    ac.embed_dim, ac.num_heads, ac.head_dim, ac.is_causal, ac.use_rope, ac.rope_theta = E, H, E // H, True, True, 500000.0
    ac.mask_config = C.pointer(cfg)
    tc.hidden_dim, tc.norm_type, tc.activation_type = hidden, abi.BLT_NORM_RMSNORM, abi.BLT_ACTIVATION_SWIGLU
    tx, to = abi.tensor_view(x.ctypes.data, x.shape, CPU), abi.tensor_view(theirs.ctypes.data, theirs.shape, CPU)
    arena = ref.blt_arena_create(64 << 20, CPU)
    try:
        ref.blt_transformer_forward(C.byref(tx), C.byref(wt), C.byref(to), C.byref(tc), arena)
    finally:
        ref.blt_arena_destroy(arena)
    assert np.isfinite(theirs).all()
    assert mine.tobytes() == theirs.tobytes(), shape


def test_encoder_ops_bit_exact(oracle, ref):
    """The encoder's three small ops and its hashing against the reference build: indexed row
    accumulation with sentinel entries, in-place scale, patch pooling (mean and maximum, patches of
    1 ... 30 rows), and the bucket index list of every n-gram size 1 ... 8 out of the reference's
    own rolling-hash state machine (csrc/models/hash_ngram.c:16-79)."""
    rs = np.random.RandomState(77)
    T, E, V = 91, 24, 131
    table = rs.randn(V, E).astype(np.float32)
    idx = rs.randint(0, V, size=T).astype(np.uint32)
    idx[rs.randint(0, T, size=9)] = abi.BLT_IDX_SENTINEL
    io0 = rs.randn(T, E).astype(np.float32)
    mine, theirs = io0.copy(), io0.copy()
    u32 = C.POINTER(C.c_uint32)
    assert oracle.orc_indexed_row_accumulate(binding.fptr(table.reshape(-1)), V, idx.ctypes.data_as(u32),
                                             binding.fptr(mine.reshape(-1)), T, E) == 0
    tt, ti = abi.tensor_view(table.ctypes.data, table.shape, CPU), abi.tensor_view(theirs.ctypes.data, theirs.shape, CPU)
    ref.blt_indexed_row_accumulate(C.byref(tt), idx.ctypes.data_as(u32), C.byref(ti))
    assert mine.tobytes() == theirs.tobytes() and not np.array_equal(mine, io0)
    oracle.orc_scale(binding.fptr(mine.reshape(-1)), mine.size, 1.0 / 7.0)
    ref.blt_scale(C.byref(ti), 1.0 / 7.0)
    assert mine.tobytes() == theirs.tobytes()

    lengths = [1, 30, 2, 7, 1, 13, 5, 9, 23]
    patches = decoder.patch_table(lengths)
    h = rs.randn(sum(lengths), E).astype(np.float32)
    for pool in (abi.BLT_POOL_MEAN, abi.BLT_POOL_MAX):
        a, b = (np.zeros((len(lengths), E), dtype=np.float32) for _ in range(2))
        assert oracle.orc_patch_pool_forward(binding.fptr(h.reshape(-1)), h.shape[0], E, patches, len(lengths), pool,
                                             binding.fptr(a.reshape(-1))) == 0
        th, tb = abi.tensor_view(h.ctypes.data, h.shape, CPU), abi.tensor_view(b.ctypes.data, b.shape, CPU)
        ref.blt_patch_pool_forward(C.byref(th), patches, len(lengths), pool, C.byref(tb))
        assert a.tobytes() == b.tobytes() and np.abs(a).sum() > 0

    class State(C.Structure):   # csrc/models/hash_ngram.h:29-38
        _fields_ = [("current_hash", C.c_uint64), ("prime", C.c_uint64), ("modulus", C.c_uint64),
                    ("prime_pow_n", C.c_uint64), ("window", C.c_uint8 * 8), ("window_start", C.c_size_t),
                    ("n", C.c_size_t), ("positions_seen", C.c_size_t)]
    ref.blt_rolling_hash_init.restype = None
    ref.blt_rolling_hash_init.argtypes = [C.POINTER(State), C.c_size_t, C.c_uint64, C.c_uint64]
    ref.blt_rolling_hash_update.restype = C.c_uint64
    ref.blt_rolling_hash_update.argtypes = [C.POINTER(State), C.c_uint8]
    data = rs.randint(0, 256, size=300).astype(np.uint8)
    data[40:60] = 7
    for n in range(1, 9):
        for prime, modulus in ((1000003, 50021), (31, 2), (2 ** 31 - 1, 2 ** 31 + 11)):
            got = np.zeros(data.size, dtype=np.uint32)
            assert oracle.orc_ngram_indices(data.ctypes.data_as(C.POINTER(C.c_uint8)), data.size, n, prime, modulus,
                                            got.ctypes.data_as(u32)) == 0
            st = State()
            ref.blt_rolling_hash_init(C.byref(st), n, prime, modulus)
            want = []
            for b in data:
                hv = ref.blt_rolling_hash_update(C.byref(st), int(b))
                want.append(abi.BLT_IDX_SENTINEL if hv == 2 ** 64 - 1 else hv & 0xFFFFFFFF)
            assert got.tolist() == want, (n, prime, modulus)


ENCODER_SHAPES = [
    dict(T=37, E=16, H=2, XH=2, L=1, hidden=24, ngrams=(3,), vocab=101, k=1, window=0, placement=0, all_layers=True,
         pool="mean", docs=None, normalize=True, mean_patch=3),
    dict(T=64, E=32, H=2, XH=4, L=2, hidden=40, ngrams=(2, 5, 8), vocab=257, k=2, window=9, placement=0,
         all_layers=False, pool="max", docs=[20, 41], normalize=False, mean_patch=5),
    dict(T=50, E=24, H=3, XH=1, L=3, hidden=32, ngrams=(0, 4, 60), vocab=64, k=3, window=0, placement=4,
         all_layers=False, pool="mean", docs=[25], normalize=True, mean_patch=2),
    dict(T=29, E=16, H=1, XH=2, L=2, hidden=16, ngrams=(), vocab=8, k=1, window=5, placement=1, all_layers=True,
         pool="mean", docs=None, normalize=True, mean_patch=7),
    dict(T=48, E=32, H=4, XH=2, L=2, hidden=48, ngrams=(3, 4, 5, 6, 7, 8), vocab=509, k=1, window=0, placement=3,
         all_layers=False, pool="max", docs=None, normalize=True, mean_patch=4),
]


@pytest.mark.parametrize("shape", range(len(ENCODER_SHAPES)))
def test_local_encoder_bit_exact(shape, oracle, ref):
    """orc_local_encoder_forward against blt_local_encoder_forward compiled from the reference:
    patch_out and byte_hidden_out bit for bit, over sub-token splits, window, documents, every kind
    of cross placement (none at all included), both pools, 0 ... 6 n-gram tables (sizes of 0 and
    beyond the sequence are skipped as the reference skips them)."""
    from tests import encoder_runs
    from tests.golden.block_cases import encoder_case
    c = ENCODER_SHAPES[shape]
    data, lengths, weights = encoder_case(np.random.RandomState(900 + shape), c)
    mine = encoder_runs.run_oracle(oracle, c, data, lengths, weights)
    theirs = encoder_runs.run_reference(ref, oracle, c, data, lengths, weights)
    for a, b in zip(mine, theirs):
        assert np.isfinite(b).all() and np.abs(b).sum() > 0
        assert a.tobytes() == b.tobytes(), shape



# ---------------------------------------------------------------------------
# the plain decoder forward and the whole-model forward (csrc/models/local_decoder.c:233-351,
# csrc/models/model.c:68-144)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("case", range(len(DECODER_CASES)))
@pytest.mark.parametrize("closed,docs", [(0, []), (1, []), (0, [5, 11])])
def test_local_decoder_forward_bit_exact(case, closed, docs, oracle, ref):
    """orc_local_decoder_forward against blt_local_decoder_forward_ext of the reference build: every
    decoder configuration of this file (sub-token split, window, placements), trailing_closed, and
    document boundaries in the byte mask."""
    from fblt_amd import decoder
    c = DECODER_CASES[case]
    CPU = abi.BLT_BACKEND_CPU
    bound = _host_decoder(oracle, c, 900 + case)
    rs = np.random.RandomState(900 + case)
    lengths = [3, 4, 2, 5, 1, 6]
    T, P, E, V = sum(lengths), len(lengths), c["E"], c["V"]
    patches = decoder.patch_table(lengths)
    pdim = c["E"] * c["k"]
    hidden = rs.randn(T, E).astype(np.float32)
    patch_in = rs.randn(P, pdim).astype(np.float32)
    bounds = abi.size_array(docs) if docs else None
    num_docs = len(docs) + 1 if docs else 0
    want, got = np.zeros((T, V), dtype=np.float32), np.zeros((T, V), dtype=np.float32)
    th, tp = abi.tensor_view(hidden.ctypes.data, hidden.shape, CPU), abi.tensor_view(patch_in.ctypes.data, patch_in.shape, CPU)
    tl = abi.tensor_view(want.ctypes.data, want.shape, CPU)
    arena = ref.blt_arena_create(64 << 20, CPU)
    try:
        ref.blt_local_decoder_forward_ext(bound.ptr, C.byref(th), C.byref(tp), patches, P, None, None, bounds, num_docs,
                                          None, closed, C.byref(tl), None, arena)
    finally:
        ref.blt_arena_destroy(arena)
    assert oracle.orc_local_decoder_forward(bound.ptr, binding.fptr(hidden.reshape(-1)), T,
                                            binding.fptr(patch_in.reshape(-1)), patches, P, bounds, num_docs, closed,
                                            binding.fptr(got.reshape(-1))) == 0
    assert got.tobytes() == want.tobytes()


@pytest.mark.parametrize("name", ["model_T96", "model_T200_docs_window"])
def test_model_forward_bit_exact(name, oracle, ref):
    """blt_model_encode + blt_model_decode of the reference build (encoder, patch transformer,
    decoder, LM head; the inference forward without the loss) against the composition of the
    restated stages: logits bit for bit."""
    from fblt_amd import decoder
    from tests import model_runs
    if not hasattr(ref, "blt_model_encode"):
        pytest.skip("oracle/_ref/libblt_ref.so predates the model driver: rebuild it (make -C oracle ref)")
    args = model_runs.inputs(name)

    def fill(t, arr):
        C.memmove(t.contents.data, arr.ctypes.data, arr.nbytes)

    want = model_runs.run(ref, ref, oracle, abi.BLT_BACKEND_CPU, decoder.host_place, fill, lambda: None, *args)
    got = model_runs.run_oracle(oracle, *args)
    assert np.isfinite(want).all() and np.abs(want).max() > 1e-3
    assert got.tobytes() == want.tobytes()
