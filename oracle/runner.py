"""TEST INFRASTRUCTURE -- runs a workload through the CPU checker.

The call decomposition is the reference's: one attention-core call per
(sequence, head); a dense additive mask built by the restated mask builder and
passed in for the dense configurations; write-through then attend for the
KV-cache step (csrc/models/attention.c:197-202, cross_attention.c:145-150,
csrc/infer/kv_cache.c:343-390).
"""
import ctypes as C
import time

import numpy as np

from fblt_amd import abi
from oracle import binding

_fp = C.POINTER(C.c_float)


def _mask_for(lib, w, head, cache):
    """Dense additive mask [nq, nk] of a head, built by the restated builders."""
    if head.mask == "none":
        return None
    if head.mask == "causal":
        key = ("causal", head.nq, head.nk, head.causal_offset, head.window)
        if key not in cache:
            cfg = abi.BltMaskConfig()
            cfg.seq_len_q, cfg.seq_len_kv = head.nq, head.nk
            cfg.is_causal = True
            cfg.causal_offset = head.causal_offset
            cfg.sliding_window = head.window
            out = np.empty(head.nq * head.nk, dtype=np.float32)
            rc = lib.orc_build_attention_mask(C.byref(cfg), binding.fptr(out))
            assert rc == 0, rc
            cache[key] = out
        return cache[key]
    if head.mask == "range":
        lo_name, hi_name, off = head.mask_ref
        key = ("range", lo_name, off, head.nq, head.nk)
        if key not in cache:
            lo = w.ranges[lo_name][off:off + head.nq]
            hi = w.ranges[hi_name][off:off + head.nq]
            # group ids: query row i is group i, key j belongs to the row whose range holds it
            kv = np.full(head.nk, head.nq, dtype=np.uint64)
            for i in range(head.nq):
                kv[lo[i]:hi[i]] = i
            qg = abi.size_array(range(head.nq))
            kg = abi.size_array(kv)
            cfg = abi.BltMaskConfig()
            cfg.seq_len_q, cfg.seq_len_kv = head.nq, head.nk
            cfg.query_group_ids = qg
            cfg.kv_group_ids = kg
            cfg.bidirectional_within_group = True
            out = np.empty(head.nq * head.nk, dtype=np.float32)
            rc = lib.orc_build_attention_mask(C.byref(cfg), binding.fptr(out))
            assert rc in (0, 4), rc
            cache[key] = out
        return cache[key]
    if head.mask == "dense":
        name, off = head.mask_ref
        return w.buffers[name][off:off + head.nq * head.nk]
    raise ValueError(head.mask)


def head_arg_array(lib, w, use_causal_flag=False, weights=None):
    """(ctypes array of blt_attention_head_args over host buffers, keep-alive list)."""
    keep, cache = [], {}
    arr = (abi.BltAttentionHeadArgs * len(w.heads))()
    max_scores = max(h.nq * h.nk for h in w.heads)
    scratch = np.empty(max_scores, dtype=np.float32)
    keep.append(scratch)
    for t, h in enumerate(w.heads):
        mask = None
        causal = False
        if h.mask == "causal" and use_causal_flag and h.causal_offset == 0 and h.window == 0:
            causal = True
        else:
            mask = _mask_for(lib, w, h, cache)
        qb, kb, vb, ob = w.buffers[h.q[0]], w.buffers[h.k[0]], w.buffers[h.v[0]], w.buffers[h.out[0]]
        a = binding.head_args(qb, kb, vb, ob, h.nq, h.nk, h.hd, h.scale, h.q[2], h.k[2], h.v[2], h.out[2], h.out[3],
                              q_off=h.q[1], k_off=h.k[1], v_off=h.v[1],
                              weights=None if weights is None else weights[t], scratch=scratch, mask=mask,
                              causal=causal)
        a.combined = ob.ctypes.data + 4 * h.out[1]
        arr[t] = a
        keep.append(mask)
    keep.append(cache)
    return arr, keep


def run(w, lib=None, use_causal_flag=False, weights=None, timed=False):
    """Fill the workload's output buffers through the checker; returns seconds when timed."""
    lib = lib or binding.load_oracle()
    arr, keep = head_arg_array(lib, w, use_causal_flag, weights)
    t0 = time.perf_counter()
    rc = lib.orc_attention_head_core_many(arr, len(w.heads))
    dt = time.perf_counter() - t0
    assert rc == 0, rc
    del keep
    return dt if timed else None


def run_ref(w, ref, lib=None, timed=False):
    """The same pass through the reference's own blt_attention_head_core (oracle/_ref build), one call
    per (sequence, head) as its callers make them; masks come from the restated builder (untimed)."""
    lib = lib or binding.load_oracle()
    arr, keep = head_arg_array(lib, w)
    t0 = time.perf_counter()
    for t in range(len(w.heads)):
        ref.blt_attention_head_core(abi.BLT_BACKEND_CPU, C.byref(arr[t]))
    dt = time.perf_counter() - t0
    del keep
    return dt if timed else None


def run_kv(kw, lib=None, steps=None, timed=False):
    """KV-cache workload: returns combined [steps, batch*n, E]; mutates a COPY of the cache."""
    lib = lib or binding.load_oracle()
    steps = kw.steps if steps is None else steps
    E, H, n, batch = kw.E, kw.H, kw.n, kw.batch
    ck, cv = kw.cache_k.copy(), kw.cache_v.copy()
    lens = kw.lens.astype(np.int64).copy()
    out = np.zeros((steps, batch * n, E), dtype=np.float32)
    elapsed = 0.0
    for s in range(steps):
        t0 = time.perf_counter()
        for b in range(batch):
            rows = slice(b * n, (b + 1) * n)
            q = np.ascontiguousarray(kw.q_new[s, rows])
            k = np.ascontiguousarray(kw.k_new[s, rows])
            v = np.ascontiguousarray(kw.v_new[s, rows])
            comb = out[s, rows]
            base = int(lens[b])
            if kw.rope_cos is not None and kw.kind == "causal":
                rc = lib.orc_kv_rope_attend_step(binding.fptr(ck.reshape(-1)), binding.fptr(cv.reshape(-1)),
                                                 kw.max_seq_len, E, H, b, base, n, kw.window, binding.fptr(q), E,
                                                 binding.fptr(k), E, binding.fptr(v), E,
                                                 binding.fptr(kw.rope_cos.reshape(-1)),
                                                 binding.fptr(kw.rope_sin.reshape(-1)), kw.rope_cos.shape[0],
                                                 binding.fptr(comb.reshape(-1)))
                assert rc == 0, rc
                continue
            if kw.rope_cos is not None:
                q, k = _rotate_rows(lib, kw, base, q), _rotate_rows(lib, kw, base, k)
            if kw.kind == "causal":
                rc = lib.orc_kv_attend_step(binding.fptr(ck.reshape(-1)), binding.fptr(cv.reshape(-1)),
                                            kw.max_seq_len, E, H, b, base, n, kw.window, binding.fptr(q),
                                            binding.fptr(k), binding.fptr(v), binding.fptr(comb.reshape(-1)))
                assert rc == 0, rc
            else:
                _block_rows(lib, kw, ck, cv, b, base, q, k, v, comb)
        elapsed += time.perf_counter() - t0
        if kw.commit:
            lens += n
    return (out, ck, cv, elapsed) if timed else (out, ck, cv)


def _rotate_rows(lib, kw, base, x):
    """Rows [n, E] at positions base..base+n-1 rotated head by head
    (csrc/infer/kv_cache.c:262-271, 349-358; block rows: models/block_diffusion.c:264-277)."""
    n, H, hd = x.shape[0], kw.H, kw.hd
    half = hd // 2
    pos = abi.size_array(range(base, base + n))
    rc, rs = np.empty(n * half, dtype=np.float32), np.empty(n * half, dtype=np.float32)
    assert lib.orc_rope_position_gather(binding.fptr(kw.rope_cos.reshape(-1)), binding.fptr(kw.rope_sin.reshape(-1)),
                                        kw.rope_cos.shape[0], half, pos, n, binding.fptr(rc), binding.fptr(rs)) == 0
    out = np.empty_like(x)
    lib.orc_rope_apply(binding.fptr(np.ascontiguousarray(x).reshape(-1)), n, H, hd, binding.fptr(rc), binding.fptr(rs),
                       binding.fptr(out.reshape(-1)))
    return out


def _block_rows(lib, kw, ck, cv, b, base, q, k, v, comb):
    """Block rows of the [prefix ; block] sequence under the INFER mask
    (csrc/models/block_diffusion.c:196-204, 293-319): K/V rows of the block are
    in place at rows [base, base+B), the B queries use mask rows [base, base+B)."""
    E, H, n, hd = kw.E, kw.H, kw.n, kw.hd
    S = base + n
    r0 = b * kw.max_seq_len
    ck[r0 + base:r0 + S] = k
    cv[r0 + base:r0 + S] = v
    cfg = abi.BltBlockDiffusionConfig()
    cfg.mode = abi.BLT_BDM_INFER
    cfg.seq_len, cfg.num_clean = S, base
    full = np.empty(S * S, dtype=np.float32)
    rc = lib.orc_build_block_diffusion_mask(C.byref(cfg), binding.fptr(full))
    assert rc == 0, rc
    mask = np.ascontiguousarray(full.reshape(S, S)[base:S])
    scratch = np.empty(n * S, dtype=np.float32)
    comb[:] = 0.0
    kflat, vflat = ck.reshape(-1), cv.reshape(-1)
    for h in range(H):
        a = binding.head_args(q, kflat, vflat, comb, n, S, hd, float(np.float32(1.0) / np.sqrt(np.float32(hd))),
                              E, E, E, E, h * hd, q_off=h * hd, k_off=r0 * E + h * hd, v_off=r0 * E + h * hd,
                              scratch=scratch, mask=mask)
        rc = lib.orc_attention_head_core(C.byref(a))
        assert rc == 0, rc
