"""Writes tests/golden/attention_golden.npz from the reference's own CPU ops.

Run in a container that holds the reference sources:
    make -C oracle ref && python tests/golden/make_golden.py

For every case the seeded workload (fblt_amd/workloads.py) is pushed through
oracle/_ref/libblt_ref.so with the reference's call decomposition (one
blt_attention_head_core call per (sequence, head), dense masks from
blt_build_attention_mask / blt_build_block_diffusion_mask, write-through by
blt_strided_copy before attending).  Inputs are regenerated from the seed by
the tests, so only outputs are stored: the SHA-256 of the full output bytes
(bit-exact check for the CPU checker) and 4096 sampled values per case
(tolerance check for the GPU path at full size).
"""
import ctypes as C
import hashlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from fblt_amd import abi, workloads  # noqa: E402
from oracle import binding  # noqa: E402

CPU = abi.BLT_BACKEND_CPU
_fp = C.POINTER(C.c_float)

DENSE_CASES = {
    "c1_full": lambda: workloads.config1(),
    "c2_full": lambda: workloads.config2(),
    "c3_full": lambda: workloads.config3(),
    "c1_small": lambda: workloads.config1(batch=1, T=96, H=2, hd=32),
    "c2_small": lambda: workloads.config2(batch=2, P=48, H=2, hd=64, T_bytes=192),
    "c3_small": lambda: workloads.config3(batch=2, T=128, P=32, H=2, hd=32),
}
KV_CASES = {
    "c4_full_8steps": lambda: workloads.config4(steps=8),
    "c4_full_256steps": lambda: workloads.config4(),   # BASELINE config 4 as stated: 64 sequences, 256 consecutive steps
    "c4_small": lambda: workloads.config4(batch=3, steps=5, len_hi=70),
    "c5_B4": lambda: workloads.config5(B=4),
    "c5_B8": lambda: workloads.config5(B=8),
    "c5_B16": lambda: workloads.config5(B=16),
    "c4_rope_small": lambda: workloads.config4(batch=5, steps=6, len_hi=90, rope=True),
    "c5_B8_rope_small": lambda: workloads.config5(batch=4, B=8, len_hi=120, max_seq_len=160, rope=True),
}


def ref_mask(ref, arena, h, w):
    cfg = abi.BltMaskConfig()
    cfg.seq_len_q, cfg.seq_len_kv = h.nq, h.nk
    keep = []
    if h.mask == "causal":
        cfg.is_causal = True
    else:
        lo_name, hi_name, off = h.mask_ref
        lo, hi = w.ranges[lo_name][off:off + h.nq], w.ranges[hi_name][off:off + h.nq]
        starts, lens = lo.astype(np.int64), (hi - lo).astype(np.int64)
        patches = abi.patch_array(starts, lens)
        qg, kg = abi.size_array([0] * h.nq), abi.size_array([0] * h.nk)
        ref.blt_patch_build_group_ids(patches, h.nq, h.nk, qg, kg)   # the reference's own byte->patch index
        keep += [qg, kg]
        cfg.query_group_ids, cfg.kv_group_ids = qg, kg
        cfg.bidirectional_within_group = True
    t = abi.BltTensor()
    ref.blt_build_attention_mask(C.byref(cfg), C.byref(t), arena)
    return t.data, keep


def run_dense(ref, w):
    arena = ref.blt_arena_create(64 << 20, CPU)
    scratch = np.empty(max(h.nq * h.nk for h in w.heads), dtype=np.float32)
    masks = {}
    for h in w.heads:
        key = (h.mask, h.mask_ref, h.nq, h.nk)
        if key not in masks:
            masks[key] = ref_mask(ref, arena, h, w)
        a = binding.head_args(w.buffers[h.q[0]], w.buffers[h.k[0]], w.buffers[h.v[0]], w.buffers[h.out[0]], h.nq,
                              h.nk, h.hd, h.scale, h.q[2], h.k[2], h.v[2], h.out[2], h.out[3], q_off=h.q[1],
                              k_off=h.k[1], v_off=h.v[1], weights=scratch)
        a.combined = w.buffers[h.out[0]].ctypes.data + 4 * h.out[1]
        a.mask = masks[key][0]
        ref.blt_attention_head_core(CPU, C.byref(a))
    ref.blt_arena_destroy(arena)
    return w.buffers["out"].copy()


def run_kv(ref, kw):
    E, H, hd, n = kw.E, kw.H, kw.hd, kw.n
    ck, cv = kw.cache_k.copy(), kw.cache_v.copy()
    kd, vd = ck.reshape(-1), cv.reshape(-1)
    lens = kw.lens.astype(np.int64).copy()
    out = np.zeros((kw.steps, kw.batch * n, E), dtype=np.float32)
    arena = ref.blt_arena_create(64 << 20, CPU)
    scale = float(np.float32(1) / np.sqrt(np.float32(hd)))
    for s in range(kw.steps):
        for b in range(kw.batch):
            base = int(lens[b])
            total = base + n
            slab = b * kw.max_seq_len * E
            q = np.ascontiguousarray(kw.q_new[s, b * n:(b + 1) * n])
            k = np.ascontiguousarray(kw.k_new[s, b * n:(b + 1) * n])
            v = np.ascontiguousarray(kw.v_new[s, b * n:(b + 1) * n])
            if kw.rope_cos is not None:
                # kv_cache.c:262-271, 349-358: rows of the tables at positions base..base+n-1 (the position
                # gather is a row copy), then the reference's blt_rope_apply on Q and K
                rc, rs = kw.rope_cos[base:base + n], kw.rope_sin[base:base + n]
                q = binding.ref_rope_apply(ref, q.reshape(n, H, hd), rc, rs).reshape(n, E)
                k = binding.ref_rope_apply(ref, k.reshape(n, H, hd), rc, rs).reshape(n, E)
            for h in range(H):   # write-through first (kv_cache.c:363-365)
                for dst, src in ((kd, k), (vd, v)):
                    ref.blt_strided_copy(CPU, C.cast(dst.ctypes.data + 4 * (slab + base * E + h * hd), _fp), E,
                                         C.cast(src.ctypes.data + 4 * h * hd, _fp), E, n, hd)
            arena.contents.offset = 0
            t = abi.BltTensor()
            if kw.kind == "causal":
                cfg = abi.BltMaskConfig()   # same cells as the inline host loop kv_cache.c:229-236
                cfg.seq_len_q, cfg.seq_len_kv = n, total
                cfg.is_causal, cfg.causal_offset, cfg.sliding_window = True, base, kw.window
                ref.blt_build_attention_mask(C.byref(cfg), C.byref(t), arena)
                mask_ptr = t.data
            else:
                cfg = abi.BltBlockDiffusionConfig()
                cfg.mode, cfg.seq_len, cfg.num_clean = abi.BLT_BDM_INFER, total, base
                ref.blt_build_block_diffusion_mask(C.byref(cfg), C.byref(t), arena)
                mask_ptr = t.data + 4 * base * total   # rows [base, total) are the block rows
            scratch = np.empty(n * total, dtype=np.float32)
            comb = out[s, b * n:(b + 1) * n]
            for h in range(H):
                a = binding.head_args(q.reshape(-1), kd, vd, comb.reshape(-1), n, total, hd, scale, E, E, E, E,
                                      h * hd, q_off=h * hd, k_off=slab + h * hd, v_off=slab + h * hd, scratch=scratch)
                a.combined = comb.ctypes.data
                a.mask = mask_ptr
                ref.blt_attention_head_core(CPU, C.byref(a))
        if kw.commit:
            lens += n
    ref.blt_arena_destroy(arena)
    return out, ck, cv


def pack(store, name, arr, rs):
    flat = np.ascontiguousarray(arr).reshape(-1)
    idx = np.sort(rs.choice(flat.size, size=min(4096, flat.size), replace=False)).astype(np.int64)
    store[name + "/sha256"] = np.frombuffer(hashlib.sha256(flat.tobytes()).digest(), dtype=np.uint8)
    store[name + "/idx"] = idx
    store[name + "/val"] = flat[idx]
    store[name + "/size"] = np.array([flat.size], dtype=np.int64)


def main():
    ref = binding.load_ref()
    if ref is None:
        raise SystemExit("oracle/_ref/libblt_ref.so is missing: run `make -C oracle ref` first")
    rs = np.random.RandomState(20240601)
    store = {}
    for name, make in DENSE_CASES.items():
        pack(store, name + "/out", run_dense(ref, make()), rs)
        print("done", name)
    for name, make in KV_CASES.items():
        out, ck, cv = run_kv(ref, make())
        pack(store, name + "/out", out, rs)
        pack(store, name + "/cache_k", ck, rs)
        pack(store, name + "/cache_v", cv, rs)
        print("done", name)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "attention_golden.npz")
    np.savez_compressed(path, **store)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
