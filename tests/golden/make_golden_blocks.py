"""Writes tests/golden/blocks_golden.npz from the reference build (oracle/_ref):
blt_multihead_attention, blt_cross_attention_forward, the script of
blt_kv_cache_refresh_cross + blt_kv_decode_step calls and the
blt_transformer_forward and blt_local_decoder_forward_diffusion_infer cases of block_cases.py.

Run in a container that holds the reference sources:
    make -C oracle ref && python tests/golden/make_golden_blocks.py

Stored per case: SHA-256 of the full outputs (bit-exact check for the CPU checker) and up to
4096 sampled values (tolerance check for the GPU path).  Inputs are regenerated from the seed.
"""
import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from fblt_amd import abi, decoder  # noqa: E402
from oracle import binding  # noqa: E402
from tests.golden import block_cases as bc  # noqa: E402
from tests.golden.make_golden import pack  # noqa: E402

CPU = abi.BLT_BACKEND_CPU


def view(a):
    return abi.tensor_view(a.ctypes.data, a.shape, CPU)


def rope_tables(ref, rows, hd):
    cos, sin = np.zeros((rows, hd // 2), dtype=np.float32), np.zeros((rows, hd // 2), dtype=np.float32)
    vc, vs = view(cos), view(sin)
    cfg = binding.BltRopeConfig(bc.THETA, hd)
    ref.blt_rope_precompute(rows, C.byref(cfg), C.byref(vc), C.byref(vs))
    return cos, sin


def run_mha(ref, arena, name):
    c, x, wqkv, wproj = bc.mha_inputs(name)
    T, E, H = c["T"], c["E"], c["H"]
    causal, window, docs = bc.mha_mask(c)
    cfg = abi.BltMaskConfig()
    cfg.seq_len_q = cfg.seq_len_kv = T
    cfg.is_causal, cfg.sliding_window = causal, window
    keep = abi.size_array(docs) if docs else None
    if docs:
        cfg.doc_boundaries, cfg.num_docs = keep, len(docs) + 1
    ac = abi.BltAttentionConfig()
    ac.embed_dim, ac.num_heads, ac.head_dim = E, H, E // H
    ac.use_rope, ac.rope_theta, ac.mask_config = c["rope"], bc.THETA, C.pointer(cfg)
    out = np.zeros((T, E), dtype=np.float32)
    tx, tq, tp, to = view(x), view(wqkv), view(wproj), view(out)
    arena.contents.offset = 0
    ref.blt_multihead_attention(C.byref(tx), C.byref(tq), C.byref(tp), C.byref(to), C.byref(ac), arena)
    return out


def run_xattn(ref, arena, name):
    c, xq, xkv, ws, groups = bc.xattn_inputs(name)
    P, T, E, H = c["P"], c["T"], c["E"], c["H"]
    cfg = abi.BltMaskConfig()
    cfg.seq_len_q, cfg.seq_len_kv = P, T
    keep = (abi.size_array(list(range(P))), abi.size_array(groups.tolist()))
    cfg.query_group_ids, cfg.kv_group_ids, cfg.bidirectional_within_group = keep[0], keep[1], True
    out = np.zeros((P, E), dtype=np.float32)
    tq, tkv, to = view(xq), view(xkv), view(out)
    tw = [view(w) for w in ws]
    wts = abi.BltCrossAttentionWeights(*(C.pointer(t) for t in tw))
    cc = abi.BltCrossAttentionConfig()
    cc.embed_dim, cc.num_heads, cc.head_dim, cc.mask_config = E, H, E // H, C.pointer(cfg)
    arena.contents.offset = 0
    ref.blt_cross_attention_forward(C.byref(tq), C.byref(tkv), C.byref(wts), C.byref(to), C.byref(cc), arena)
    return out


def run_step(ref, arena, name):
    c, weights, d0, latents = bc.step_inputs(name)
    E, V = c["E"], c["V"]
    cos, sin = rope_tables(ref, c["max_len"], E // c["H"])
    bound = decoder.bind(weights, cos, sin, CPU, decoder.host_place, E, c["H"], c["XH"], c["hidden"], V, c["max_len"],
                         patch_dim=c["k"] * E, window=c["window"], all_layers=c["all_layers"],
                         placement=c["placement"], theta=bc.THETA)
    arena.contents.offset = 0
    cache = ref.blt_kv_cache_create_batched(arena, bound.ptr, c["max_len"], 1)
    mark = arena.contents.offset
    logits, done = [], 0
    for (lengths, from_patch, n, closed), pin in zip(bc.STEP_SCRIPT, latents):
        P = len(lengths)
        patches = decoder.patch_table(lengths)
        tp = view(pin)
        ref.blt_kv_cache_truncate(cache, cache.contents.self_len, min(from_patch, cache.contents.cross_num_patches))
        arena.contents.offset = mark
        ref.blt_kv_cache_refresh_cross(cache, C.byref(tp), patches, P, from_patch, arena)
        rows = np.ascontiguousarray(d0[done:done + n])
        out = np.zeros((n, V), dtype=np.float32)
        td, tl = view(rows), view(out)
        ref.blt_kv_decode_step(cache, C.byref(tp), patches, P, C.byref(td), closed, C.byref(tl), arena)
        logits.append(out)
        done += n
    tiers = {}
    for tier in ("self_k", "self_v", "cross_k", "cross_v"):
        tiers[tier] = np.stack([np.ctypeslib.as_array(C.cast(getattr(cache.contents, tier)[l].data,
                                                             C.POINTER(C.c_float)), shape=(c["max_len"], E)).copy()
                                for l in range(c["L"])])
    ref.blt_kv_cache_destroy(cache)
    return np.concatenate(logits), tiers


def run_diffusion(ref, arena, name):
    c, weights, hidden, latents, batch = bc.diffusion_inputs(name)
    E, V = c["E"], c["V"]
    cos, sin = rope_tables(ref, c["max_len"], E // c["H"])
    bound = decoder.bind(weights, cos, sin, CPU, decoder.host_place, E, c["H"], c["XH"], c["hidden"], V, c["max_len"],
                         patch_dim=c["k"] * E, window=c["window"], all_layers=c["all_layers"],
                         placement=c["placement"], theta=bc.THETA)
    N, P = sum(c["lengths"]), len(c["lengths"])
    out = np.zeros((N + c["R"], V), dtype=np.float32)
    th, tp, tl = view(hidden), view(latents), view(out)
    arena.contents.offset = 0
    ref.blt_local_decoder_forward_diffusion_infer(bound.ptr, C.byref(th), C.byref(tp), decoder.patch_table(c["lengths"]),
                                                  P, batch.ptr, abi.BLT_D0_LEARNED if c["learned"] else abi.BLT_D0_ZEROS,
                                                  C.byref(tl), arena)
    return out


WEIGHT_ORDER = ("norm1", "qkv", "proj", "norm2", "up", "gate", "down")


def transformer_structs(w, cfg, E, H, hidden, make_view):
    """blt_transformer_weights / blt_transformer_config over the case's arrays (views kept alive by the caller)."""
    tv = {n: make_view(w[n]) for n in WEIGHT_ORDER}
    wt = abi.BltTransformerWeights()
    wt.norm1_weight, wt.attn_qkv_w, wt.attn_proj_w = C.pointer(tv["norm1"]), C.pointer(tv["qkv"]), C.pointer(tv["proj"])
    wt.norm2_weight, wt.ffn_up_w, wt.ffn_gate_w = C.pointer(tv["norm2"]), C.pointer(tv["up"]), C.pointer(tv["gate"])
    wt.ffn_down_w = C.pointer(tv["down"])
    tc = abi.BltTransformerConfig()
    ac = tc.attn_config
    ac.embed_dim, ac.num_heads, ac.head_dim, ac.is_causal, ac.use_rope, ac.rope_theta = E, H, E // H, True, True, bc.THETA
    ac.mask_config = C.pointer(cfg)
    tc.hidden_dim, tc.norm_type, tc.activation_type = hidden, abi.BLT_NORM_RMSNORM, abi.BLT_ACTIVATION_SWIGLU
    return wt, tc, tv


def run_transformer(ref, arena, name):
    T, E, H, hidden, _mask, x, w, cfg, _keep = bc.transformer_inputs(name)
    wt, tc, _tv = transformer_structs(w, cfg, E, H, hidden, view)
    out = np.zeros((T, E), dtype=np.float32)
    tx, to = view(x), view(out)
    arena.contents.offset = 0
    ref.blt_transformer_forward(C.byref(tx), C.byref(wt), C.byref(to), C.byref(tc), arena)
    return out


def run_encoder(ref, name):
    """blt_local_encoder_forward of the reference build on host tensors."""
    from tests import encoder_runs
    c, data, lengths, weights = bc.encoder_inputs(name)
    return encoder_runs.run_reference(ref, binding.load_oracle(), c, data, lengths, weights)


def main():
    ref = binding.load_ref()
    if ref is None:
        raise SystemExit("oracle/_ref/libblt_ref.so is missing: run `make -C oracle ref` first")
    rs = np.random.RandomState(20240701)
    store = {}
    arena = ref.blt_arena_create(64 << 20, CPU)
    for name in bc.MHA_CASES:
        pack(store, name + "/out", run_mha(ref, arena, name), rs)
    for name in bc.XATTN_CASES:
        pack(store, name + "/out", run_xattn(ref, arena, name), rs)
    for name in bc.STEP_CASES:
        logits, tiers = run_step(ref, arena, name)
        pack(store, name + "/logits", logits, rs)
        for tier, arr in tiers.items():
            pack(store, name + "/" + tier, arr, rs)
    for name in bc.TRANSFORMER_CASES:
        pack(store, name + "/out", run_transformer(ref, arena, name), rs)
    for name in bc.DIFFUSION_CASES:
        pack(store, name + "/logits", run_diffusion(ref, arena, name), rs)
    for name in bc.ENCODER_CASES:
        patch_out, byte_hidden = run_encoder(ref, name)
        pack(store, name + "/patch_out", patch_out, rs)
        pack(store, name + "/byte_hidden_out", byte_hidden, rs)
    ref.blt_arena_destroy(arena)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "blocks_golden.npz")
    np.savez_compressed(path, **store)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
