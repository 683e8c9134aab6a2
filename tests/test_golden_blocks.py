"""Golden vectors of the block-level entry points, written by tests/golden/make_golden_blocks.py
from the reference build: blt_multihead_attention, blt_cross_attention_forward, a script of
blt_kv_cache_refresh_cross + blt_kv_decode_step calls and blt_local_decoder_forward_diffusion_infer.  CPU: the checker reproduces every output
bit for bit (SHA-256).  GPU: the HIP library matches the stored samples within
|got - ref| <= 1e-5 + 1e-4 |ref|."""
import ctypes as C
import hashlib
import os

import numpy as np
import pytest

from fblt_amd import abi, decoder
from oracle import binding
from tests.golden import block_cases as bc

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "blocks_golden.npz"))
CPU, HIP = abi.BLT_BACKEND_CPU, abi.BLT_BACKEND_HIP


def check(arr, key, exact):
    flat = np.ascontiguousarray(arr).reshape(-1)
    assert flat.size == int(GOLD[key + "/size"][0])
    if exact:
        digest = np.frombuffer(hashlib.sha256(flat.tobytes()).digest(), dtype=np.uint8)
        assert (digest == GOLD[key + "/sha256"]).all(), key
    got, want = flat[GOLD[key + "/idx"]].astype(np.float64), GOLD[key + "/val"].astype(np.float64)
    assert (np.abs(got - want) <= (0.0 if exact else 1e-5 + 1e-4 * np.abs(want))).all(), (key, float(np.abs(got - want).max()))


def mask_config(c):
    causal, window, docs = bc.mha_mask(c)
    cfg = abi.BltMaskConfig()
    cfg.seq_len_q = cfg.seq_len_kv = c["T"]
    cfg.is_causal, cfg.sliding_window = causal, window
    keep = abi.size_array(docs) if docs else None
    if docs:
        cfg.doc_boundaries, cfg.num_docs = keep, len(docs) + 1
    return cfg, keep


def group_config(P, T, groups):
    cfg = abi.BltMaskConfig()
    cfg.seq_len_q, cfg.seq_len_kv = P, T
    keep = (abi.size_array(list(range(P))), abi.size_array(groups.tolist()))
    cfg.query_group_ids, cfg.kv_group_ids, cfg.bidirectional_within_group = keep[0], keep[1], True
    return cfg, keep


def host_tables(oracle, rows, hd):
    cos, sin = (np.empty(rows * (hd // 2), dtype=np.float32) for _ in range(2))
    assert oracle.orc_rope_precompute(rows, bc.THETA, hd, binding.fptr(cos), binding.fptr(sin)) == 0
    return cos.reshape(rows, hd // 2), sin.reshape(rows, hd // 2)


# ---------------------------------------------------------------------------- CPU: the checker
@pytest.mark.parametrize("name", list(bc.MHA_CASES))
def test_oracle_reproduces_reference_attention_block(name, oracle):
    c, x, wqkv, wproj = bc.mha_inputs(name)
    cfg, _keep = mask_config(c)
    out = np.zeros((c["T"], c["E"]), dtype=np.float32)
    assert oracle.orc_multihead_attention(*(binding.fptr(a.reshape(-1)) for a in (x, wqkv, wproj, out)), c["T"],
                                          c["E"], c["H"], 0, int(c["rope"]), bc.THETA, None, None,
                                          C.byref(cfg)) == 0
    check(out, name + "/out", exact=True)


@pytest.mark.parametrize("name", list(bc.XATTN_CASES))
def test_oracle_reproduces_reference_cross_block(name, oracle):
    c, xq, xkv, ws, groups = bc.xattn_inputs(name)
    cfg, _keep = group_config(c["P"], c["T"], groups)
    out = np.zeros((c["P"], c["E"]), dtype=np.float32)
    assert oracle.orc_cross_attention_forward(*(binding.fptr(a.reshape(-1)) for a in (xq, xkv, *ws, out)), c["P"],
                                              c["T"], c["E"], c["H"], C.byref(cfg)) == 0
    check(out, name + "/out", exact=True)


@pytest.mark.parametrize("name", list(bc.STEP_CASES))
def test_oracle_reproduces_reference_decoder_steps(name, oracle):
    c, weights, d0, latents = bc.step_inputs(name)
    E, V = c["E"], c["V"]
    cos, sin = host_tables(oracle, c["max_len"], E // c["H"])
    bound = decoder.bind(weights, cos, sin, CPU, decoder.host_place, E, c["H"], c["XH"], c["hidden"], V, c["max_len"],
                         patch_dim=c["k"] * E, window=c["window"], all_layers=c["all_layers"],
                         placement=c["placement"], theta=bc.THETA)
    cache = decoder.HostCache(bound, c["max_len"])
    logits, done = [], 0
    for (lengths, from_patch, n, closed), pin in zip(bc.STEP_SCRIPT, latents):
        P = len(lengths)
        assert oracle.orc_kv_cache_refresh_cross(cache.ptr, 0, binding.fptr(pin.reshape(-1)), P, from_patch) == 0
        rows = np.ascontiguousarray(d0[done:done + n])
        out = np.zeros((n, V), dtype=np.float32)
        assert oracle.orc_kv_decode_step(cache.ptr, 0, done, decoder.patch_table(lengths), P,
                                         binding.fptr(rows.reshape(-1)), n, closed, binding.fptr(out.reshape(-1))) == 0
        logits.append(out)
        done += n
    check(np.concatenate(logits), name + "/logits", exact=True)
    for tier in ("self_k", "self_v", "cross_k", "cross_v"):
        check(np.stack(cache.tiers[tier]), name + "/" + tier, exact=True)


@pytest.mark.parametrize("name", list(bc.TRANSFORMER_CASES))
def test_oracle_reproduces_reference_transformer_block(name, oracle):
    T, E, H, hidden, _mask, x, w, cfg, _keep = bc.transformer_inputs(name)
    out = np.zeros((T, E), dtype=np.float32)
    order = ("norm1", "qkv", "proj", "norm2", "up", "gate", "down")
    assert oracle.orc_transformer_forward(binding.fptr(x.reshape(-1)), *(binding.fptr(w[n].reshape(-1)) for n in order),
                                          binding.fptr(out.reshape(-1)), T, E, hidden, H, 1, 1, bc.THETA, None, None,
                                          C.byref(cfg)) == 0
    check(out, name + "/out", exact=True)


@pytest.mark.parametrize("name", list(bc.ENCODER_CASES))
def test_oracle_reproduces_reference_local_encoder(name, oracle):
    from tests import encoder_runs
    c, data, lengths, weights = bc.encoder_inputs(name)
    patch_out, byte_hidden = encoder_runs.run_oracle(oracle, c, data, lengths, weights)
    check(patch_out, name + "/patch_out", exact=True)
    check(byte_hidden, name + "/byte_hidden_out", exact=True)


def _diffusion_decoder(oracle, c, weights, backend, place):
    cos, sin = host_tables(oracle, c["max_len"], c["E"] // c["H"])
    return decoder.bind(weights, cos, sin, backend, place, c["E"], c["H"], c["XH"], c["hidden"], c["V"], c["max_len"],
                        patch_dim=c["k"] * c["E"], window=c["window"], all_layers=c["all_layers"],
                        placement=c["placement"], theta=bc.THETA)


@pytest.mark.parametrize("name", list(bc.DIFFUSION_CASES))
def test_oracle_reproduces_reference_diffusion_forward(name, oracle):
    """The dense restatement, and the cached form (prefix through the incremental step without a
    window, block rows through the block step), both bit for bit what the reference build wrote."""
    c, weights, hidden, latents, batch = bc.diffusion_inputs(name)
    bound = _diffusion_decoder(oracle, c, weights, CPU, decoder.host_place)
    N, P, R, V = sum(c["lengths"]), len(c["lengths"]), c["R"], c["V"]
    mode = abi.BLT_D0_LEARNED if c["learned"] else abi.BLT_D0_ZEROS
    patches = decoder.patch_table(c["lengths"])
    out = np.zeros((N + R, V), dtype=np.float32)
    assert oracle.orc_local_decoder_forward_diffusion_infer(
        bound.ptr, binding.fptr(hidden.reshape(-1)), binding.fptr(latents.reshape(-1)), patches, P, batch.ptr, mode,
        binding.fptr(out.reshape(-1))) == 0
    check(out, name + "/logits", exact=True)
    bound.struct.config.local_window = 0
    cache = decoder.HostCache(bound, c["max_len"])
    assert oracle.orc_kv_cache_refresh_cross(cache.ptr, 0, binding.fptr(latents.reshape(-1)), P, 0) == 0
    two = np.zeros((N + R, V), dtype=np.float32)
    assert oracle.orc_kv_decode_step(cache.ptr, 0, 0, patches, P, binding.fptr(hidden.reshape(-1)), N, c["closed"],
                                     binding.fptr(two[:N].reshape(-1))) == 0
    assert oracle.orc_kv_block_step(cache.ptr, 0, N, P, batch.ptr, mode, binding.fptr(two[N:].reshape(-1))) == 0
    check(two, name + "/logits", exact=True)


# ---------------------------------------------------------------------------- GPU: the library
def dev_view(t):
    return abi.tensor_view(t.data_ptr(), tuple(t.shape), HIP)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(bc.MHA_CASES))
def test_hip_matches_reference_attention_block(name):
    import torch
    from fblt_amd import api
    lib = api.load()
    c, x, wqkv, wproj = bc.mha_inputs(name)
    cfg, _keep = mask_config(c)
    tx, tq, tp = (torch.from_numpy(a).cuda() for a in (x, wqkv, wproj))
    to = torch.full((c["T"], c["E"]), 7.0, dtype=torch.float32, device="cuda")
    ac = abi.BltAttentionConfig()
    ac.embed_dim, ac.num_heads, ac.head_dim = c["E"], c["H"], c["E"] // c["H"]
    ac.use_rope, ac.rope_theta, ac.mask_config = c["rope"], bc.THETA, C.pointer(cfg)
    vx, vq, vp, vo = (dev_view(t) for t in (tx, tq, tp, to))
    arena = lib.blt_arena_create(32 << 20, HIP)
    lib.blt_multihead_attention(C.byref(vx), C.byref(vq), C.byref(vp), C.byref(vo), C.byref(ac), arena)
    lib.blt_backend_pass_sync_hip()
    out = to.cpu().numpy()
    lib.blt_arena_destroy(arena)
    check(out, name + "/out", exact=False)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(bc.XATTN_CASES))
def test_hip_matches_reference_cross_block(name):
    import torch
    from fblt_amd import api
    lib = api.load()
    c, xq, xkv, ws, groups = bc.xattn_inputs(name)
    cfg, _keep = group_config(c["P"], c["T"], groups)
    tens = [torch.from_numpy(a).cuda() for a in (xq, xkv, *ws)]
    to = torch.full((c["P"], c["E"]), 7.0, dtype=torch.float32, device="cuda")
    views = [dev_view(t) for t in tens]
    vo = dev_view(to)
    wts = abi.BltCrossAttentionWeights(*(C.pointer(v) for v in views[2:]))
    cc = abi.BltCrossAttentionConfig()
    cc.embed_dim, cc.num_heads, cc.head_dim, cc.mask_config = c["E"], c["H"], c["E"] // c["H"], C.pointer(cfg)
    arena = lib.blt_arena_create(32 << 20, HIP)
    lib.blt_cross_attention_forward(C.byref(views[0]), C.byref(views[1]), C.byref(wts), C.byref(vo), C.byref(cc), arena)
    lib.blt_backend_pass_sync_hip()
    out = to.cpu().numpy()
    lib.blt_arena_destroy(arena)
    check(out, name + "/out", exact=False)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(bc.STEP_CASES))
def test_hip_matches_reference_decoder_steps(name, oracle):
    import torch
    from fblt_amd import api
    lib = api.load()
    c, weights, d0, latents = bc.step_inputs(name)
    E, V, L = c["E"], c["V"], c["L"]
    cos, sin = host_tables(oracle, c["max_len"], E // c["H"])   # the table formula is pinned separately
    bound = decoder.bind(weights, cos, sin, HIP, decoder.device_place, E, c["H"], c["XH"], c["hidden"], V, c["max_len"],
                         patch_dim=c["k"] * E, window=c["window"], all_layers=c["all_layers"],
                         placement=c["placement"], theta=bc.THETA)
    arena = lib.blt_arena_create(64 << 20, HIP)
    cache = lib.blt_kv_cache_create(arena, bound.ptr, c["max_len"])
    mark = arena.contents.offset
    logits, done = [], 0
    for (lengths, from_patch, n, closed), pin in zip(bc.STEP_SCRIPT, latents):
        P = len(lengths)
        patches = decoder.patch_table(lengths)
        tp = torch.from_numpy(pin).cuda()
        vp = dev_view(tp)
        lib.blt_kv_cache_truncate(cache, cache.contents.self_len, min(from_patch, cache.contents.cross_num_patches))
        arena.contents.offset = mark
        lib.blt_kv_cache_refresh_cross(cache, C.byref(vp), patches, P, from_patch, arena)
        td = torch.from_numpy(np.ascontiguousarray(d0[done:done + n])).cuda()
        tl = torch.full((n, V), 7.0, dtype=torch.float32, device="cuda")
        vd, vl = dev_view(td), dev_view(tl)
        lib.blt_kv_decode_step(cache, C.byref(vp), patches, P, C.byref(vd), closed, C.byref(vl), arena)
        lib.blt_backend_pass_sync_hip()
        logits.append(tl.cpu().numpy())
        done += n
    check(np.concatenate(logits), name + "/logits", exact=False)
    for tier in ("self_k", "self_v", "cross_k", "cross_v"):
        got = np.empty((L, c["max_len"], E), dtype=np.float32)
        for l in range(L):
            lib.blt_hip_memcpy_d2h(got[l].ctypes.data, getattr(cache.contents, tier)[l].data, got[l].nbytes)
        check(got, name + "/" + tier, exact=False)
    lib.blt_kv_cache_destroy(cache)
    lib.blt_arena_destroy(arena)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(bc.DIFFUSION_CASES))
def test_hip_matches_reference_diffusion_forward(name, oracle):
    import torch
    from fblt_amd import api
    lib = api.load()
    c, weights, hidden, latents, batch = bc.diffusion_inputs(name)
    bound = _diffusion_decoder(oracle, c, weights, HIP, decoder.device_place)
    N, P, R, V = sum(c["lengths"]), len(c["lengths"]), c["R"], c["V"]
    mode = abi.BLT_D0_LEARNED if c["learned"] else abi.BLT_D0_ZEROS
    th, tp = torch.from_numpy(hidden).cuda(), torch.from_numpy(latents).cuda()
    tl = torch.full((N + R, V), 7.0, dtype=torch.float32, device="cuda")
    vh, vp, vl = dev_view(th), dev_view(tp), dev_view(tl)
    arena = lib.blt_arena_create(128 << 20, HIP)
    lib.blt_local_decoder_forward_diffusion_infer(bound.ptr, C.byref(vh), C.byref(vp), decoder.patch_table(c["lengths"]),
                                                  P, batch.ptr, mode, C.byref(vl), arena)
    lib.blt_backend_pass_sync_hip()
    out = tl.cpu().numpy()
    lib.blt_arena_destroy(arena)
    check(out, name + "/logits", exact=False)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(bc.TRANSFORMER_CASES))
def test_hip_matches_reference_transformer_block(name):
    import torch
    from fblt_amd import api
    from tests.golden.make_golden_blocks import transformer_structs
    lib = api.load()
    T, E, H, hidden, _mask, x, w, cfg, _keep = bc.transformer_inputs(name)
    tens = {n: torch.from_numpy(a).cuda() for n, a in w.items()}
    wt, tc, _tv = transformer_structs(tens, cfg, E, H, hidden, dev_view)
    tx = torch.from_numpy(x).cuda()
    to = torch.full((T, E), 7.0, dtype=torch.float32, device="cuda")
    vx, vo = dev_view(tx), dev_view(to)
    arena = lib.blt_arena_create(128 << 20, HIP)
    lib.blt_transformer_forward(C.byref(vx), C.byref(wt), C.byref(vo), C.byref(tc), arena)
    lib.blt_backend_pass_sync_hip()
    out = to.cpu().numpy()
    lib.blt_arena_destroy(arena)
    check(out, name + "/out", exact=False)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(bc.ENCODER_CASES))
def test_hip_matches_reference_local_encoder(name, oracle):
    from fblt_amd import api
    from tests import encoder_runs
    lib = api.load()
    c, data, lengths, weights = bc.encoder_inputs(name)
    patch_out, byte_hidden = encoder_runs.run_device(lib.blt_local_encoder_forward, lib, oracle, c, data, lengths,
                                                     weights)
    check(patch_out, name + "/patch_out", exact=False)
    check(byte_hidden, name + "/byte_hidden_out", exact=False)

