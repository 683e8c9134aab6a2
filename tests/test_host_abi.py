"""CPU-only checks of the shipped library: it loads, exports every symbol the
public header declares, its host-side integer code agrees with the checker,
and it fails loudly (never falls back) when asked for CPU compute."""
import ctypes as C
import os
import re
import subprocess
import sys

import numpy as np
import pytest

from fblt_amd import abi, api

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "blt_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(blt_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    lib = C.CDLL(api.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 35
    for n in names:
        assert hasattr(lib, n), "include/blt_hip.h declares %s but the library does not export it" % n
    assert set(names) == set(api.SYMBOLS), set(names) ^ set(api.SYMBOLS)
    assert b"gfx950" in api.load().blt_hip_build_info()


# what the reference's caller code references but this library leaves to the reference build:
# training passes and ops of other model parts, none of them reached from the forward attention
# blocks or the KV-cache step (csrc/models/attention.c:130-207, cross_attention.c:101-157,
# csrc/infer/kv_cache.c:112-428, csrc/models/block_diffusion.c:776-795)
OFF_PATH = {"blt_attention_head_core_backward", "blt_matmul_backward", "blt_rmsnorm_backward",
            "blt_rmsnorm_backward_add", "blt_rope_apply_packed_backward", "blt_swiglu_backward",
            "blt_cross_entropy_forward", "blt_cross_entropy_backward", "blt_gelu_forward",
            "blt_layernorm_forward", "blt_cast", "blt_tensor_view_2d", "blt_tensor_view_3d",
            # training side of csrc/models/block_diffusion.c (D_0 table gradient)
            "blt_indexed_row_scatter_add"}
# the same for the layer stack, patch transformer and local encoder (csrc/models/transformer_stack.c,
# global_transformer.c, local_encoder.c, hash_ngram.c, byte_embedding.c): backward passes, weight
# casts for the reduced-precision modes and pure host helpers that stay with the reference build
STACK_OFF_PATH = OFF_PATH | {"blt_cross_attention_backward", "blt_multihead_attention_backward", "blt_patch_pool_backward",
                             "blt_embedding_scatter_add", "blt_indexed_row_scatter_add_normalized", "blt_scaled_copy",
                             "blt_local_byte_grad_view", "blt_local_byte_layer_config", "blt_local_byte_weights_view",
                             "blt_local_cross_weights_view", "blt_local_layer_grad_alloc",
                             "blt_local_layer_storage_alloc", "blt_transformer_backward", "blt_transformer_forward_cached",
                             "blt_cast_fp32_to_bf16", "blt_cast_fp32_to_fp8", "blt_matmul_bf16", "blt_matmul_fp8"}


def test_reference_callers_find_their_ops_in_the_library():
    """The reference's attention blocks and KV-cache step, compiled unmodified, leave their tensor
    ops undefined; every one of those that is on the path is exported by the HIP library under the
    reference's own name (the drop-in arrangement the GPU tests then run)."""
    so = os.path.join(ROOT, "oracle", "_ref", "libblt_ref_callers.so")
    if not os.path.exists(so):
        pytest.skip("oracle/_ref/libblt_ref_callers.so was not built (needs the reference sources)")
    out = subprocess.run(["nm", "-D", "-u", so], capture_output=True, text=True, check=True).stdout
    wanted = {line.split()[-1] for line in out.splitlines() if line.split()[-1].startswith("blt_")}
    assert len(wanted) >= 25
    lib = C.CDLL(api.LIB_PATH)
    missing = {n for n in wanted - OFF_PATH if not hasattr(lib, n)}
    assert not missing, missing
    for n in ("blt_attention_head_core", "blt_build_attention_mask", "blt_matmul", "blt_rope_apply", "blt_rows_gather",
              "blt_strided_copy", "blt_rmsnorm_forward", "blt_swiglu_forward", "blt_add", "blt_tensor_create",
              "blt_tensor_upload", "blt_arena_alloc"):
        assert n in wanted, n


def test_reference_encoder_and_stack_find_their_ops_in_the_library():
    """The same for the reference's layer stack, patch transformer and local encoder: everything
    their forward passes call is exported here, the two fused blocks (blt_transformer_forward,
    blt_cross_attention_forward) and the encoder's small ops included."""
    so = os.path.join(ROOT, "oracle", "_ref", "libblt_ref_stack_callers.so")
    if not os.path.exists(so):
        pytest.skip("oracle/_ref/libblt_ref_stack_callers.so was not built (needs the reference sources)")
    out = subprocess.run(["nm", "-D", "-u", so], capture_output=True, text=True, check=True).stdout
    wanted = {line.split()[-1] for line in out.splitlines() if line.split()[-1].startswith("blt_")}
    lib = C.CDLL(api.LIB_PATH)
    ref = C.CDLL(os.path.join(ROOT, "oracle", "_ref", "libblt_ref.so"))
    missing = {n for n in wanted if not hasattr(lib, n) and not hasattr(ref, n)}
    assert not missing, missing
    for n in ("blt_transformer_forward", "blt_cross_attention_forward", "blt_embedding_lookup",
              "blt_indexed_row_accumulate", "blt_scale", "blt_patch_pool_forward", "blt_rmsnorm_forward", "blt_add",
              "blt_strided_copy", "blt_tensor_create", "blt_tensor_download", "blt_patch_build_group_ids"):
        assert n in wanted and hasattr(lib, n), n
    off = {n for n in wanted if not hasattr(lib, n)}
    assert off <= STACK_OFF_PATH, off - STACK_OFF_PATH


def test_header_layout_assertions_compile():
    """include/blt_abi.h carries its own static assertions; compile it as C99 and C++17."""
    for cc, std, lang in (("gcc", "-std=c99", "c"), ("g++", "-std=c++17", "c++")):
        src = '#include "blt_abi.h"\n#include "blt_hip.h"\nint main(void){return 0;}\n'
        p = subprocess.run([cc, std, "-x", lang, "-fsyntax-only", "-I", os.path.join(ROOT, "include"), "-"],
                           input=src, text=True, capture_output=True)
        assert p.returncode == 0, p.stderr


LAYOUT_PROBE = r"""
#include <stdio.h>
#include <stddef.h>
%s
#define S(t) printf(#t " %%zu\n", sizeof(t))
#define O(t, f) printf(#t "." #f " %%zu\n", offsetof(t, f))
int main(void) {
    S(blt_tensor); O(blt_tensor, strides); O(blt_tensor, dtype); O(blt_tensor, is_view); S(blt_arena);
    S(blt_attention_head_args); O(blt_attention_head_args, combined_col_offset); O(blt_attention_head_args, lse_out);
    O(blt_attention_head_args, mask); O(blt_attention_head_args, is_causal); O(blt_attention_head_args, scale);
    S(blt_mask_config); O(blt_mask_config, doc_boundaries); O(blt_mask_config, kv_group_ids);
    O(blt_mask_config, is_causal); O(blt_mask_config, causal_offset);
    S(blt_block_diffusion_config); S(blt_patch_info); O(blt_patch_info, peak_entropy);
    S(blt_rope_config); S(blt_attention_config); O(blt_attention_config, use_rope); O(blt_attention_config, rope_theta);
    O(blt_attention_config, mask_config);
    S(blt_cross_attention_config); O(blt_cross_attention_config, split_mode); O(blt_cross_attention_config, num_heads);
    O(blt_cross_attention_config, mask_config); S(blt_cross_attention_weights); O(blt_cross_attention_weights, weight_proj);
    S(blt_transformer_weights); O(blt_transformer_weights, ffn_gate_w);
    S(blt_local_layer_storage); O(blt_local_layer_storage, cross_norm_weight); O(blt_local_layer_storage, cross_weight_proj);
    S(blt_local_decoder_config); O(blt_local_decoder_config, cross_attn_all_layers);
    O(blt_local_decoder_config, cross_attn_placement); O(blt_local_decoder_config, rope_theta);
    O(blt_local_decoder_config, max_seq_len); O(blt_local_decoder_config, vocab_size);
    S(blt_local_decoder); O(blt_local_decoder, rope_sin_cache); O(blt_local_decoder, layers);
    O(blt_local_decoder, lm_head_weight); O(blt_local_decoder, d0_embed_weight);
    S(blt_kv_cache); O(blt_kv_cache, k); O(blt_kv_cache, self_k); O(blt_kv_cache, self_len); O(blt_kv_cache, cross_k);
    O(blt_kv_cache, cross_num_patches); O(blt_kv_cache, cached_patches);
    S(blt_transformer_config); O(blt_transformer_config, hidden_dim); O(blt_transformer_config, layer_norm_eps);
    O(blt_transformer_config, norm_type); O(blt_transformer_config, activation_type); O(blt_transformer_config, use_bf16);
    S(blt_block_batch); O(blt_block_batch, t); O(blt_block_batch, tokens); O(blt_block_batch, positions);
    O(blt_block_batch, groups); O(blt_block_batch, loss_scale); O(blt_block_batch, trailing_closed);
    S(blt_local_decoder_d0_opts); O(blt_local_decoder_d0_opts, num_hfinal_rows);
    O(blt_local_decoder_d0_opts, d0_extra_tokens);
    S(blt_hash_ngram_config); O(blt_hash_ngram_config, num_ngram_sizes); O(blt_hash_ngram_config, per_ngram_vocab);
    O(blt_hash_ngram_config, hash_prime); O(blt_hash_ngram_config, normalize); O(blt_hash_ngram_config, embed_dim);
    S(blt_hash_ngram_weights); O(blt_hash_ngram_weights, num_tables);
    S(blt_local_encoder_config); O(blt_local_encoder_config, patch_dim); O(blt_local_encoder_config, cross_attn_all_layers);
    O(blt_local_encoder_config, cross_attn_placement); O(blt_local_encoder_config, pool_type);
    O(blt_local_encoder_config, ngram_config); O(blt_local_encoder_config, rope_theta);
    O(blt_local_encoder_config, max_seq_len);
    S(blt_local_encoder); O(blt_local_encoder, byte_embedding_weight); O(blt_local_encoder, ngram_weights);
    O(blt_local_encoder, rope_cos_cache); O(blt_local_encoder, rope_sin_cache); O(blt_local_encoder, layers);
    printf("enum3 %%d %%u %%d\n", (int)BLT_POOL_MAX, (unsigned)BLT_IDX_SENTINEL, (int)BLT_MAX_NGRAM_SIZES);
    printf("enum %%d %%d %%d %%d %%d %%u\n", (int)BLT_XATTN_FIRST, (int)BLT_DTYPE_FP32, (int)BLT_BACKEND_CPU,
           (int)BLT_CROSS_ATTN_SPLIT_KV, (int)BLT_D0_LEARNED, (unsigned)BLT_MASK_TOKEN_ID);
    printf("enum2 %%d %%d\n", (int)BLT_NORM_RMSNORM, (int)BLT_ACTIVATION_SWIGLU);
    return 0;
}
"""

REF_ROOT = "/root/reference/csrc"


@pytest.mark.skipif(not os.path.isdir(REF_ROOT), reason="the reference headers are not on this machine")
def test_layout_matches_reference_headers(tmp_path):
    """Sizes and member offsets of every mirrored struct, printed once by a program compiled against
    the reference's own headers and once against include/blt_abi.h, must read the same."""
    ref_inc = "\n".join('#include "%s"' % h for h in (
        "core/tensor.h", "core/allocator.h", "ops/attn_core.h", "ops/mask_builder.h", "ops/rope.h",
        "models/attention.h", "models/cross_attention.h", "models/transformer.h", "models/patcher.h",
        "models/local_decoder.h", "infer/kv_cache.h", "models/block_diffusion.h", "models/local_encoder.h",
        "ops/gather_scatter.h"))
    outs = []
    for tag, inc_dir, inc in (("ref", REF_ROOT, ref_inc), ("own", os.path.join(ROOT, "include"), '#include "blt_abi.h"')):
        src = tmp_path / (tag + ".c")
        src.write_text(LAYOUT_PROBE % inc)
        exe = str(tmp_path / tag)
        p = subprocess.run(["gcc", "-std=c99", "-D_POSIX_C_SOURCE=200809L", "-I", inc_dir, str(src), "-o", exe],
                           capture_output=True, text=True)
        assert p.returncode == 0, p.stderr
        outs.append(subprocess.run([exe], capture_output=True, text=True, check=True).stdout)
    assert outs[0] == outs[1] and outs[0].count("\n") > 50


def test_kv_cache_container_bookkeeping():
    """Host side of csrc/infer/kv_cache.c:27-110 on a host arena: shapes, zero fill, truncate,
    common patches, reset, and the placement rule of csrc/models/local_common.c:49-64."""
    lib = api.load()
    dec = abi.BltLocalDecoder()
    dec.config.embed_dim, dec.config.patch_dim, dec.config.max_seq_len, dec.config.num_layers = 8, 24, 32, 3
    arena = lib.blt_arena_create(1 << 20, abi.BLT_BACKEND_CPU)
    cache = lib.blt_kv_cache_create_batched(arena, C.byref(dec), 20, 5)
    c = cache.contents
    assert (c.max_seq_len, c.batch_size, c.max_subtokens, c.embed_dim, c.k, c.patch_dim) == (20, 5, 20, 8, 3, 24)
    for l in range(3):
        for tier in (c.self_k, c.self_v, c.cross_k, c.cross_v):
            assert tuple(tier[l].shape[:2]) == (100, 8) and tier[l].numel == 800
            assert not np.ctypeslib.as_array(C.cast(tier[l].data, C.POINTER(C.c_float)), shape=(800,)).any()
    assert c.self_len == 0 and c.cross_num_patches == 0
    new = abi.patch_array([0, 3, 7], [3, 4, 2])
    assert lib.blt_kv_cache_common_patches(cache, new, 3) == 0      # nothing cached yet
    for i, (s0, ln) in enumerate(((0, 3), (3, 4), (7, 5))):
        c.cached_patches[i].start_idx, c.cached_patches[i].length = s0, ln
    lib.blt_kv_cache_truncate(cache, 12, 3)
    assert (c.self_len, c.cross_num_patches) == (12, 3)
    assert lib.blt_kv_cache_common_patches(cache, new, 3) == 2      # the third patch changed its length
    assert lib.blt_kv_cache_common_patches(cache, new, 1) == 1
    lib.blt_kv_cache_reset(cache)
    assert (c.self_len, c.cross_num_patches) == (0, 0)
    lib.blt_kv_cache_destroy(cache)
    lib.blt_arena_destroy(arena)
    fires = lambda placement, all_layers, L: [bool(lib.blt_local_cross_attn_fires(placement, all_layers, L, l))
                                              for l in range(L)]
    assert fires(abi.BLT_XATTN_DEFAULT, True, 3) == [True, True, True]
    assert fires(abi.BLT_XATTN_DEFAULT, False, 3) == [False, False, True]
    assert fires(abi.BLT_XATTN_NONE, True, 3) == [False, False, False]
    assert fires(abi.BLT_XATTN_LAST, True, 3) == [False, False, True]
    assert fires(abi.BLT_XATTN_ALL, False, 3) == [True, True, True]
    assert fires(abi.BLT_XATTN_FIRST, True, 3) == [True, False, False]


def test_patch_helpers_match_checker(oracle):
    lib = api.load()
    rs = np.random.RandomState(21)
    for _ in range(80):
        P = rs.randint(1, 14)
        lens = rs.randint(1, 17, size=P)
        starts = np.concatenate(([0], np.cumsum(lens)[:-1]))
        if rs.randint(4) == 0:
            starts = starts + rs.randint(1, 5)
        p = abi.patch_array(starts, lens)
        T = int(starts[-1] + lens[-1])
        for pos in range(T + 4):
            assert lib.blt_patch_decoder_latent_at(p, P, pos) == oracle.orc_patch_decoder_latent_at(p, P, pos)
        if starts[0] == 0:
            q1, k1, q2, k2 = (abi.size_array([7] * max(P, T)) for _ in range(4))
            lib.blt_patch_build_group_ids(p, P, T, q1, k1)
            assert oracle.orc_patch_build_group_ids(p, P, T, q2, k2) == 0
            assert list(q1)[:P] == list(q2)[:P] and list(k1)[:T] == list(k2)[:T]
            k = rs.randint(1, 4)
            e1, e2 = abi.size_array([0] * (T * k)), abi.size_array([0] * (T * k))
            lib.blt_patch_expand_group_ids(k1, T, k, e1)
            oracle.orc_patch_expand_group_ids(k2, T, k, e2)
            assert list(e1) == list(e2)
    # the reference's vectors (tests/unit/models/unit_local_decoder.c:94-113)
    p = abi.patch_array([0, 3, 7, 8, 15], [3, 4, 1, 7, 1])
    assert [lib.blt_patch_decoder_latent_at(p, 5, i) for i in range(16)] == [0, 0, 0, 0, 0, 0, 1, 2, 2, 2, 2, 2, 2,
                                                                            2, 3, 3]
    assert lib.blt_patch_decoder_latent_at(p, 5, 100) == 4


def test_row_ranges_describe_the_dense_mask(oracle):
    from oracle import binding
    lib = api.load()
    rs = np.random.RandomState(22)
    claimed = 0
    for trial in range(300):
        nq, nk = rs.randint(1, 30), rs.randint(1, 30)
        cfg = abi.BltMaskConfig()
        cfg.seq_len_q, cfg.seq_len_kv = nq, nk
        cfg.is_causal = bool(rs.randint(2))
        cfg.sliding_window = int(rs.choice([0, 0, 1, 4]))
        cfg.causal_offset = int(rs.choice([0, 0, 2, 11]))
        keep = []
        if rs.randint(2):
            b = abi.size_array(sorted(rs.randint(0, 32, size=rs.randint(1, 4)).tolist()))
            keep.append(b)
            cfg.doc_boundaries, cfg.num_docs = b, len(b) + 1
        sorted_groups = True
        if rs.randint(2):
            sorted_groups = bool(rs.randint(2))
            qa = abi.size_array(rs.randint(0, 4, nq))
            ka = abi.size_array(np.sort(rs.randint(0, 4, nk)) if sorted_groups else rs.randint(0, 4, nk))
            keep += [qa, ka]
            cfg.query_group_ids, cfg.kv_group_ids = qa, ka
            cfg.bidirectional_within_group = bool(rs.randint(2))
        dense = np.empty(nq * nk, dtype=np.float32)
        rc = oracle.orc_build_attention_mask(C.byref(cfg), binding.fptr(dense))
        lo, hi = (C.c_uint32 * nq)(), (C.c_uint32 * nq)()
        ok = lib.blt_mask_config_row_ranges(C.byref(cfg), lo, hi)
        if sorted_groups:
            assert ok == 1
        if not ok:
            continue
        claimed += 1
        allowed = dense.reshape(nq, nk) == 0
        for i in range(nq):
            row = np.zeros(nk, dtype=bool)
            row[lo[i]:hi[i]] = True
            if rc == 4 and not allowed[i].any():
                assert lo[i] == hi[i]
                break          # the dense builder stops at the first dead row
            assert (row == allowed[i]).all(), (trial, i)
    assert claimed > 150


def test_host_arena_and_tensor():
    lib = api.load()
    arena = lib.blt_arena_create(4096, abi.BLT_BACKEND_CPU)
    assert arena.contents.capacity == 4096 and arena.contents.offset == 0
    p1 = lib.blt_arena_alloc(arena, 10, 1)
    p2 = lib.blt_arena_alloc(arena, 4, 64)
    assert p2 % 64 == 0 and p2 > p1 and arena.contents.offset == (p2 - arena.contents.buffer) + 4
    shape = (C.c_size_t * 2)(3, 5)
    t = lib.blt_tensor_create(arena, shape, 2, abi.BLT_DTYPE_FP32)
    assert t.numel == 15 and t.strides[0] == 5 and t.strides[1] == 1 and t.data % 64 == 0
    assert t.backend == abi.BLT_BACKEND_CPU and not t.is_view
    vals = np.arange(15, dtype=np.float32)
    lib.blt_tensor_upload(C.byref(t), vals.ctypes.data, vals.nbytes)
    back = np.zeros(15, dtype=np.float32)
    lib.blt_tensor_download(C.byref(t), back.ctypes.data, back.nbytes)
    assert (back == vals).all()
    lib.blt_arena_reset(arena)
    assert arena.contents.offset == 0
    lib.blt_arena_destroy(arena)


def test_containers_are_host_memory_for_a_device_arena():
    """blt_container_alloc (csrc/core/tensor.c:154-162): arena memory on the CPU backend; for a device arena zeroed,
    64-byte aligned host memory plus a one-byte token of the arena, released with the arena's reset or at the first
    allocation (container or tensor) after a rewind.  The device
    arena here is a hand-made struct whose buffer is never touched, so this runs without a GPU."""
    lib = api.load()
    host = lib.blt_arena_create(4096, abi.BLT_BACKEND_CPU)
    p = lib.blt_container_alloc(host, 100)
    assert p % 64 == 0 and host.contents.buffer <= p < host.contents.buffer + 4096 and host.contents.offset >= 100
    lib.blt_arena_destroy(host)

    dev = abi.BltArena()
    dev.buffer, dev.capacity, dev.offset, dev.backend = 0x10000, 1 << 20, 0, abi.BLT_BACKEND_HIP

    def take(size):
        before = dev.offset
        q = lib.blt_container_alloc(C.byref(dev), size)
        assert q % 64 == 0 and dev.offset == before + 1  # the block's token in the arena
        view = (C.c_ubyte * size).from_address(q)
        assert not any(view)
        for i in range(size):
            view[i] = 0xA5  # host-writable
        return q

    keep = take(100)
    marker = dev.offset
    for _ in range(3):  # a caller that rewinds to its marker every round (csrc/infer/self_speculation.c:359-401)
        take(8)
        dev.offset += 4096
        take(4000)
        take(1)
        dev.offset = marker
    take(64)
    assert all(b == 0xA5 for b in (C.c_ubyte * 100).from_address(keep))  # handed out below the marker: still alive
    lib.blt_arena_reset(C.byref(dev))
    assert dev.offset == 0


FATAL_SNIPPETS = {
    "cpu_backend_rows_gather": """
t = abi.BltTensor(); t.backend = abi.BLT_BACKEND_CPU
pos = (C.c_size_t * 1)(0)
lib.blt_rows_gather(C.byref(t), pos, C.byref(t))
""",
    "rope_position_gather_out_of_range": """
import numpy as np
tab = np.zeros((8, 4), dtype=np.float32)
v = abi.tensor_view(tab.ctypes.data, tab.shape, abi.BLT_BACKEND_CPU)
arena = lib.blt_arena_create(1 << 12, abi.BLT_BACKEND_CPU)
pos = (C.c_size_t * 2)(1, 8)
a, b = abi.BltTensor(), abi.BltTensor()
lib.blt_rope_position_gather(C.byref(v), C.byref(v), pos, 2, C.byref(a), C.byref(b), arena)
""",
    "cpu_backend_attention": """
a = abi.BltAttentionHeadArgs()
lib.blt_attention_head_core(abi.BLT_BACKEND_CPU, C.byref(a))
""",
    "cpu_arena_mask": """
arena = lib.blt_arena_create(1 << 16, abi.BLT_BACKEND_CPU)
cfg = abi.BltMaskConfig(); cfg.seq_len_q = cfg.seq_len_kv = 4
t = abi.BltTensor()
lib.blt_build_attention_mask(C.byref(cfg), C.byref(t), arena)
""",
    "arena_overflow": """
arena = lib.blt_arena_create(64, abi.BLT_BACKEND_CPU)
lib.blt_arena_alloc(arena, 65, 1)
""",
    "cpu_cross_attention": """
import numpy as np
x = np.zeros((2, 4), dtype=np.float32)
t = abi.tensor_view(x.ctypes.data, x.shape, abi.BLT_BACKEND_CPU)
w = abi.BltCrossAttentionWeights(C.pointer(t), C.pointer(t), C.pointer(t), C.pointer(t))
m = abi.BltMaskConfig(); m.seq_len_q = m.seq_len_kv = 2
c = abi.BltCrossAttentionConfig(); c.embed_dim, c.num_heads, c.mask_config = 4, 2, C.pointer(m)
arena = lib.blt_arena_create(1 << 16, abi.BLT_BACKEND_CPU)
lib.blt_cross_attention_forward(C.byref(t), C.byref(t), C.byref(w), C.byref(t), C.byref(c), arena)
""",
    "kv_cache_longer_than_decoder": """
dec = abi.BltLocalDecoder(); dec.config.embed_dim, dec.config.max_seq_len, dec.config.num_layers = 8, 16, 1
arena = lib.blt_arena_create(1 << 20, abi.BLT_BACKEND_CPU)
lib.blt_kv_cache_create(arena, C.byref(dec), 17)
""",
    "kv_cache_truncate_past_capacity": """
dec = abi.BltLocalDecoder(); dec.config.embed_dim, dec.config.max_seq_len, dec.config.num_layers = 8, 16, 1
arena = lib.blt_arena_create(1 << 20, abi.BLT_BACKEND_CPU)
cache = lib.blt_kv_cache_create(arena, C.byref(dec), 16)
assert cache.contents.max_subtokens == 16 and cache.contents.k == 1
lib.blt_kv_cache_truncate(cache, 17, 0)
""",
    "cpu_decode_step": """
import numpy as np
dec = abi.BltLocalDecoder(); dec.config.embed_dim, dec.config.max_seq_len, dec.config.num_layers = 8, 16, 1
arena = lib.blt_arena_create(1 << 20, abi.BLT_BACKEND_CPU)
cache = lib.blt_kv_cache_create(arena, C.byref(dec), 16)
x = np.zeros((1, 8), dtype=np.float32)
t = abi.tensor_view(x.ctypes.data, x.shape, abi.BLT_BACKEND_CPU)
p = abi.patch_array([0], [1])
lib.blt_kv_decode_step(cache, C.byref(t), p, 1, C.byref(t), 0, C.byref(t), arena)
""",
    "bad_patch_tiling": """
p = abi.patch_array([0, 4], [3, 2])
q, k = abi.size_array([0] * 8), abi.size_array([0] * 8)
lib.blt_patch_build_group_ids(p, 2, 6, q, k)
""",
}


@pytest.mark.parametrize("name", list(FATAL_SNIPPETS))
def test_fatal_errors_exit_like_the_reference(name):
    """csrc/core/backend.h:13-31: message on stderr, exit(EXIT_FAILURE); never a silent fallback."""
    code = "import ctypes as C, sys\nsys.path.insert(0, %r)\nfrom fblt_amd import abi, api\nlib = api.load()\n" % ROOT
    code += FATAL_SNIPPETS[name] + "\nprint('SURVIVED')\n"
    p = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert p.returncode == 1, (p.returncode, p.stdout, p.stderr)
    assert "BLT Fatal Error [" in p.stderr and "SURVIVED" not in p.stdout
