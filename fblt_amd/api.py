"""ctypes binding of libfblt_hip.so (the C-ABI declared in include/blt_hip.h).

PyTorch is used by callers only to own device memory; every signature here is
plain pointers and sizes.  There is no fallback: if the library is missing,
`load()` raises.
"""
import ctypes as C
import os

from . import abi

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libfblt_hip.so")

BLT_ATTN_MASK_FROM_HEAD = 0
BLT_ATTN_MASK_CAUSAL = 1
BLT_ATTN_MASK_ROW_RANGE = 2

BLT_KV_STEP_CAUSAL = 0
BLT_KV_STEP_BLOCK = 1


class BltAttentionProblem(C.Structure):
    _fields_ = [
        ("head", abi.BltAttentionHeadArgs),
        ("mask_kind", C.c_uint32),
        ("row_span", C.c_uint32),
        ("causal_offset", C.c_size_t),
        ("window", C.c_size_t),
        ("row_lo", C.c_void_p),
        ("row_hi", C.c_void_p),
    ]


class BltKvAttnCache(C.Structure):
    _fields_ = [
        ("self_k", C.c_void_p),
        ("self_v", C.c_void_p),
        ("self_len", C.c_void_p),
        ("batch", C.c_size_t),
        ("max_seq_len", C.c_size_t),
        ("embed_dim", C.c_size_t),
        ("num_heads", C.c_size_t),
        ("window", C.c_size_t),
    ]


class BltHipKernelTime(C.Structure):
    _fields_ = [("name", C.c_char * 48), ("launches", C.c_uint64), ("total_ms", C.c_double),
                ("min_ms", C.c_double), ("max_ms", C.c_double)]


KV_REFRESH_ARGS = [C.POINTER(abi.BltKvCache), C.POINTER(abi.BltTensor), C.POINTER(abi.BltPatchInfo), C.c_size_t,
                   C.c_size_t, C.POINTER(abi.BltArena)]
KV_STEP_ARGS = [C.POINTER(abi.BltKvCache), C.POINTER(abi.BltTensor), C.POINTER(abi.BltPatchInfo), C.c_size_t,
                C.POINTER(abi.BltTensor), C.c_int, C.POINTER(abi.BltTensor), C.POINTER(abi.BltArena)]

# name -> (restype, argtypes); every symbol include/blt_hip.h declares
SYMBOLS = {
    "blt_attention_head_core_hip": (None, [C.c_int, C.POINTER(abi.BltAttentionHeadArgs)]),
    "blt_build_attention_mask_hip": (None, [C.POINTER(abi.BltMaskConfig), C.POINTER(abi.BltTensor),
                                            C.POINTER(abi.BltArena)]),
    "blt_build_block_diffusion_mask_hip": (None, [C.POINTER(abi.BltBlockDiffusionConfig), C.POINTER(abi.BltTensor),
                                                  C.POINTER(abi.BltArena)]),
    "blt_strided_copy_hip": (None, [C.c_int, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t,
                                    C.c_size_t]),
    "blt_rows_gather_hip": (None, [C.POINTER(abi.BltTensor), abi.c_size_p, C.POINTER(abi.BltTensor)]),
    "blt_softmax_masked_row_inplace_hip": (None, [C.c_int, C.c_void_p, C.c_size_t, C.c_size_t, C.c_bool, C.c_void_p,
                                                  C.c_float]),
    "blt_vec_dot_hip": (C.c_float, [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t]),
    "blt_hip_malloc": (C.c_void_p, [C.c_size_t]),
    "blt_hip_free": (None, [C.c_void_p]),
    "blt_hip_memset": (None, [C.c_void_p, C.c_int, C.c_size_t]),
    "blt_hip_memcpy_h2d": (None, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "blt_hip_memcpy_d2h": (None, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "blt_backend_pass_sync_hip": (None, []),
    "blt_arena_create": (C.POINTER(abi.BltArena), [C.c_size_t, C.c_int]),
    "blt_arena_destroy": (None, [C.POINTER(abi.BltArena)]),
    "blt_arena_reset": (None, [C.POINTER(abi.BltArena)]),
    "blt_arena_alloc": (C.c_void_p, [C.POINTER(abi.BltArena), C.c_size_t, C.c_size_t]),
    "blt_container_alloc": (C.c_void_p, [C.POINTER(abi.BltArena), C.c_size_t]),
    "blt_tensor_create": (abi.BltTensor, [C.POINTER(abi.BltArena), C.POINTER(C.c_size_t), C.c_size_t, C.c_int]),
    "blt_tensor_create_uninit": (abi.BltTensor, [C.POINTER(abi.BltArena), C.POINTER(C.c_size_t), C.c_size_t,
                                                 C.c_int]),
    "blt_tensor_upload": (None, [C.POINTER(abi.BltTensor), C.c_void_p, C.c_size_t]),
    "blt_tensor_download": (None, [C.POINTER(abi.BltTensor), C.c_void_p, C.c_size_t]),
    "blt_backend_pass_sync": (None, [C.c_int]),
    "blt_attention_head_core": (None, [C.c_int, C.POINTER(abi.BltAttentionHeadArgs)]),
    "blt_build_attention_mask": (None, [C.POINTER(abi.BltMaskConfig), C.POINTER(abi.BltTensor),
                                        C.POINTER(abi.BltArena)]),
    "blt_build_block_diffusion_mask": (None, [C.POINTER(abi.BltBlockDiffusionConfig), C.POINTER(abi.BltTensor),
                                              C.POINTER(abi.BltArena)]),
    "blt_strided_copy": (None, [C.c_int, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t]),
    "blt_softmax_masked_row_inplace": (None, [C.c_int, C.c_void_p, C.c_size_t, C.c_size_t, C.c_bool, C.c_void_p,
                                              C.c_float]),
    "blt_vec_dot": (C.c_float, [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t]),
    "blt_rows_gather": (None, [C.POINTER(abi.BltTensor), abi.c_size_p, C.POINTER(abi.BltTensor)]),
    "blt_rope_position_gather": (None, [C.POINTER(abi.BltTensor), C.POINTER(abi.BltTensor), abi.c_size_p, C.c_size_t,
                                        C.POINTER(abi.BltTensor), C.POINTER(abi.BltTensor), C.POINTER(abi.BltArena)]),
    "blt_patch_build_group_ids": (None, [C.POINTER(abi.BltPatchInfo), C.c_size_t, C.c_size_t, abi.c_size_p,
                                         abi.c_size_p]),
    "blt_patch_decoder_latent_at": (C.c_size_t, [C.POINTER(abi.BltPatchInfo), C.c_size_t, C.c_size_t]),
    "blt_patch_expand_group_ids": (None, [abi.c_size_p, C.c_size_t, C.c_size_t, abi.c_size_p]),
    "blt_attention_batch_hip": (None, [C.POINTER(BltAttentionProblem), C.c_size_t]),
    "blt_attention_plan_create_hip": (C.c_void_p, [C.POINTER(BltAttentionProblem), C.c_size_t]),
    "blt_attention_plan_run_hip": (None, [C.c_void_p]),
    "blt_attention_plan_destroy_hip": (None, [C.c_void_p]),
    "blt_attention_plan_kernel_hip": (C.c_char_p, [C.c_void_p]),
    "blt_mask_config_row_ranges": (C.c_int, [C.POINTER(abi.BltMaskConfig), C.POINTER(C.c_uint32),
                                             C.POINTER(C.c_uint32)]),
    "blt_kv_attend_step_hip": (None, [C.POINTER(BltKvAttnCache), C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t,
                                      C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t, C.c_int, C.c_int,
                                      C.c_size_t]),
    "blt_kv_attend_step_noalloc_hip": (None, [C.POINTER(BltKvAttnCache), C.c_void_p, C.c_size_t, C.c_void_p,
                                              C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t,
                                              C.c_int, C.c_int, C.c_size_t]),
    "blt_kv_rope_attend_step_hip": (None, [C.POINTER(BltKvAttnCache), C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t,
                                           C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p,
                                           C.c_size_t, C.c_size_t, C.c_int, C.c_int, C.c_size_t]),
    "blt_kv_attend_step_lens_hip": (None, [C.POINTER(BltKvAttnCache), C.POINTER(C.c_uint32), C.c_void_p, C.c_size_t,
                                           C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p,
                                           C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t, C.c_int]),
    "blt_local_decoder_forward_diffusion_infer_hip": (None, [C.POINTER(abi.BltLocalDecoder), C.POINTER(abi.BltTensor),
                                                             C.POINTER(abi.BltTensor), C.POINTER(abi.BltPatchInfo),
                                                             C.c_size_t, C.POINTER(abi.BltBlockBatch), C.c_int,
                                                             C.POINTER(abi.BltTensor), C.POINTER(abi.BltArena)]),
    "blt_local_decoder_forward_diffusion_infer": (None, [C.POINTER(abi.BltLocalDecoder), C.POINTER(abi.BltTensor),
                                                         C.POINTER(abi.BltTensor), C.POINTER(abi.BltPatchInfo),
                                                         C.c_size_t, C.POINTER(abi.BltBlockBatch), C.c_int,
                                                         C.POINTER(abi.BltTensor), C.POINTER(abi.BltArena)]),
    "blt_transformer_forward": (None, [C.POINTER(abi.BltTensor), C.POINTER(abi.BltTransformerWeights),
                                       C.POINTER(abi.BltTensor), C.POINTER(abi.BltTransformerConfig),
                                       C.POINTER(abi.BltArena)]),
    "blt_transformer_forward_hip": (None, [C.POINTER(abi.BltTensor), C.POINTER(abi.BltTransformerWeights),
                                           C.POINTER(abi.BltTensor), C.POINTER(abi.BltTransformerConfig),
                                           C.POINTER(abi.BltArena)]),
    "blt_indexed_row_accumulate": (None, [C.POINTER(abi.BltTensor), C.POINTER(C.c_uint32), C.POINTER(abi.BltTensor)]),
    "blt_indexed_row_accumulate_hip": (None, [C.POINTER(abi.BltTensor), C.POINTER(C.c_uint32),
                                              C.POINTER(abi.BltTensor)]),
    "blt_scale": (None, [C.POINTER(abi.BltTensor), C.c_float]),
    "blt_scale_hip": (None, [C.POINTER(abi.BltTensor), C.c_float]),
    "blt_patch_pool_forward": (None, [C.POINTER(abi.BltTensor), C.POINTER(abi.BltPatchInfo), C.c_size_t, C.c_int,
                                      C.POINTER(abi.BltTensor)]),
    "blt_patch_pool_forward_hip": (None, [C.POINTER(abi.BltTensor), C.POINTER(abi.BltPatchInfo), C.c_size_t, C.c_int,
                                          C.POINTER(abi.BltTensor)]),
    "blt_local_encoder_forward": (None, [C.POINTER(abi.BltLocalEncoder), C.POINTER(abi.BltTensor),
                                         C.POINTER(abi.BltPatchInfo), C.c_size_t, abi.c_size_p, C.c_size_t,
                                         C.POINTER(abi.BltTensor), C.POINTER(abi.BltTensor), C.POINTER(abi.BltArena)]),
    "blt_local_decoder_forward_ext_hip": (None, [C.POINTER(abi.BltLocalDecoder), C.POINTER(abi.BltTensor),
                                                 C.POINTER(abi.BltTensor), C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t,
                                                 C.c_int, C.POINTER(abi.BltTensor), C.POINTER(abi.BltArena)]),
    "blt_local_decoder_forward_ext": (None, [C.POINTER(abi.BltLocalDecoder), C.POINTER(abi.BltTensor),
                                             C.POINTER(abi.BltTensor), C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p,
                                             C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.POINTER(abi.BltTensor),
                                             C.c_void_p, C.POINTER(abi.BltArena)]),
    "blt_local_encoder_forward_hip": (None, [C.POINTER(abi.BltLocalEncoder), C.POINTER(abi.BltTensor),
                                             C.POINTER(abi.BltPatchInfo), C.c_size_t, abi.c_size_p, C.c_size_t,
                                             C.POINTER(abi.BltTensor), C.POINTER(abi.BltTensor),
                                             C.POINTER(abi.BltArena)]),
    "blt_embedding_lookup": (None, [C.POINTER(abi.BltTensor), C.POINTER(C.c_uint32), C.POINTER(abi.BltTensor)]),
    "blt_embedding_lookup_hip": (None, [C.POINTER(abi.BltTensor), C.POINTER(C.c_uint32), C.POINTER(abi.BltTensor)]),
    "blt_kv_block_step_hip": (None, [C.POINTER(abi.BltKvCache), C.c_size_t, C.POINTER(abi.BltBlockBatch), C.c_int,
                                     C.POINTER(abi.BltTensor), C.POINTER(abi.BltArena)]),
    "blt_matmul_hip": (None, [C.POINTER(abi.BltTensor)] * 3),
    "blt_matmul": (None, [C.POINTER(abi.BltTensor)] * 3),
    "blt_rope_apply_hip": (None, [C.POINTER(abi.BltTensor)] * 4),
    "blt_rope_apply": (None, [C.POINTER(abi.BltTensor)] * 4),
    "blt_rope_apply_packed_hip": (None, [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p,
                                         C.c_void_p]),
    "blt_rope_apply_packed": (None, [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p,
                                     C.c_void_p, C.c_int]),
    "blt_rope_precompute": (None, [C.c_size_t, C.POINTER(abi.BltRopeConfig), C.POINTER(abi.BltTensor),
                                   C.POINTER(abi.BltTensor)]),
    "blt_multihead_attention_hip": (None, [C.POINTER(abi.BltTensor)] * 4 + [C.POINTER(abi.BltAttentionConfig),
                                                                           C.POINTER(abi.BltArena)]),
    "blt_multihead_attention": (None, [C.POINTER(abi.BltTensor)] * 4 + [C.POINTER(abi.BltAttentionConfig),
                                                                       C.POINTER(abi.BltArena)]),
    "blt_rmsnorm_forward_hip": (None, [C.POINTER(abi.BltTensor)] * 3),
    "blt_rmsnorm_forward": (None, [C.POINTER(abi.BltTensor)] * 3),
    "blt_add_hip": (None, [C.POINTER(abi.BltTensor)] * 3),
    "blt_add": (None, [C.POINTER(abi.BltTensor)] * 3),
    "blt_swiglu_forward_hip": (None, [C.POINTER(abi.BltTensor)] * 3),
    "blt_swiglu_forward": (None, [C.POINTER(abi.BltTensor)] * 3),
    "blt_kv_decode_layer_hip": (None, [C.POINTER(BltKvAttnCache), C.POINTER(abi.BltTransformerWeights), C.c_void_p,
                                       C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_int, C.c_int,
                                       C.c_size_t, C.POINTER(abi.BltArena)]),
    "blt_cross_attention_forward_hip": (None, [C.POINTER(abi.BltTensor), C.POINTER(abi.BltTensor),
                                               C.POINTER(abi.BltCrossAttentionWeights), C.POINTER(abi.BltTensor),
                                               C.POINTER(abi.BltCrossAttentionConfig), C.POINTER(abi.BltArena)]),
    "blt_cross_attention_forward": (None, [C.POINTER(abi.BltTensor), C.POINTER(abi.BltTensor),
                                           C.POINTER(abi.BltCrossAttentionWeights), C.POINTER(abi.BltTensor),
                                           C.POINTER(abi.BltCrossAttentionConfig), C.POINTER(abi.BltArena)]),
    "blt_kv_cache_create": (C.POINTER(abi.BltKvCache), [C.POINTER(abi.BltArena), C.POINTER(abi.BltLocalDecoder),
                                                        C.c_size_t]),
    "blt_kv_cache_create_batched": (C.POINTER(abi.BltKvCache), [C.POINTER(abi.BltArena),
                                                                C.POINTER(abi.BltLocalDecoder), C.c_size_t,
                                                                C.c_size_t]),
    "blt_kv_cache_destroy": (None, [C.POINTER(abi.BltKvCache)]),
    "blt_kv_cache_reset": (None, [C.POINTER(abi.BltKvCache)]),
    "blt_kv_cache_truncate": (None, [C.POINTER(abi.BltKvCache), C.c_size_t, C.c_size_t]),
    "blt_kv_cache_common_patches": (C.c_size_t, [C.POINTER(abi.BltKvCache), C.POINTER(abi.BltPatchInfo), C.c_size_t]),
    "blt_local_cross_attn_fires": (C.c_bool, [C.c_int, C.c_bool, C.c_size_t, C.c_size_t]),
    "blt_kv_cache_refresh_cross": (None, KV_REFRESH_ARGS),
    "blt_kv_cache_refresh_cross_hip": (None, KV_REFRESH_ARGS),
    "blt_kv_cache_refresh_cross_seq_hip": (None, [KV_REFRESH_ARGS[0], C.c_size_t] + KV_REFRESH_ARGS[1:]),
    "blt_kv_decode_step": (None, KV_STEP_ARGS),
    "blt_kv_decode_step_hip": (None, KV_STEP_ARGS),
    "blt_kv_decode_step_batched_hip": (None, [C.POINTER(abi.BltKvCache), abi.c_size_p,
                                              C.POINTER(C.POINTER(abi.BltPatchInfo)), abi.c_size_p,
                                              C.POINTER(C.c_int), C.POINTER(abi.BltTensor), C.POINTER(abi.BltTensor),
                                              C.POINTER(abi.BltArena)]),
    "blt_hip_set_stream": (None, [C.c_void_p]),
    "blt_hip_get_stream": (C.c_void_p, []),
    "blt_hip_capture_begin": (None, []),
    "blt_hip_capture_end": (C.c_void_p, []),
    "blt_hip_graph_launch": (None, [C.c_void_p]),
    "blt_hip_graph_destroy": (None, [C.c_void_p]),
    "blt_hip_profile_begin": (None, []),
    "blt_hip_profile_end": (C.c_size_t, [C.POINTER(BltHipKernelTime), C.c_size_t]),
    "blt_hip_profile_end_list": (C.c_size_t, [C.POINTER(C.c_float), C.c_size_t]),
    "blt_hip_build_info": (C.c_char_p, []),
}

_lib = None


def load():
    """The shared library with typed entry points; raises when it was never built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("%s is missing: run `python -m fblt_amd.build` (there is no fallback path)" % LIB_PATH)
    # One HIP runtime per process: PyTorch-ROCm ships its own libamdhip64 with the
    # same SONAME the library needs.  Whoever is loaded first wins, and a process
    # that ends up with two runtimes loses its device.  The Python callers here use
    # torch for device memory, so let torch bring in its runtime first.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SYMBOLS.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def head_args(q_ptr, k_ptr, v_ptr, out_ptr, nq, nk, hd, scale, q_stride, k_stride, v_stride, out_stride, out_col,
              weights=None, scratch=None, lse=None, mask=None, causal=False):
    """blt_attention_head_args over raw addresses (ints)."""
    a = abi.BltAttentionHeadArgs()
    a.q, a.k, a.v = q_ptr, k_ptr, v_ptr
    a.q_stride, a.k_stride, a.v_stride = q_stride, k_stride, v_stride
    a.combined = out_ptr
    a.combined_stride, a.combined_col_offset = out_stride, out_col
    a.weights_out = weights
    a.scores_scratch = scratch
    a.lse_out = lse
    a.mask = mask
    a.nq, a.nk, a.head_dim = nq, nk, hd
    a.is_causal = bool(causal)
    a.scale = float(scale)
    return a


def problem(head, kind=BLT_ATTN_MASK_FROM_HEAD, causal_offset=0, window=0, row_lo=None, row_hi=None, row_span=0):
    p = BltAttentionProblem()
    p.head = head
    p.mask_kind = kind
    p.row_span = row_span
    p.causal_offset = causal_offset
    p.window = window
    p.row_lo = row_lo
    p.row_hi = row_hi
    return p


def problem_array(problems):
    arr = (BltAttentionProblem * max(len(problems), 1))()
    for i, p in enumerate(problems):
        arr[i] = p
    return arr


def profile_end_list(capacity=1 << 16):
    """Close the open profile: the duration of every launch since `begin`, in milliseconds, in issue order."""
    buf = (C.c_float * capacity)()
    n = load().blt_hip_profile_end_list(buf, capacity)
    return [buf[i] for i in range(min(n, capacity))]


def profile_end():
    """Close the open profile: {kernel tag: (launches, total_ms, min_ms, max_ms)}."""
    rows = (BltHipKernelTime * 16)()
    n = load().blt_hip_profile_end(rows, 16)
    return {rows[i].name.decode(): (int(rows[i].launches), rows[i].total_ms, rows[i].min_ms, rows[i].max_ms)
            for i in range(min(n, 16))}
