"""TEST INFRASTRUCTURE -- ctypes loaders for the CPU checker.

Only tests/, the smoke check and the benchmark's cpu_baseline leg import this.
`load_oracle()` loads oracle/liboracle.so (our restatement, built by
`make -C oracle`); `load_ref()` loads oracle/_ref/libblt_ref.so (the reference's
own core + CPU ops compiled from its sources, built by `make -C oracle ref`
where those sources exist) or returns None.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from fblt_amd import abi

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "liboracle.so")
REF_SO = os.path.join(HERE, "_ref", "libblt_ref.so")

_fp = C.POINTER(C.c_float)
_sp = C.POINTER(C.c_size_t)


def build(ref=True):
    """Compile the checker (and the reference build when its sources exist)."""
    subprocess.check_call(["make", "-s", "-B", "-C", HERE, "all"])
    if ref and os.path.isdir(os.environ.get("REF_ROOT", "/root/reference")):
        subprocess.check_call(["make", "-s", "-B", "-C", HERE, "ref"])
        if os.path.exists(os.path.join(HERE, "..", "fblt_amd", "lib", "libfblt_hip.so")):
            subprocess.check_call(["make", "-s", "-C", HERE, "callers", "stack_callers", "model_callers", "model_driver"])


def load_oracle():
    if not os.path.exists(ORACLE_SO):
        build(ref=False)
    lib = C.CDLL(ORACLE_SO)
    A = abi.BltAttentionHeadArgs
    lib.orc_vec_dot.restype = C.c_float
    lib.orc_vec_dot.argtypes = [_fp, _fp, C.c_size_t]
    lib.orc_softmax_masked_row_inplace.restype = None
    lib.orc_softmax_masked_row_inplace.argtypes = [_fp, C.c_size_t, C.c_size_t, C.c_bool, _fp, C.c_float]
    lib.orc_strided_copy.restype = None
    lib.orc_strided_copy.argtypes = [_fp, C.c_size_t, _fp, C.c_size_t, C.c_size_t, C.c_size_t]
    lib.orc_attention_head_core.restype = C.c_int
    lib.orc_attention_head_core.argtypes = [C.POINTER(A)]
    lib.orc_attention_head_core_many.restype = C.c_int
    lib.orc_attention_head_core_many.argtypes = [C.POINTER(A), C.c_size_t]
    lib.orc_build_attention_mask.restype = C.c_int
    lib.orc_build_attention_mask.argtypes = [C.POINTER(abi.BltMaskConfig), _fp]
    lib.orc_build_block_diffusion_mask.restype = C.c_int
    lib.orc_build_block_diffusion_mask.argtypes = [C.POINTER(abi.BltBlockDiffusionConfig), _fp]
    lib.orc_patch_build_group_ids.restype = C.c_int
    lib.orc_patch_build_group_ids.argtypes = [C.POINTER(abi.BltPatchInfo), C.c_size_t, C.c_size_t, _sp, _sp]
    lib.orc_patch_decoder_latent_at.restype = C.c_size_t
    lib.orc_patch_decoder_latent_at.argtypes = [C.POINTER(abi.BltPatchInfo), C.c_size_t, C.c_size_t]
    lib.orc_patch_expand_group_ids.restype = None
    lib.orc_patch_expand_group_ids.argtypes = [_sp, C.c_size_t, C.c_size_t, _sp]
    lib.orc_kv_row.restype = C.c_size_t
    lib.orc_kv_row.argtypes = [C.c_size_t] * 3
    lib.orc_kv_slot.restype = C.c_size_t
    lib.orc_kv_slot.argtypes = [C.c_size_t] * 7
    lib.orc_kv_self_mask.restype = None
    lib.orc_kv_self_mask.argtypes = [_fp, C.c_size_t, C.c_size_t, C.c_size_t]
    lib.orc_kv_attend_step.restype = C.c_int
    lib.orc_kv_attend_step.argtypes = [_fp, _fp, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t,
                                       C.c_size_t, C.c_size_t, _fp, _fp, _fp, _fp]
    lib.orc_rope_precompute.restype = C.c_int
    lib.orc_rope_precompute.argtypes = [C.c_size_t, C.c_float, C.c_size_t, _fp, _fp]
    lib.orc_rope_apply.restype = None
    lib.orc_rope_apply.argtypes = [_fp, C.c_size_t, C.c_size_t, C.c_size_t, _fp, _fp, _fp]
    lib.orc_rope_position_gather.restype = C.c_int
    lib.orc_rope_position_gather.argtypes = [_fp, _fp, C.c_size_t, C.c_size_t, _sp, C.c_size_t, _fp, _fp]
    lib.orc_matmul.restype = None
    lib.orc_matmul.argtypes = [_fp, _fp, _fp, C.c_size_t, C.c_size_t, C.c_size_t]
    lib.orc_rope_apply_packed.restype = None
    lib.orc_rope_apply_packed.argtypes = [_fp, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, _fp, _fp]
    lib.orc_multihead_attention.restype = C.c_int
    lib.orc_multihead_attention.argtypes = [_fp, _fp, _fp, _fp, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int, C.c_int,
                                            C.c_float, _fp, _fp, C.POINTER(abi.BltMaskConfig)]
    _u8 = C.POINTER(C.c_uint8)
    _u32 = C.POINTER(C.c_uint32)
    lib.orc_indexed_row_accumulate.restype = C.c_int
    lib.orc_indexed_row_accumulate.argtypes = [_fp, C.c_size_t, _u32, _fp, C.c_size_t, C.c_size_t]
    lib.orc_scale.restype = None
    lib.orc_scale.argtypes = [_fp, C.c_size_t, C.c_float]
    lib.orc_patch_pool_forward.restype = C.c_int
    lib.orc_patch_pool_forward.argtypes = [_fp, C.c_size_t, C.c_size_t, C.POINTER(abi.BltPatchInfo), C.c_size_t, C.c_int,
                                           _fp]
    lib.orc_ngram_indices.restype = C.c_int
    lib.orc_ngram_indices.argtypes = [_u8, C.c_size_t, C.c_size_t, C.c_uint64, C.c_uint64, _u32]
    lib.orc_embed_bytes.restype = C.c_int
    lib.orc_embed_bytes.argtypes = [_fp, C.POINTER(abi.BltHashNgramConfig), C.POINTER(abi.BltHashNgramWeights), _u8,
                                    C.c_size_t, _fp]
    lib.orc_local_encoder_forward.restype = C.c_int
    lib.orc_local_encoder_forward.argtypes = [C.POINTER(abi.BltLocalEncoder), _u8, C.c_size_t,
                                              C.POINTER(abi.BltPatchInfo), C.c_size_t, abi.c_size_p, C.c_size_t, _fp, _fp]
    lib.orc_local_decoder_forward.restype = C.c_int
    lib.orc_local_decoder_forward.argtypes = [C.POINTER(abi.BltLocalDecoder), _fp, C.c_size_t, _fp,
                                              C.POINTER(abi.BltPatchInfo), C.c_size_t, abi.c_size_p, C.c_size_t, C.c_int,
                                              _fp]
    lib.orc_transformer_forward.restype = C.c_int
    lib.orc_transformer_forward.argtypes = [_fp] * 9 + [C.c_size_t] * 4 + [C.c_int, C.c_int, C.c_float, _fp, _fp,
                                                                         C.POINTER(abi.BltMaskConfig)]
    lib.orc_rmsnorm_forward.restype = None
    lib.orc_rmsnorm_forward.argtypes = [_fp, _fp, _fp, C.c_size_t, C.c_size_t]
    lib.orc_add.restype = None
    lib.orc_add.argtypes = [_fp, _fp, _fp, C.c_size_t]
    lib.orc_swiglu_forward.restype = None
    lib.orc_swiglu_forward.argtypes = [_fp, _fp, _fp, C.c_size_t]
    lib.orc_kv_decode_layer.restype = C.c_int
    lib.orc_kv_decode_layer.argtypes = ([_fp, _fp] + [C.c_size_t] * 7 + [_fp] * 7 + [C.c_size_t, _fp, _fp, C.c_size_t,
                                                                                _fp, _fp])
    lib.orc_cross_attention_forward.restype = C.c_int
    lib.orc_cross_attention_forward.argtypes = [_fp] * 7 + [C.c_size_t] * 4 + [C.POINTER(abi.BltMaskConfig)]
    lib.orc_local_cross_attn_fires.restype = C.c_int
    lib.orc_local_cross_attn_fires.argtypes = [C.c_int, C.c_int, C.c_size_t, C.c_size_t]
    lib.orc_kv_cache_refresh_cross.restype = C.c_int
    lib.orc_kv_cache_refresh_cross.argtypes = [C.POINTER(abi.BltKvCache), C.c_size_t, _fp, C.c_size_t, C.c_size_t]
    lib.orc_kv_cross_block.restype = C.c_int
    lib.orc_kv_cross_block.argtypes = [_fp, _fp] + [C.c_size_t] * 6 + [abi.c_size_p, C.c_size_t] + [_fp] * 5
    lib.orc_kv_decode_step.restype = C.c_int
    lib.orc_kv_decode_step.argtypes = [C.POINTER(abi.BltKvCache), C.c_size_t, C.c_size_t,
                                       C.POINTER(abi.BltPatchInfo), C.c_size_t, _fp, C.c_size_t, C.c_int, _fp]
    lib.orc_local_decoder_forward_diffusion_infer.restype = C.c_int
    lib.orc_local_decoder_forward_diffusion_infer.argtypes = [C.POINTER(abi.BltLocalDecoder), _fp, _fp,
                                                              C.POINTER(abi.BltPatchInfo), C.c_size_t,
                                                              C.POINTER(abi.BltBlockBatch), C.c_int, _fp]
    lib.orc_kv_block_step.restype = C.c_int
    lib.orc_kv_block_step.argtypes = [C.POINTER(abi.BltKvCache), C.c_size_t, C.c_size_t, C.c_size_t,
                                      C.POINTER(abi.BltBlockBatch), C.c_int, _fp]
    lib.orc_kv_rope_attend_step.restype = C.c_int
    lib.orc_kv_rope_attend_step.argtypes = [_fp, _fp] + [C.c_size_t] * 7 + [_fp, C.c_size_t, _fp, C.c_size_t, _fp,
                                                                           C.c_size_t, _fp, _fp, C.c_size_t, _fp]
    return lib


class BltRopeConfig(C.Structure):
    """blt_rope_config, csrc/ops/rope.h:10-13"""
    _fields_ = [("theta", C.c_float), ("head_dim", C.c_size_t)]


def ref_rope_apply(ref, x, cos_rows, sin_rows):
    """x [rows, heads, hd] through the reference's blt_rope_apply with cos/sin rows [rows, hd/2]."""
    rows, heads, hd = x.shape
    x = np.ascontiguousarray(x, dtype=np.float32)
    cos_rows = np.ascontiguousarray(cos_rows, dtype=np.float32)
    sin_rows = np.ascontiguousarray(sin_rows, dtype=np.float32)
    out = np.empty_like(x)
    tx, tc, ts, to = abi.BltTensor(), abi.BltTensor(), abi.BltTensor(), abi.BltTensor()
    ref.blt_tensor_view_3d(C.byref(tx), x.ctypes.data, rows, heads, hd, abi.BLT_BACKEND_CPU)
    ref.blt_tensor_view_3d(C.byref(to), out.ctypes.data, rows, heads, hd, abi.BLT_BACKEND_CPU)
    ref.blt_tensor_view_2d(C.byref(tc), cos_rows.ctypes.data, rows, hd // 2, abi.BLT_BACKEND_CPU)
    ref.blt_tensor_view_2d(C.byref(ts), sin_rows.ctypes.data, rows, hd // 2, abi.BLT_BACKEND_CPU)
    ref.blt_rope_apply(C.byref(tx), C.byref(tc), C.byref(ts), C.byref(to))
    return out


def load_ref():
    """The reference's own CPU ops, or None where they were never built."""
    if not os.path.exists(REF_SO):
        return None
    lib = C.CDLL(REF_SO)
    A = abi.BltAttentionHeadArgs
    lib.blt_attention_head_core.restype = None
    lib.blt_attention_head_core.argtypes = [C.c_int, C.POINTER(A)]
    lib.blt_softmax_masked_row_inplace.restype = None
    lib.blt_softmax_masked_row_inplace.argtypes = [C.c_int, _fp, C.c_size_t, C.c_size_t, C.c_bool, _fp, C.c_float]
    lib.blt_vec_dot.restype = C.c_float
    lib.blt_vec_dot.argtypes = [C.c_int, _fp, _fp, C.c_size_t]
    lib.blt_strided_copy.restype = None
    lib.blt_strided_copy.argtypes = [C.c_int, _fp, C.c_size_t, _fp, C.c_size_t, C.c_size_t, C.c_size_t]
    lib.blt_arena_create.restype = C.POINTER(abi.BltArena)
    lib.blt_arena_create.argtypes = [C.c_size_t, C.c_int]
    lib.blt_arena_destroy.restype = None
    lib.blt_arena_destroy.argtypes = [C.POINTER(abi.BltArena)]
    lib.blt_build_attention_mask.restype = None
    lib.blt_build_attention_mask.argtypes = [C.POINTER(abi.BltMaskConfig), C.POINTER(abi.BltTensor),
                                             C.POINTER(abi.BltArena)]
    T = C.POINTER(abi.BltTensor)
    lib.blt_tensor_view_2d.restype = None
    lib.blt_tensor_view_2d.argtypes = [T, C.c_void_p, C.c_size_t, C.c_size_t, C.c_int]
    lib.blt_tensor_view_3d.restype = None
    lib.blt_tensor_view_3d.argtypes = [T, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int]
    lib.blt_rope_precompute.restype = None
    lib.blt_rope_precompute.argtypes = [C.c_size_t, C.POINTER(BltRopeConfig), T, T]
    lib.blt_rope_apply.restype = None
    lib.blt_rope_apply.argtypes = [T, T, T, T]
    lib.blt_matmul.restype = None
    lib.blt_matmul.argtypes = [T, T, T]
    for name in ("blt_add", "blt_swiglu_forward", "blt_rmsnorm_forward"):
        getattr(lib, name).restype = None
        getattr(lib, name).argtypes = [T, T, T]
    lib.blt_rope_apply_packed.restype = None
    lib.blt_rope_apply_packed.argtypes = [_fp, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, _fp, _fp, C.c_int]
    lib.blt_multihead_attention.restype = None
    lib.blt_multihead_attention.argtypes = [T, T, T, T, C.POINTER(abi.BltAttentionConfig), C.POINTER(abi.BltArena)]
    lib.blt_transformer_forward.restype = None
    lib.blt_transformer_forward.argtypes = [T, C.POINTER(abi.BltTransformerWeights), T,
                                            C.POINTER(abi.BltTransformerConfig), C.POINTER(abi.BltArena)]
    lib.blt_cross_attention_forward.restype = None
    lib.blt_cross_attention_forward.argtypes = [T, T, C.POINTER(abi.BltCrossAttentionWeights), T,
                                                C.POINTER(abi.BltCrossAttentionConfig), C.POINTER(abi.BltArena)]
    lib.blt_kv_cache_create_batched.restype = C.POINTER(abi.BltKvCache)
    lib.blt_kv_cache_create_batched.argtypes = [C.POINTER(abi.BltArena), C.POINTER(abi.BltLocalDecoder), C.c_size_t,
                                                C.c_size_t]
    lib.blt_kv_cache_destroy.restype = None
    lib.blt_kv_cache_destroy.argtypes = [C.POINTER(abi.BltKvCache)]
    lib.blt_kv_cache_truncate.restype = None
    lib.blt_kv_cache_truncate.argtypes = [C.POINTER(abi.BltKvCache), C.c_size_t, C.c_size_t]
    lib.blt_kv_cache_common_patches.restype = C.c_size_t
    lib.blt_kv_cache_common_patches.argtypes = [C.POINTER(abi.BltKvCache), C.POINTER(abi.BltPatchInfo), C.c_size_t]
    lib.blt_kv_cache_refresh_cross.restype = None
    lib.blt_kv_cache_refresh_cross.argtypes = [C.POINTER(abi.BltKvCache), T, C.POINTER(abi.BltPatchInfo), C.c_size_t,
                                               C.c_size_t, C.POINTER(abi.BltArena)]
    lib.blt_kv_decode_step.restype = None
    lib.blt_kv_decode_step.argtypes = [C.POINTER(abi.BltKvCache), T, C.POINTER(abi.BltPatchInfo), C.c_size_t, T,
                                       C.c_int, T, C.POINTER(abi.BltArena)]
    lib.blt_local_cross_attn_fires.restype = C.c_bool
    lib.blt_local_cross_attn_fires.argtypes = [C.c_int, C.c_bool, C.c_size_t, C.c_size_t]
    # blt_local_decoder_forward_ext(model, byte_hidden_in, patch_in, patches, num_patches, bytes_in, targets,
    #                               doc_boundaries, num_docs, d0_opts, trailing_closed, logits_out, loss_out, arena)
    lib.blt_local_decoder_forward_ext.restype = None
    lib.blt_local_decoder_forward_ext.argtypes = [C.POINTER(abi.BltLocalDecoder), T, T, C.POINTER(abi.BltPatchInfo),
                                                  C.c_size_t, T, T, abi.c_size_p, C.c_size_t, C.c_void_p, C.c_int, T,
                                                  T, C.POINTER(abi.BltArena)]
    if hasattr(lib, "blt_local_decoder_forward_diffusion_infer"):   # csrc/models/block_diffusion.h:131-134
        lib.blt_local_decoder_forward_diffusion_infer.restype = None
        lib.blt_local_decoder_forward_diffusion_infer.argtypes = [C.POINTER(abi.BltLocalDecoder), T, T,
                                                                  C.POINTER(abi.BltPatchInfo), C.c_size_t,
                                                                  C.POINTER(abi.BltBlockBatch), C.c_int, T,
                                                                  C.POINTER(abi.BltArena)]
    if hasattr(lib, "blt_local_encoder_forward"):   # csrc/models/local_encoder.h:71-73
        _encoder_entry(lib)
    if hasattr(lib, "blt_model_encode"):
        _model_entry(lib)
        lib.blt_indexed_row_accumulate.restype = None
        lib.blt_indexed_row_accumulate.argtypes = [T, C.POINTER(C.c_uint32), T]
        lib.blt_scale.restype = None
        lib.blt_scale.argtypes = [T, C.c_float]
        lib.blt_patch_pool_forward.restype = None
        lib.blt_patch_pool_forward.argtypes = [T, C.POINTER(abi.BltPatchInfo), C.c_size_t, C.c_int, T]
    lib.blt_build_block_diffusion_mask.restype = None
    lib.blt_build_block_diffusion_mask.argtypes = [C.POINTER(abi.BltBlockDiffusionConfig),
                                                   C.POINTER(abi.BltTensor), C.POINTER(abi.BltArena)]
    lib.blt_patch_build_group_ids.restype = None
    lib.blt_patch_build_group_ids.argtypes = [C.POINTER(abi.BltPatchInfo), C.c_size_t, C.c_size_t, _sp, _sp]
    lib.blt_patch_decoder_latent_at.restype = C.c_size_t
    lib.blt_patch_decoder_latent_at.argtypes = [C.POINTER(abi.BltPatchInfo), C.c_size_t, C.c_size_t]
    lib.blt_patch_expand_group_ids.restype = None
    lib.blt_patch_expand_group_ids.argtypes = [_sp, C.c_size_t, C.c_size_t, _sp]
    return lib


def _encoder_entry(lib):
    T = C.POINTER(abi.BltTensor)
    lib.blt_local_encoder_forward.restype = None
    lib.blt_local_encoder_forward.argtypes = [C.POINTER(abi.BltLocalEncoder), T, C.POINTER(abi.BltPatchInfo), C.c_size_t,
                                              abi.c_size_p, C.c_size_t, T, T, C.POINTER(abi.BltArena)]


CALLERS_SO = os.path.join(HERE, "_ref", "libblt_ref_callers.so")


STACK_CALLERS_SO = os.path.join(HERE, "_ref", "libblt_ref_stack_callers.so")


class BltGlobalTransformerConfig(C.Structure):
    """csrc/models/global_transformer.h:15-24"""
    _fields_ = [("embed_dim", C.c_size_t), ("num_layers", C.c_size_t), ("hidden_dim", C.c_size_t),
                ("num_heads", C.c_size_t), ("rope_theta", C.c_float), ("max_seq_len", C.c_size_t),
                ("use_bf16", C.c_bool), ("use_fp8", C.c_bool)]


class BltTransformerStack(C.Structure):
    """csrc/models/transformer_stack.h:14-33"""
    _fields_ = [("layer_config", abi.BltTransformerConfig), ("layer_storage", C.c_void_p),
                ("layer_weights", C.POINTER(abi.BltTransformerWeights)), ("layer_weights_bf16", C.c_void_p),
                ("layer_weights_fp8", C.c_void_p), ("rope_cos_cache", abi.BltTensor), ("rope_sin_cache", abi.BltTensor),
                ("num_layers", C.c_size_t), ("embed_dim", C.c_size_t), ("hidden_dim", C.c_size_t),
                ("num_heads", C.c_size_t), ("head_dim", C.c_size_t), ("max_seq_len", C.c_size_t),
                ("use_bf16", C.c_int), ("use_fp8", C.c_int)]


class BltGlobalTransformer(C.Structure):
    """csrc/models/global_transformer.h:26-29"""
    _fields_ = [("config", BltGlobalTransformerConfig), ("stack", BltTransformerStack)]


class BltModelConfig(C.Structure):
    """csrc/models/model.h:16-20"""
    _fields_ = [("encoder_config", abi.BltLocalEncoderConfig), ("global_config", BltGlobalTransformerConfig),
                ("decoder_config", abi.BltLocalDecoderConfig)]


class BltModel(C.Structure):
    """csrc/models/model.h:22-27"""
    _fields_ = [("config", BltModelConfig), ("encoder", C.POINTER(abi.BltLocalEncoder)),
                ("global_", C.POINTER(BltGlobalTransformer)), ("decoder", C.POINTER(abi.BltLocalDecoder))]


class BltModelEncOut(C.Structure):
    """csrc/models/model.h:42-47"""
    _fields_ = [("patch_out", abi.BltTensor), ("global_out", abi.BltTensor), ("byte_hidden_out", abi.BltTensor),
                ("patch_doc_boundaries", abi.c_size_p)]


def _model_entry(lib):
    """The two stages of the model's inference forward, blt_model_encode and blt_model_decode
    (csrc/models/model.c:68-131; blt_model_forward itself always asks for the loss), and the patch
    transformer's constructor."""
    T, A = C.POINTER(abi.BltTensor), C.POINTER(abi.BltArena)
    lib.blt_global_transformer_create.restype = C.POINTER(BltGlobalTransformer)
    lib.blt_global_transformer_create.argtypes = [A, C.POINTER(BltGlobalTransformerConfig)]
    lib.blt_model_encode.restype = None
    lib.blt_model_encode.argtypes = [C.POINTER(BltModel), T, C.POINTER(abi.BltPatchInfo), C.c_size_t, abi.c_size_p,
                                     C.c_size_t, C.POINTER(BltModelEncOut), A]
    lib.blt_model_decode.restype = None
    lib.blt_model_decode.argtypes = [C.POINTER(BltModel), C.POINTER(BltModelEncOut), C.POINTER(abi.BltPatchInfo),
                                     C.c_size_t, T, T, abi.c_size_p, C.c_size_t, C.c_void_p, T, T, A]


def load_ref_stack_callers():
    """The reference's transformer_stack.c and global_transformer.c, compiled unmodified and linked
    against the HIP library without the reference's transformer.c, so that every layer of the
    patch transformer runs through the library's blt_transformer_forward (`make -C oracle
    stack_callers`); None where that was never built."""
    if not os.path.exists(STACK_CALLERS_SO) or not os.path.exists(REF_SO):
        return None
    load_ref()
    lib = C.CDLL(STACK_CALLERS_SO)
    T, A = C.POINTER(abi.BltTensor), C.POINTER(abi.BltArena)
    lib.blt_global_transformer_create.restype = C.POINTER(BltGlobalTransformer)
    lib.blt_global_transformer_create.argtypes = [A, C.POINTER(BltGlobalTransformerConfig)]
    lib.blt_global_transformer_forward.restype = None
    lib.blt_global_transformer_forward.argtypes = [C.POINTER(BltGlobalTransformer), T, abi.c_size_p, C.c_size_t, T, A]
    if hasattr(lib, "blt_local_encoder_forward"):
        _encoder_entry(lib)
    if hasattr(lib, "blt_model_encode"):
        _model_entry(lib)
    return lib


MODEL_CALLERS_SO = os.path.join(HERE, "_ref", "libblt_ref_model_callers.so")


def load_ref_model_callers():
    """The reference's whole-model driver, patch transformer and local decoder, compiled unmodified
    and linked against the HIP library WITHOUT the reference's encoder sources, so that
    blt_model_encode runs the library's own blt_local_encoder_forward (`make -C oracle
    model_callers`); None where that was never built."""
    if not os.path.exists(MODEL_CALLERS_SO) or not os.path.exists(REF_SO):
        return None
    load_ref()
    lib = C.CDLL(MODEL_CALLERS_SO)
    _model_entry(lib)
    return lib


MODEL_DRIVER_SO = os.path.join(HERE, "_ref", "libblt_ref_model_driver.so")


def load_ref_model_driver():
    """The reference's whole-model driver and patch transformer alone, compiled unmodified and
    linked against the HIP library without the reference's encoder and decoder sources: both local
    models run through the library's own entries (`make -C oracle model_driver`); None where that
    was never built."""
    if not os.path.exists(MODEL_DRIVER_SO) or not os.path.exists(REF_SO):
        return None
    load_ref()
    lib = C.CDLL(MODEL_DRIVER_SO)
    _model_entry(lib)
    return lib


def load_ref_callers():
    """The reference's attention blocks and KV-cache step, compiled unmodified and linked against
    the HIP library so that every tensor op they call lands there (`make -C oracle callers`); None
    where that was never built.  Import torch and load the HIP library before calling this (the
    dependency must resolve to the copy that is already loaded)."""
    if not os.path.exists(CALLERS_SO) or not os.path.exists(REF_SO):
        return None
    load_ref()          # its own scope first: its internal calls must keep resolving to itself
    lib = C.CDLL(CALLERS_SO)
    T = C.POINTER(abi.BltTensor)
    K = C.POINTER(abi.BltKvCache)
    A = C.POINTER(abi.BltArena)
    P = C.POINTER(abi.BltPatchInfo)
    lib.blt_multihead_attention.restype = None
    lib.blt_multihead_attention.argtypes = [T, T, T, T, C.POINTER(abi.BltAttentionConfig), A]
    lib.blt_cross_attention_forward.restype = None
    lib.blt_cross_attention_forward.argtypes = [T, T, C.POINTER(abi.BltCrossAttentionWeights), T,
                                                C.POINTER(abi.BltCrossAttentionConfig), A]
    lib.blt_transformer_forward.restype = None
    lib.blt_transformer_forward.argtypes = [T, C.POINTER(abi.BltTransformerWeights), T,
                                            C.POINTER(abi.BltTransformerConfig), A]
    lib.blt_kv_cache_create.restype = K
    lib.blt_kv_cache_create.argtypes = [A, C.POINTER(abi.BltLocalDecoder), C.c_size_t]
    for name in ("blt_kv_cache_destroy", "blt_kv_cache_reset"):
        getattr(lib, name).restype = None
        getattr(lib, name).argtypes = [K]
    lib.blt_kv_cache_truncate.restype = None
    lib.blt_kv_cache_truncate.argtypes = [K, C.c_size_t, C.c_size_t]
    lib.blt_kv_cache_common_patches.restype = C.c_size_t
    lib.blt_kv_cache_common_patches.argtypes = [K, P, C.c_size_t]
    lib.blt_kv_cache_refresh_cross.restype = None
    lib.blt_kv_cache_refresh_cross.argtypes = [K, T, P, C.c_size_t, C.c_size_t, A]
    lib.blt_kv_decode_step.restype = None
    lib.blt_kv_decode_step.argtypes = [K, T, P, C.c_size_t, T, C.c_int, T, A]
    if hasattr(lib, "blt_local_decoder_forward_diffusion_infer"):
        lib.blt_local_decoder_forward_diffusion_infer.restype = None
        lib.blt_local_decoder_forward_diffusion_infer.argtypes = [C.POINTER(abi.BltLocalDecoder), T, T, P, C.c_size_t,
                                                                  C.POINTER(abi.BltBlockBatch), C.c_int, T, A]
    return lib


def fptr(a):
    """float* into a C-contiguous float32 numpy array (or NULL for None)."""
    if a is None:
        return None
    assert a.dtype.name == "float32" and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_fp)


def head_args(q, k, v, combined, nq, nk, hd, scale, q_stride, k_stride, v_stride, c_stride, c_off,
              q_off=0, k_off=0, v_off=0, weights=None, scratch=None, lse=None, mask=None, causal=False):
    """blt_attention_head_args over HOST numpy buffers (element offsets)."""
    a = abi.BltAttentionHeadArgs()
    a.q = q.ctypes.data + 4 * q_off
    a.k = k.ctypes.data + 4 * k_off
    a.v = v.ctypes.data + 4 * v_off
    a.q_stride, a.k_stride, a.v_stride = q_stride, k_stride, v_stride
    a.combined = combined.ctypes.data
    a.combined_stride, a.combined_col_offset = c_stride, c_off
    a.weights_out = weights.ctypes.data if weights is not None else None
    a.scores_scratch = scratch.ctypes.data if scratch is not None else None
    a.lse_out = lse.ctypes.data if lse is not None else None
    a.mask = mask.ctypes.data if mask is not None else None
    a.nq, a.nk, a.head_dim = nq, nk, hd
    a.is_causal = bool(causal)
    a.scale = float(scale)
    return a
