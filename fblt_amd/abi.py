"""ctypes view of the boundary structs declared in include/blt_abi.h.

Field order and types follow that header one to one; `check_layout()` asserts
the sizes the header's static assertions state, so a drift between the two is
caught at import time.
"""
import ctypes as C

BLT_BACKEND_CPU = 0
BLT_BACKEND_HIP = 1

BLT_DTYPE_FP32 = 0

BLT_BDM_TRAIN = 0
BLT_BDM_INFER = 1

BLT_MAX_NDIM = 4

c_float_p = C.POINTER(C.c_float)
c_size_p = C.POINTER(C.c_size_t)


class BltTensor(C.Structure):
    _fields_ = [
        ("data", C.c_void_p),
        ("shape", C.c_size_t * BLT_MAX_NDIM),
        ("strides", C.c_size_t * BLT_MAX_NDIM),
        ("ndim", C.c_size_t),
        ("numel", C.c_size_t),
        ("dtype", C.c_int),
        ("backend", C.c_int),
        ("is_view", C.c_bool),
    ]


class BltArena(C.Structure):
    _fields_ = [
        ("buffer", C.c_void_p),
        ("capacity", C.c_size_t),
        ("offset", C.c_size_t),
        ("backend", C.c_int),
    ]


class BltAttentionHeadArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p),
        ("q_stride", C.c_size_t),
        ("k", C.c_void_p),
        ("k_stride", C.c_size_t),
        ("v", C.c_void_p),
        ("v_stride", C.c_size_t),
        ("combined", C.c_void_p),
        ("combined_stride", C.c_size_t),
        ("combined_col_offset", C.c_size_t),
        ("weights_out", C.c_void_p),
        ("lse_out", C.c_void_p),
        ("scores_scratch", C.c_void_p),
        ("mask", C.c_void_p),
        ("nq", C.c_size_t),
        ("nk", C.c_size_t),
        ("head_dim", C.c_size_t),
        ("is_causal", C.c_bool),
        ("scale", C.c_float),
    ]


class BltMaskConfig(C.Structure):
    _fields_ = [
        ("seq_len_q", C.c_size_t),
        ("seq_len_kv", C.c_size_t),
        ("sliding_window", C.c_size_t),
        ("doc_boundaries", c_size_p),
        ("num_docs", C.c_size_t),
        ("query_group_ids", c_size_p),
        ("kv_group_ids", c_size_p),
        ("bidirectional_within_group", C.c_bool),
        ("is_causal", C.c_bool),
        ("causal_offset", C.c_size_t),
    ]


class BltBlockDiffusionConfig(C.Structure):
    _fields_ = [
        ("mode", C.c_int),
        ("seq_len", C.c_size_t),
        ("num_clean", C.c_size_t),
        ("block_size", C.c_size_t),
        ("block_starts", c_size_p),
        ("num_blocks", C.c_size_t),
    ]


class BltRopeConfig(C.Structure):
    _fields_ = [("theta", C.c_float), ("head_dim", C.c_size_t)]


class BltAttentionConfig(C.Structure):
    _fields_ = [
        ("embed_dim", C.c_size_t),
        ("num_heads", C.c_size_t),
        ("head_dim", C.c_size_t),
        ("is_causal", C.c_bool),
        ("use_rope", C.c_bool),
        ("rope_theta", C.c_float),
        ("rope_cos_cache", C.POINTER(BltTensor)),
        ("rope_sin_cache", C.POINTER(BltTensor)),
        ("mask_config", C.POINTER(BltMaskConfig)),
    ]


BLT_NORM_LAYERNORM, BLT_NORM_RMSNORM = 0, 1
BLT_ACTIVATION_GELU, BLT_ACTIVATION_SWIGLU = 0, 1


class BltTransformerConfig(C.Structure):
    """csrc/models/transformer.h:31-38"""
    _fields_ = [
        ("attn_config", BltAttentionConfig),
        ("hidden_dim", C.c_size_t),
        ("layer_norm_eps", C.c_float),
        ("norm_type", C.c_int),
        ("activation_type", C.c_int),
        ("use_bf16", C.c_int),
    ]


class BltCrossAttentionConfig(C.Structure):
    """csrc/models/cross_attention.h:27-34"""
    _fields_ = [
        ("embed_dim", C.c_size_t),
        ("patch_dim", C.c_size_t),
        ("split_mode", C.c_int),
        ("num_heads", C.c_size_t),
        ("head_dim", C.c_size_t),
        ("mask_config", C.POINTER(BltMaskConfig)),
    ]


class BltCrossAttentionWeights(C.Structure):
    _fields_ = [(n, C.POINTER(BltTensor)) for n in ("weight_q", "weight_k", "weight_v", "weight_proj")]


class BltTransformerWeights(C.Structure):
    _fields_ = [(n, C.POINTER(BltTensor)) for n in ("norm1_weight", "norm1_bias", "attn_qkv_w", "attn_proj_w",
                                                    "norm2_weight", "norm2_bias", "ffn_up_w", "ffn_gate_w",
                                                    "ffn_down_w")]


class BltPatchInfo(C.Structure):
    _fields_ = [
        ("start_idx", C.c_size_t),
        ("length", C.c_size_t),
        ("peak_entropy", C.c_float),
    ]


class BltLocalLayerStorage(C.Structure):
    """csrc/models/local_common.h:21-35"""
    _fields_ = [(n, BltTensor) for n in (
        "norm1_weight", "attn_qkv_w", "attn_proj_w", "norm2_weight", "ffn_up_w", "ffn_gate_w", "ffn_down_w",
        "cross_norm_weight", "cross_weight_q", "cross_weight_k", "cross_weight_v", "cross_weight_proj")]


class BltLocalDecoderConfig(C.Structure):
    """csrc/models/local_decoder.h:17-30"""
    _fields_ = [
        ("embed_dim", C.c_size_t),
        ("patch_dim", C.c_size_t),
        ("num_layers", C.c_size_t),
        ("hidden_dim", C.c_size_t),
        ("num_heads", C.c_size_t),
        ("cross_attn_heads", C.c_size_t),
        ("local_window", C.c_size_t),
        ("cross_attn_all_layers", C.c_bool),
        ("cross_attn_placement", C.c_int),
        ("rope_theta", C.c_float),
        ("max_seq_len", C.c_size_t),
        ("vocab_size", C.c_size_t),
    ]


class BltLocalDecoder(C.Structure):
    """csrc/models/local_decoder.h:60-72"""
    _fields_ = [
        ("config", BltLocalDecoderConfig),
        ("rope_cos_cache", BltTensor),
        ("rope_sin_cache", BltTensor),
        ("layers", C.POINTER(BltLocalLayerStorage)),
        ("lm_head_weight", BltTensor),
        ("d0_embed_weight", BltTensor),
    ]


class BltKvCache(C.Structure):
    """csrc/infer/kv_cache.h:45-65"""
    _fields_ = [
        ("decoder", C.POINTER(BltLocalDecoder)),
        ("max_seq_len", C.c_size_t),
        ("batch_size", C.c_size_t),
        ("max_subtokens", C.c_size_t),
        ("embed_dim", C.c_size_t),
        ("k", C.c_size_t),
        ("patch_dim", C.c_size_t),
        ("self_k", C.POINTER(BltTensor)),
        ("self_v", C.POINTER(BltTensor)),
        ("self_len", C.c_size_t),
        ("cross_k", C.POINTER(BltTensor)),
        ("cross_v", C.POINTER(BltTensor)),
        ("cross_num_patches", C.c_size_t),
        ("cached_patches", C.POINTER(BltPatchInfo)),
    ]


BLT_XATTN_DEFAULT, BLT_XATTN_NONE, BLT_XATTN_LAST, BLT_XATTN_ALL, BLT_XATTN_FIRST = range(5)
BLT_D0_HFINAL, BLT_D0_ZEROS, BLT_D0_LEARNED = range(3)
BLT_MASK_TOKEN_ID = 256


class BltBlockBatch(C.Structure):
    """csrc/models/block_diffusion.h:37-86"""
    _fields_ = [
        ("num_clean", C.c_size_t),
        ("block_size", C.c_size_t),
        ("num_blocks", C.c_size_t),
        ("n_block_rows", C.c_size_t),
        ("t", C.c_float),
        ("tokens", C.POINTER(C.c_uint32)),
        ("positions", C.POINTER(C.c_size_t)),
        ("targets", C.POINTER(C.c_uint8)),
        ("cell_valid", C.POINTER(C.c_uint8)),
        ("cell_masked", C.POINTER(C.c_uint8)),
        ("groups", C.POINTER(C.c_size_t)),
        ("loss_scale", C.c_float),
        ("last_row_scale", C.c_float),
        ("clean_sum", C.c_int),
        ("mask_norm", C.c_int),
        ("trailing_closed", C.c_int),
    ]


BLT_POOL_MEAN, BLT_POOL_MAX = range(2)
BLT_IDX_SENTINEL = 0xFFFFFFFF
BLT_MAX_NGRAM_SIZES = 6
BLT_DTYPE_UINT8 = 3


class BltHashNgramConfig(C.Structure):
    """csrc/models/hash_ngram.h:13-22"""
    _fields_ = [
        ("ngram_sizes", C.c_size_t * BLT_MAX_NGRAM_SIZES),
        ("num_ngram_sizes", C.c_size_t),
        ("per_ngram_vocab", C.c_size_t),
        ("hash_prime", C.c_uint64),
        ("normalize", C.c_bool),
        ("embed_dim", C.c_size_t),
    ]


class BltHashNgramWeights(C.Structure):
    """csrc/models/hash_ngram.h:24-27"""
    _fields_ = [("tables", BltTensor * BLT_MAX_NGRAM_SIZES), ("num_tables", C.c_size_t)]


class BltLocalEncoderConfig(C.Structure):
    """csrc/models/local_encoder.h:22-36"""
    _fields_ = [
        ("embed_dim", C.c_size_t),
        ("num_layers", C.c_size_t),
        ("patch_dim", C.c_size_t),
        ("hidden_dim", C.c_size_t),
        ("num_heads", C.c_size_t),
        ("cross_attn_heads", C.c_size_t),
        ("local_window", C.c_size_t),
        ("cross_attn_all_layers", C.c_bool),
        ("cross_attn_placement", C.c_int),
        ("pool_type", C.c_int),
        ("ngram_config", BltHashNgramConfig),
        ("rope_theta", C.c_float),
        ("max_seq_len", C.c_size_t),
    ]


class BltLocalEncoder(C.Structure):
    """csrc/models/local_encoder.h:40-47"""
    _fields_ = [
        ("config", BltLocalEncoderConfig),
        ("byte_embedding_weight", BltTensor),
        ("ngram_weights", BltHashNgramWeights),
        ("rope_cos_cache", BltTensor),
        ("rope_sin_cache", BltTensor),
        ("layers", C.POINTER(BltLocalLayerStorage)),
    ]


def check_layout():
    assert C.sizeof(BltHashNgramConfig) == 88 and BltHashNgramConfig.hash_prime.offset == 64
    assert C.sizeof(BltHashNgramWeights) == 632
    assert C.sizeof(BltLocalEncoderConfig) == 176 and BltLocalEncoderConfig.ngram_config.offset == 72
    assert C.sizeof(BltLocalEncoder) == 1128 and BltLocalEncoder.layers.offset == 1120
    assert C.sizeof(BltTransformerConfig) == 80
    assert C.sizeof(BltBlockBatch) == 112
    assert C.sizeof(BltTensor) == 104
    assert C.sizeof(BltArena) == 32
    assert C.sizeof(BltAttentionHeadArgs) == 136
    assert BltAttentionHeadArgs.mask.offset == 96
    assert BltAttentionHeadArgs.is_causal.offset == 128
    assert BltAttentionHeadArgs.scale.offset == 132
    assert C.sizeof(BltMaskConfig) == 72
    assert BltMaskConfig.causal_offset.offset == 64
    assert C.sizeof(BltBlockDiffusionConfig) == 48
    assert C.sizeof(BltPatchInfo) == 24
    assert C.sizeof(BltRopeConfig) == 16 and BltRopeConfig.head_dim.offset == 8
    assert C.sizeof(BltAttentionConfig) == 56 and BltAttentionConfig.rope_theta.offset == 28
    assert BltAttentionConfig.mask_config.offset == 48
    assert C.sizeof(BltTransformerWeights) == 72
    assert C.sizeof(BltCrossAttentionConfig) == 48 and BltCrossAttentionConfig.num_heads.offset == 24
    assert C.sizeof(BltCrossAttentionWeights) == 32
    assert C.sizeof(BltLocalLayerStorage) == 1248 and C.sizeof(BltLocalDecoderConfig) == 88
    assert C.sizeof(BltLocalDecoder) == 512 and BltLocalDecoder.layers.offset == 296
    assert C.sizeof(BltKvCache) == 112 and BltKvCache.cached_patches.offset == 104


def tensor_view(ptr, shape, backend, dtype=BLT_DTYPE_FP32):
    """A row-major blt_tensor view of existing memory (csrc/core/tensor.c:48-75)."""
    t = BltTensor()
    t.data = ptr
    numel, stride = 1, 1
    for d in range(len(shape)):
        t.shape[d] = shape[d]
        numel *= shape[d]
    for d in reversed(range(len(shape))):
        t.strides[d] = stride
        stride *= shape[d]
    t.ndim, t.numel, t.dtype, t.backend, t.is_view = len(shape), numel, dtype, backend, True
    return t


check_layout()


def size_array(values):
    """A ctypes size_t[] holding `values` (kept alive by the caller)."""
    values = [int(v) for v in values]
    return (C.c_size_t * max(len(values), 1))(*values)


def patch_array(starts, lengths):
    n = len(starts)
    arr = (BltPatchInfo * max(n, 1))()
    for i in range(n):
        arr[i].start_idx = int(starts[i])
        arr[i].length = int(lengths[i])
        arr[i].peak_entropy = 0.0
    return arr
