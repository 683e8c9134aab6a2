"""Local-decoder weights and two-tier cache descriptors for the decode step
(reference layouts: csrc/models/local_decoder.h:17-72, csrc/models/
local_common.h:21-35, csrc/infer/kv_cache.h:45-65).

The arrays are made with numpy; `bind` lays the ctypes structs over any memory
the caller owns (numpy arrays for a host checker, device tensors for the
library), so the same seeded weights reach both sides of a parity test.
"""
import ctypes as C

import numpy as np

from . import abi

LAYER_FIELDS = ("norm1_weight", "attn_qkv_w", "attn_proj_w", "norm2_weight", "ffn_up_w", "ffn_gate_w", "ffn_down_w",
                "cross_norm_weight", "cross_weight_q", "cross_weight_k", "cross_weight_v", "cross_weight_proj")


def layer_shapes(E, hidden):
    return {"norm1_weight": (E,), "attn_qkv_w": (E, 3 * E), "attn_proj_w": (E, E), "norm2_weight": (E,),
            "ffn_up_w": (E, hidden), "ffn_gate_w": (E, hidden), "ffn_down_w": (hidden, E),
            "cross_norm_weight": (E,), "cross_weight_q": (E, E), "cross_weight_k": (E, E), "cross_weight_v": (E, E),
            "cross_weight_proj": (E, E)}


def random_weights(E, hidden, L, V, seed):
    """Seeded weights: matrices ~ N(0, 1/fan_in), norm weights ~ 1 + N(0, 0.01)."""
    rs = np.random.RandomState(seed)
    layers = []
    for _ in range(L):
        w = {}
        for name, shape in layer_shapes(E, hidden).items():
            if len(shape) == 1:
                w[name] = (1.0 + 0.1 * rs.randn(*shape)).astype(np.float32)
            else:
                w[name] = (rs.randn(*shape) / np.sqrt(shape[0])).astype(np.float32)
        layers.append(w)
    lm_head = (rs.randn(E, V) / np.sqrt(E)).astype(np.float32)
    # drawn last, so that the weights above are what they were before the table existed
    d0_embed = (0.5 * rs.randn(257, E)).astype(np.float32)   # [BLT_D0_VOCAB, E], local_decoder.h:40
    return {"layers": layers, "lm_head_weight": lm_head, "d0_embed_weight": d0_embed}


class BoundDecoder:
    """A blt_local_decoder whose tensors point at memory owned by `keep`."""

    def __init__(self, struct, layers, keep):
        self.struct, self.layers, self.keep = struct, layers, keep

    @property
    def ptr(self):
        return C.pointer(self.struct)


def bind(weights, rope_cos, rope_sin, backend, place, E, H, XH, hidden, V, max_seq_len, patch_dim=0, window=0,
         all_layers=True, placement=abi.BLT_XATTN_DEFAULT, theta=500000.0):
    """`place(array) -> (owner, address)` puts one numpy array where the decoder should read it
    (identity for host memory, a device copy for the library)."""
    keep = []

    def tensor(arr):
        owner, addr = place(np.ascontiguousarray(arr, dtype=np.float32))
        keep.append(owner)
        return abi.tensor_view(addr, arr.shape, backend)

    L = len(weights["layers"])
    layers = (abi.BltLocalLayerStorage * L)()
    for l, w in enumerate(weights["layers"]):
        for name in LAYER_FIELDS:
            setattr(layers[l], name, tensor(w[name]))
    dec = abi.BltLocalDecoder()
    cfg = dec.config
    cfg.embed_dim, cfg.patch_dim, cfg.num_layers, cfg.hidden_dim = E, patch_dim, L, hidden
    cfg.num_heads, cfg.cross_attn_heads, cfg.local_window = H, XH, window
    cfg.cross_attn_all_layers, cfg.cross_attn_placement, cfg.rope_theta = all_layers, placement, theta
    cfg.max_seq_len, cfg.vocab_size = max_seq_len, V
    dec.rope_cos_cache, dec.rope_sin_cache = tensor(rope_cos), tensor(rope_sin)
    dec.layers = C.cast(layers, C.POINTER(abi.BltLocalLayerStorage))
    dec.lm_head_weight = tensor(weights["lm_head_weight"])
    if "d0_embed_weight" in weights:
        dec.d0_embed_weight = tensor(weights["d0_embed_weight"])
    return BoundDecoder(dec, layers, keep)


def host_place(arr):
    return arr, arr.ctypes.data


def device_place(arr):
    import torch
    t = torch.from_numpy(arr).cuda()
    return t, t.data_ptr()


class HostCache:
    """A blt_kv_cache over numpy slabs, for a host checker (layout of kv_cache.c:27-71)."""

    def __init__(self, bound, max_seq_len, batch=1):
        cfg = bound.struct.config
        E, L = cfg.embed_dim, cfg.num_layers
        patch_dim = cfg.patch_dim or E
        self.tiers = {name: [np.zeros((batch * max_seq_len, E), dtype=np.float32) for _ in range(L)]
                      for name in ("self_k", "self_v", "cross_k", "cross_v")}
        self.handles = {name: (abi.BltTensor * L)(*(abi.tensor_view(a.ctypes.data, a.shape, abi.BLT_BACKEND_CPU)
                                                    for a in arrs)) for name, arrs in self.tiers.items()}
        self.patch_table = (abi.BltPatchInfo * (batch * max_seq_len))()
        c = abi.BltKvCache()
        c.decoder = bound.ptr
        c.max_seq_len, c.batch_size, c.max_subtokens, c.embed_dim = max_seq_len, batch, max_seq_len, E
        c.k, c.patch_dim = patch_dim // E, patch_dim
        for name in self.tiers:
            setattr(c, name, C.cast(self.handles[name], C.POINTER(abi.BltTensor)))
        c.cached_patches = C.cast(self.patch_table, C.POINTER(abi.BltPatchInfo))
        self.struct, self.bound = c, bound

    @property
    def ptr(self):
        return C.pointer(self.struct)


class BlockBatch:
    """A blt_block_batch for the inference forward (csrc/models/block_diffusion.h:37-86,
    filled as csrc/infer/block_generation.c:171-215 fills it): R block rows behind num_clean
    clean rows; tokens / positions / groups as given (defaults: all [MASK], positions
    num_clean + r, every row on the last latent)."""

    def __init__(self, num_clean, R, num_patches, tokens=None, positions=None, groups=None, trailing_closed=1,
                 num_blocks=1):
        self.tokens = (C.c_uint32 * R)(*(tokens if tokens is not None else [abi.BLT_MASK_TOKEN_ID] * R))
        self.positions = (C.c_size_t * R)(*(positions if positions is not None else range(num_clean, num_clean + R)))
        self.groups = (C.c_size_t * R)(*(groups if groups is not None else [num_patches - 1] * R))
        self.masked = (C.c_uint8 * R)(*([1] * R))
        self.valid = (C.c_uint8 * R)(*([1] * R))
        self.targets = (C.c_uint8 * R)()
        b = abi.BltBlockBatch()
        b.num_clean, b.block_size, b.num_blocks, b.n_block_rows = num_clean, R // num_blocks, num_blocks, R
        b.tokens, b.positions, b.groups = self.tokens, self.positions, self.groups
        b.targets, b.cell_valid, b.cell_masked = self.targets, self.valid, self.masked
        b.trailing_closed = trailing_closed
        self.struct = b

    @property
    def ptr(self):
        return C.pointer(self.struct)


def patch_table(lengths):
    """blt_patch_info array tiling [0, sum(lengths)) (csrc/models/patcher.h:16-20)."""
    starts = np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(int)
    return abi.patch_array(starts.tolist(), [int(x) for x in lengths])
