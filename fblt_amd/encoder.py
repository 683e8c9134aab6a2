"""Local-encoder weights and descriptors (reference layouts: csrc/models/local_encoder.h:22-47,
csrc/models/hash_ngram.h:13-27, csrc/models/local_common.h:21-35).

Arrays are made with numpy; `bind` lays the ctypes structs over any memory the caller owns
(numpy arrays for a host checker, device tensors for the library), so the same seeded weights
reach both sides of a parity test.
"""
import ctypes as C

import numpy as np

from . import abi
from .decoder import LAYER_FIELDS, layer_shapes


def random_weights(E, hidden, L, ngram_sizes, vocab, seed):
    """Seeded weights: matrices ~ N(0, 1/fan_in), norm weights ~ 1 + N(0, 0.01), tables ~ N(0, 0.25)."""
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
    return {"layers": layers, "byte_embedding": (0.5 * rs.randn(256, E)).astype(np.float32),
            "tables": [(0.5 * rs.randn(vocab, E)).astype(np.float32) for _ in ngram_sizes]}


class BoundEncoder:
    """A blt_local_encoder whose tensors point at memory owned by `keep`."""

    def __init__(self, struct, layers, keep):
        self.struct, self.layers, self.keep = struct, layers, keep

    @property
    def ptr(self):
        return C.pointer(self.struct)


def bind(weights, rope_cos, rope_sin, backend, place, E, H, XH, hidden, max_seq_len, ngram_sizes, vocab, prime,
         normalize=True, patch_dim=0, window=0, all_layers=True, placement=abi.BLT_XATTN_DEFAULT,
         pool=abi.BLT_POOL_MEAN, theta=500000.0):
    """`place(array) -> (owner, address)` puts one numpy array where the encoder should read it."""
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
    enc = abi.BltLocalEncoder()
    cfg = enc.config
    cfg.embed_dim, cfg.num_layers, cfg.patch_dim, cfg.hidden_dim = E, L, patch_dim, hidden
    cfg.num_heads, cfg.cross_attn_heads, cfg.local_window = H, XH, window
    cfg.cross_attn_all_layers, cfg.cross_attn_placement, cfg.pool_type = all_layers, placement, pool
    ng = cfg.ngram_config
    for i, n in enumerate(ngram_sizes):
        ng.ngram_sizes[i] = n
    ng.num_ngram_sizes, ng.per_ngram_vocab, ng.hash_prime, ng.normalize, ng.embed_dim = (len(ngram_sizes), vocab, prime,
                                                                                        normalize, E)
    cfg.rope_theta, cfg.max_seq_len = theta, max_seq_len
    enc.byte_embedding_weight = tensor(weights["byte_embedding"])
    for i, t in enumerate(weights["tables"]):
        enc.ngram_weights.tables[i] = tensor(t)
    enc.ngram_weights.num_tables = len(weights["tables"])
    enc.rope_cos_cache, enc.rope_sin_cache = tensor(rope_cos), tensor(rope_sin)
    enc.layers = C.cast(layers, C.POINTER(abi.BltLocalLayerStorage))
    return BoundEncoder(enc, layers, keep)
