"""One whole-model inference forward -- blt_model_encode + blt_model_decode, csrc/models/model.c:68-131:
local encoder, patch transformer, local decoder, LM head -- through the reference's own driver code, either the CPU
reference build on host tensors or the same sources compiled unmodified on top of the HIP library,
on device tensors.  Not collected by pytest."""
import ctypes as C

import numpy as np

from fblt_amd import abi, decoder, encoder
from oracle import binding
from tests import encoder_runs

GLOBAL_ORDER = ("norm1_weight", "attn_qkv_w", "attn_proj_w", "norm2_weight", "ffn_up_w", "ffn_gate_w", "ffn_down_w")

# embed_dim shared by the three stages and patch_dim == embed_dim (csrc/models/model.c:37-39, 80-86); the encoder case dictionary of
# tests/golden/block_cases.py plus the patch transformer's and the decoder's own sizes
CASES = {
    "model_T96": dict(T=96, E=64, H=2, XH=2, hidden=96, L=2, k=1, ngrams=[3, 4], vocab=257, normalize=True, window=0,
                      all_layers=True, placement=abi.BLT_XATTN_DEFAULT, pool="mean", docs=[],
                      g_layers=2, g_hidden=128, g_heads=2, d_layers=2, d_hidden=96, V=256),
    "model_T200_docs_window": dict(T=200, E=128, H=4, XH=4, hidden=256, L=1, k=1, ngrams=[3, 5, 8], vocab=500,
                                   normalize=False, window=48, all_layers=True, placement=abi.BLT_XATTN_DEFAULT,
                                   pool="max", docs=[2], g_layers=3, g_hidden=256, g_heads=4, d_layers=3, d_hidden=256,
                                   V=256),
}


def inputs(name):
    """(case, byte ids, patch lengths, encoder / patch transformer / decoder weights); `docs` lists
    the PATCHES at which documents 1, 2, ... start."""
    c = CASES[name]
    rs = np.random.RandomState(len(name) * 131 + c["T"])
    data = rs.randint(0, 256, size=c["T"]).astype(np.uint8)
    lengths = []
    while sum(lengths) < c["T"]:
        lengths.append(int(min(rs.randint(1, 9), c["T"] - sum(lengths))))
    enc_w = encoder.random_weights(c["E"], c["hidden"], c["L"], c["ngrams"], c["vocab"], seed=int(rs.randint(1 << 30)))
    dec_w = decoder.random_weights(c["E"], c["d_hidden"], c["d_layers"], c["V"], seed=int(rs.randint(1 << 30)))
    E, GH = c["E"], c["g_hidden"]
    glob_w = []
    for _ in range(c["g_layers"]):
        w = {"norm1_weight": 1.0 + 0.1 * rs.randn(E), "attn_qkv_w": rs.randn(E, 3 * E) / np.sqrt(E),
             "attn_proj_w": rs.randn(E, E) / np.sqrt(E), "norm2_weight": 1.0 + 0.1 * rs.randn(E),
             "ffn_up_w": rs.randn(E, GH) / np.sqrt(E), "ffn_gate_w": rs.randn(E, GH) / np.sqrt(E),
             "ffn_down_w": rs.randn(GH, E) / np.sqrt(GH)}
        glob_w.append({n: np.ascontiguousarray(a, dtype=np.float32) for n, a in w.items()})
    return c, data, lengths, enc_w, glob_w, dec_w


def run(driver, mem, orc, backend, place, fill, sync, c, data, lengths, enc_w, glob_w, dec_w):
    """driver: library holding blt_model_encode / _decode and blt_global_transformer_create (reference
    sources); mem: library holding blt_arena_create / _destroy for `backend`; place: where numpy
    arrays go (decoder.host_place / device_place); fill(tensor struct, array): writes a weight the
    driver's constructor allocated; sync(): wait for the device.  Returns logits [T, V]."""
    T, E, P = c["T"], c["E"], len(lengths)
    enc = encoder_runs.bound(orc, c, enc_w, backend, place)
    cos, sin = encoder_runs.rope_tables(orc, c)
    dec = decoder.bind(dec_w, cos, sin, backend, place, E, c["H"], c["XH"], c["d_hidden"], c["V"], T, window=c["window"])
    arena = mem.blt_arena_create(512 << 20, backend)
    try:
        gcfg = binding.BltGlobalTransformerConfig(E, c["g_layers"], c["g_hidden"], c["g_heads"], 500000.0, 1024, False,
                                                  False)
        glob = driver.blt_global_transformer_create(arena, C.byref(gcfg))
        for l, w in enumerate(glob_w):
            for n in GLOBAL_ORDER:
                fill(getattr(glob.contents.stack.layer_weights[l], n), w[n])
        model = binding.BltModel()
        model.config.encoder_config = enc.struct.config
        model.config.global_config = gcfg
        model.config.decoder_config = dec.struct.config
        model.encoder, model.global_, model.decoder = enc.ptr, glob, dec.ptr
        patches = decoder.patch_table(lengths)
        starts = np.concatenate([[0], np.cumsum(lengths)[:-1]])
        # the model's convention: one entry per document, document 0 at offset 0 (model.h:49-52)
        docs = abi.size_array([0] + [int(starts[p]) for p in c["docs"]]) if c["docs"] else None
        num_docs = len(c["docs"]) + 1 if c["docs"] else 0
        owner_b, addr_b = place_bytes(place, data)
        tb = abi.tensor_view(addr_b, data.shape, backend, dtype=abi.BLT_DTYPE_UINT8)
        logits = np.zeros((T, c["V"]), dtype=np.float32)
        owner_l, addr_l = place(logits)
        tl = abi.tensor_view(addr_l, logits.shape, backend)
        # inference: encode once, decode without the loss (bytes are the encoder's input only)
        enc_out = binding.BltModelEncOut()
        driver.blt_model_encode(C.byref(model), C.byref(tb), patches, P, docs, num_docs, C.byref(enc_out), arena)
        driver.blt_model_decode(C.byref(model), C.byref(enc_out), patches, P, None, None, docs, num_docs, None,
                                C.byref(tl), None, arena)
        sync()
        return fetch(owner_l)
    finally:
        mem.blt_arena_destroy(arena)


def place_bytes(place, data):
    if place is decoder.host_place:
        return data, data.ctypes.data
    import torch
    t = torch.from_numpy(data).cuda()
    return t, t.data_ptr()


def fetch(owner):
    return owner.copy() if isinstance(owner, np.ndarray) else owner.cpu().numpy()


def run_oracle(orc, c, data, lengths, enc_w, glob_w, dec_w):
    """The same forward as a composition of the restated stages: local encoder, the patch
    transformer's blocks under the document-causal mask over patches, local decoder."""
    T, E, P = c["T"], c["E"], len(lengths)
    starts = np.concatenate([[0], np.cumsum(lengths)[:-1]])
    byte_case = dict(c, docs=[int(starts[p]) for p in c["docs"]])   # the encoder's masks count bytes
    patch_out, byte_hidden = encoder_runs.run_oracle(orc, byte_case, data, lengths, enc_w)
    mc = abi.BltMaskConfig()
    mc.seq_len_q = mc.seq_len_kv = P
    mc.is_causal = True
    patch_docs = abi.size_array(list(c["docs"])) if c["docs"] else None   # mask convention: starts of documents 1, 2, ...
    if c["docs"]:
        mc.doc_boundaries, mc.num_docs = patch_docs, len(c["docs"]) + 1
    cur = np.ascontiguousarray(patch_out)
    for w in glob_w:
        nxt = np.zeros((P, E), dtype=np.float32)
        assert orc.orc_transformer_forward(binding.fptr(cur.reshape(-1)),
                                           *(binding.fptr(w[n].reshape(-1)) for n in GLOBAL_ORDER),
                                           binding.fptr(nxt.reshape(-1)), P, E, c["g_hidden"], c["g_heads"], 1, 1, 500000.0,
                                           None, None, C.byref(mc)) == 0
        cur = nxt
    cos, sin = encoder_runs.rope_tables(orc, c)
    dec = decoder.bind(dec_w, cos, sin, abi.BLT_BACKEND_CPU, decoder.host_place, E, c["H"], c["XH"], c["d_hidden"], c["V"],
                       T, window=c["window"])
    byte_docs = abi.size_array([int(starts[p]) for p in c["docs"]]) if c["docs"] else None
    logits = np.zeros((T, c["V"]), dtype=np.float32)
    rc = orc.orc_local_decoder_forward(dec.ptr, binding.fptr(byte_hidden.reshape(-1)), T, binding.fptr(cur.reshape(-1)),
                                       decoder.patch_table(lengths), P, byte_docs, len(c["docs"]) + 1 if c["docs"] else 0,
                                       0, binding.fptr(logits.reshape(-1)))
    assert rc == 0, rc
    return logits
