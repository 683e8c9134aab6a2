"""Seeded inputs of the block-level golden cases (attention block, cross-attention block, whole
decoder step).  Shared by the generator (make_golden_blocks.py, which feeds them to the reference
build) and by the tests (which feed them to the CPU checker and to the HIP library)."""
import numpy as np

from fblt_amd import abi, decoder

MHA_CASES = {
    # T, E, H, rope, mask ("causal_flag", "causal_cfg", "window", "docs")
    "mha_T96_E64_H2_rope": dict(T=96, E=64, H=2, rope=True, mask="causal_cfg"),
    "mha_T50_E48_H3_window": dict(T=50, E=48, H=3, rope=True, mask="window"),
    "mha_T33_E32_H4_docs": dict(T=33, E=32, H=4, rope=False, mask="docs"),
}
XATTN_CASES = {
    "xattn_P16_T64_E64_H2": dict(P=16, T=64, E=64, H=2),
    "xattn_P40_T150_E32_H4": dict(P=40, T=150, E=32, H=4),
}
STEP_CASES = {
    # decoder configuration and a script of (patch lengths so far, from_patch, new rows, trailing_closed)
    "step_E64_L2_k2_window": dict(E=64, H=2, XH=2, L=2, hidden=96, V=64, max_len=48, k=2, window=9,
                                  all_layers=True, placement=0),
    "step_E32_L3_last_only": dict(E=32, H=4, XH=1, L=3, hidden=48, V=256, max_len=40, k=1, window=0,
                                  all_layers=False, placement=0),
}
STEP_SCRIPT = [([3, 4], 0, 7, 0), ([3, 4, 1], 2, 1, 0), ([3, 4, 2], 2, 1, 1), ([3, 4, 2, 5], 3, 5, 0),
               ([3, 4, 2, 5, 1], 4, 1, 0), ([3, 4, 2, 5, 4], 4, 3, 1), ([3, 4, 2, 5, 4, 3], 5, 3, 0)]
# inference-mode diffusion forward: decoder configuration, patch lengths of the clean prefix, block
# rows, trailing_closed, learned D_0 table or zeros, "draft" (all [MASK], positions N + r, every row
# on the last latent -- csrc/infer/block_generation.c:171-215) or "mixed" (seeded tokens, positions
# and groups)
DIFFUSION_CASES = {
    "diff_E64_k2_draft_B8": dict(E=64, H=2, XH=2, L=2, hidden=96, V=64, max_len=80, k=2, window=9, all_layers=True,
                                 placement=0, lengths=[5, 9, 3, 12, 7], R=8, closed=1, learned=True, fill="draft"),
    "diff_E32_last_mixed_B4": dict(E=32, H=4, XH=1, L=3, hidden=48, V=256, max_len=48, k=1, window=0,
                                   all_layers=False, placement=0, lengths=[4, 6, 5], R=4, closed=0, learned=True,
                                   fill="mixed"),
    "diff_E128_zeros_B16": dict(E=128, H=4, XH=4, L=2, hidden=256, V=256, max_len=128, k=1, window=0, all_layers=True,
                                placement=0, lengths=[16, 9, 20, 11, 14], R=16, closed=1, learned=False, fill="draft"),
}
# the transformer block (csrc/models/transformer.c:97-128): T, E, H, hidden, mask kind
TRANSFORMER_CASES = {
    "block_T128_E512_H8_docs": (128, 512, 8, 1024, "docs"),           # a layer of the patch transformer at C2 size
    "block_T96_E64_H2_docs_window": (96, 64, 2, 160, "docs_window"),  # a byte layer of the local encoder
}
# the local encoder (csrc/models/local_encoder.c:193-281): bytes, patch lengths, sizes, options
ENCODER_CASES = {
    # C3's caller at its size: 512 bytes in 128 patches, 4 x 32 heads, cross block in every layer
    "enc_T512_L2": dict(T=512, E=128, H=4, XH=4, L=2, hidden=256, ngrams=(3, 4, 5), vocab=2048, k=1, window=0,
                             placement=0, all_layers=True, pool="mean", docs=None, normalize=True, mean_patch=4),
    # sub-token split, window, documents, max pooling, cross block after the last layer only
    "enc_T150_k2_window_docs_max": dict(T=150, E=64, H=2, XH=4, L=3, hidden=96, ngrams=(2, 3, 8), vocab=257, k=2,
                                        window=40, placement=0, all_layers=False, pool="max", docs=[60, 111],
                                        normalize=False, mean_patch=6),
}
THETA = 500000.0


def seed_of(name):
    return sum(ord(ch) * (i + 1) for i, ch in enumerate(name)) % (2 ** 31)


def mha_inputs(name):
    c = MHA_CASES[name]
    rs = np.random.RandomState(seed_of(name))
    T, E = c["T"], c["E"]
    x = rs.randn(T, E).astype(np.float32)
    wqkv = (rs.randn(E, 3 * E) / np.sqrt(E)).astype(np.float32)
    wproj = (rs.randn(E, E) / np.sqrt(E)).astype(np.float32)
    return c, x, wqkv, wproj


def mha_mask(c):
    """(is_causal, sliding_window, doc boundary list or None) of the case's mask configuration."""
    if c["mask"] == "window":
        return True, 11, None
    if c["mask"] == "docs":
        return False, 0, [9, 20]
    return True, 0, None


def xattn_inputs(name):
    c = XATTN_CASES[name]
    rs = np.random.RandomState(seed_of(name))
    P, T, E = c["P"], c["T"], c["E"]
    xq, xkv = rs.randn(P, E).astype(np.float32), rs.randn(T, E).astype(np.float32)
    ws = [(rs.randn(E, E) / np.sqrt(E)).astype(np.float32) for _ in range(4)]
    groups = np.sort(np.concatenate([np.arange(P), rs.randint(0, P, size=T - P)]))
    return c, xq, xkv, ws, groups


def step_inputs(name):
    """Decoder weights, the rows of every call of the script and the patch latents per call."""
    c = STEP_CASES[name]
    rs = np.random.RandomState(seed_of(name))
    weights = decoder.random_weights(c["E"], c["hidden"], c["L"], c["V"], seed_of(name) + 1)
    total = sum(n for _l, _f, n, _c in STEP_SCRIPT)
    d0 = rs.randn(total, c["E"]).astype(np.float32)
    latents, prev = [], None
    for lengths, from_patch, _n, _closed in STEP_SCRIPT:
        pin = rs.randn(len(lengths), c["k"] * c["E"]).astype(np.float32)
        if from_patch:
            pin[:from_patch] = prev[:from_patch]   # completed patches keep their latents
        latents.append(pin)
        prev = pin
    return c, weights, d0, latents


def diffusion_inputs(name):
    """Decoder weights, clean-row states, patch latents and the block section of a diffusion case."""
    c = DIFFUSION_CASES[name]
    rs = np.random.RandomState(seed_of(name))
    weights = decoder.random_weights(c["E"], c["hidden"], c["L"], c["V"], seed_of(name) + 1)
    N, P, R = sum(c["lengths"]), len(c["lengths"]), c["R"]
    hidden = rs.randn(N, c["E"]).astype(np.float32)
    latents = rs.randn(P, c["k"] * c["E"]).astype(np.float32)
    if c["fill"] == "draft":
        batch = decoder.BlockBatch(N, R, P, trailing_closed=c["closed"])
    else:
        tokens = [int(rs.randint(0, 256)) if rs.rand() < 0.5 else 256 for _ in range(R)]
        positions = [int(x) for x in np.sort(rs.randint(0, c["max_len"], size=R))]
        groups = [int(rs.randint(0, P)) for _ in range(R)]
        batch = decoder.BlockBatch(N, R, P, tokens=tokens, positions=positions, groups=groups,
                                   trailing_closed=c["closed"])
    return c, weights, hidden, latents, batch


def transformer_case(rs, T, E, H, hidden, mask):
    """Seeded inputs of one RMSNorm + SwiGLU block and its mask configuration: "causal" (the
    decoder's), "window" (causal + sliding window), "docs" (document-causal: the patch transformer's,
    csrc/models/global_transformer.c:19-33), "docs_window" (the local encoder's); "docs_edge[_window]": document boundaries at the edges of what
    csrc/ops/mask_builder_cpu.c:10-19 accepts."""
    x = rs.randn(T, E).astype(np.float32)
    w = {"norm1": (1.0 + 0.1 * rs.randn(E)).astype(np.float32), "qkv": (rs.randn(E, 3 * E) / np.sqrt(E)).astype(np.float32),
         "proj": (rs.randn(E, E) / np.sqrt(E)).astype(np.float32), "norm2": (1.0 + 0.1 * rs.randn(E)).astype(np.float32),
         "up": (rs.randn(E, hidden) / np.sqrt(E)).astype(np.float32),
         "gate": (rs.randn(E, hidden) / np.sqrt(E)).astype(np.float32),
         "down": (rs.randn(hidden, E) / np.sqrt(hidden)).astype(np.float32)}
    cfg = abi.BltMaskConfig()
    cfg.seq_len_q = cfg.seq_len_kv = T
    cfg.is_causal = True
    keep = None
    if "window" in mask:
        cfg.sliding_window = max(2, T // 5)
    if "docs" in mask:
        cuts = sorted(set(int(v) for v in rs.randint(1, T, size=3))) if T > 4 else [1]
        if "edge" in mask:  # a boundary at 0, a repeated one, one-row documents, a boundary past the end
            cuts = [0, 1, 1, 5, T - 1, T + 3]
        keep = abi.size_array(cuts)
        cfg.doc_boundaries, cfg.num_docs = keep, len(cuts) + 1
    return x, w, cfg, keep


def encoder_case(rs, c):
    """Bytes, patch lengths and weights of one encoder configuration."""
    from fblt_amd import encoder
    T = c["T"]
    lengths = []
    while sum(lengths) < T:
        lengths.append(int(min(T - sum(lengths), max(1, rs.poisson(c["mean_patch"] - 1) + 1))))
    data = rs.randint(0, 256, size=T).astype(np.uint8)
    data[rs.randint(0, T, size=T // 4)] = 32   # repeated bytes: hash buckets get hit more than once
    weights = encoder.random_weights(c["E"], c["hidden"], c["L"], c["ngrams"], c["vocab"], int(rs.randint(1 << 30)))
    return data, lengths, weights


def encoder_inputs(name):
    c = ENCODER_CASES[name]
    return (c,) + encoder_case(np.random.RandomState(seed_of(name)), c)


def transformer_inputs(name):
    T, E, H, hidden, mask = TRANSFORMER_CASES[name]
    return (T, E, H, hidden, mask) + transformer_case(np.random.RandomState(seed_of(name)), T, E, H, hidden, mask)
