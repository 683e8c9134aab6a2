"""The five attention workloads of the benchmark, in the reference's layouts.

Each builder returns host (numpy) buffers plus a list of per-(sequence, head)
problems expressed as element offsets into those buffers, exactly the pointer
arithmetic the reference's callers do:

* packed self-attention `qkv[T, 3E]`, head h at columns h*hd / E+h*hd / 2E+h*hd,
  row stride 3E, output `[T, E]` (csrc/models/attention.c:92-128);
* cross-attention Q `[P, E]`, K/V `[T, E]`, row stride E
  (csrc/models/cross_attention.c:70-96);
* KV cache `[batch*max_seq_len, E]`, row = b*max_seq_len + position
  (csrc/infer/kv_cache.c:56-60), new rows appended before attending
  (kv_cache.c:343-390).

The same description is realised over host memory for the CPU checker and over
device memory for the HIP library, so both see identical bytes.
"""
from dataclasses import dataclass, field

import numpy as np

from . import synth


@dataclass
class Head:
    """One (sequence, head) problem; offsets and strides in float elements."""
    q: tuple          # (buffer name, element offset, row stride)
    k: tuple
    v: tuple
    out: tuple        # (buffer name, element offset of row 0 col 0, row stride, column offset)
    nq: int
    nk: int
    hd: int
    scale: float
    mask: str = "none"      # none | causal | dense | range
    mask_ref: tuple = ()    # dense: (buffer name, element offset); range: (lo name, hi name, element offset)
    causal_offset: int = 0
    window: int = 0
    seq: int = 0            # sequence index (for grouping)


@dataclass
class Workload:
    name: str
    buffers: dict                     # name -> float32 ndarray (inputs and zeroed outputs)
    ranges: dict = field(default_factory=dict)   # name -> uint32 ndarray (row ranges)
    heads: list = field(default_factory=list)
    outputs: tuple = ("out",)
    tokens: int = 0                   # query rows per pass
    flops: float = 0.0                # algorithmic: 4 * hd * visible pairs
    bytes: float = 0.0                # algorithmic: Q, K, V read once, O written once (fp32)
    meta: dict = field(default_factory=dict)


def _packed_self_attention(name, cfg_id, batch, T, H, hd):
    E = H * hd
    qkv = np.empty((batch, T, 3 * E), dtype=np.float32)
    # Q, K, V are separate seeded streams laid into the packed buffer
    qkv[:, :, 0:E] = synth.normal(synth.seed_for(cfg_id, synth.S_Q), (batch, T, E))
    qkv[:, :, E:2 * E] = synth.normal(synth.seed_for(cfg_id, synth.S_K), (batch, T, E))
    qkv[:, :, 2 * E:] = synth.normal(synth.seed_for(cfg_id, synth.S_V), (batch, T, E))
    out = np.zeros((batch, T, E), dtype=np.float32)
    scale = float(np.float32(1.0) / np.sqrt(np.float32(hd)))
    heads = []
    for b in range(batch):
        for h in range(H):
            base = b * T * 3 * E
            heads.append(Head(q=("qkv", base + h * hd, 3 * E), k=("qkv", base + E + h * hd, 3 * E),
                              v=("qkv", base + 2 * E + h * hd, 3 * E), out=("out", b * T * E, E, h * hd),
                              nq=T, nk=T, hd=hd, scale=scale, mask="causal", seq=b))
    pairs = batch * H * (T * (T + 1) // 2)
    return Workload(name=name, buffers={"qkv": qkv.reshape(-1), "out": out.reshape(-1)}, heads=heads,
                    tokens=batch * T, flops=4.0 * hd * pairs, bytes=4.0 * (qkv.size + out.size),
                    meta=dict(batch=batch, T=T, H=H, hd=hd, E=E))


def config1(batch=1, T=512, H=4, hd=32):
    """Local-decoder causal byte self-attention."""
    return _packed_self_attention("c1_local_decoder_causal", 1, batch, T, H, hd)


def config2(batch=16, P=128, H=8, hd=64, T_bytes=512):
    """Patch-transformer block-causal attention over P patches."""
    w = _packed_self_attention("c2_patch_block_causal", 2, batch, P, H, hd)
    starts, lens = synth.patch_lengths(synth.seed_for(2, synth.S_PATCH), P, T_bytes)
    w.meta.update(patch_starts=starts, patch_lens=lens)
    return w


def offset_causal(batch=2, nq=100, nk=228, H=2, hd=32, causal_offset=None, window=0, seed_cfg=6):
    """Causal attention of nq new rows over nk keys (query i sees keys up to
    i + causal_offset, optionally only the last `window` of them): the shape of
    chunked prefill and sliding-window layers.  Separate Q / K / V buffers."""
    if causal_offset is None:
        causal_offset = nk - nq
    E = H * hd
    q = synth.normal(synth.seed_for(seed_cfg, synth.S_Q), (batch, nq, E))
    k = synth.normal(synth.seed_for(seed_cfg, synth.S_K), (batch, nk, E))
    v = synth.normal(synth.seed_for(seed_cfg, synth.S_V), (batch, nk, E))
    out = np.zeros((batch, nq, E), dtype=np.float32)
    scale = float(np.float32(1.0) / np.sqrt(np.float32(hd)))
    heads = []
    pairs = 0
    for b in range(batch):
        for h in range(H):
            heads.append(Head(q=("q", b * nq * E + h * hd, E), k=("k", b * nk * E + h * hd, E),
                              v=("v", b * nk * E + h * hd, E), out=("out", b * nq * E, E, h * hd),
                              nq=nq, nk=nk, hd=hd, scale=scale, mask="causal", causal_offset=causal_offset,
                              window=window, seq=b))
    for i in range(nq):
        hi = min(nk, i + causal_offset + 1)
        lo = max(0, i + causal_offset + 1 - window) if window else 0
        pairs += max(0, hi - lo)
    pairs *= batch * H
    return Workload(name="offset_causal", buffers={"q": q.reshape(-1), "k": k.reshape(-1), "v": v.reshape(-1),
                                                   "out": out.reshape(-1)}, heads=heads, tokens=batch * nq,
                    flops=4.0 * hd * pairs, bytes=4.0 * (q.size + k.size + v.size + out.size),
                    meta=dict(batch=batch, nq=nq, nk=nk, H=H, hd=hd, E=E))


def merged(name, parts):
    """One workload holding the heads of several (buffers renamed "<k>.<name>"): a
    batch whose problems differ in shape, as a caller that flattens layers produces."""
    import dataclasses
    buffers, ranges, heads, outputs = {}, {}, [], []
    tokens, flops, nbytes = 0, 0.0, 0.0
    for k, w in enumerate(parts):
        pre = "%d." % k
        buffers.update({pre + n: a for n, a in w.buffers.items()})
        ranges.update({pre + n: a for n, a in w.ranges.items()})
        outputs += [pre + n for n in w.outputs]
        for h in w.heads:
            ref = h.mask_ref
            if h.mask == "range":
                ref = (pre + ref[0], pre + ref[1], ref[2])
            elif h.mask == "dense":
                ref = (pre + ref[0], ref[1])
            heads.append(dataclasses.replace(h, q=(pre + h.q[0],) + tuple(h.q[1:]), k=(pre + h.k[0],) + tuple(h.k[1:]),
                                             v=(pre + h.v[0],) + tuple(h.v[1:]),
                                             out=(pre + h.out[0],) + tuple(h.out[1:]), mask_ref=ref))
        tokens += w.tokens
        flops += w.flops
        nbytes += w.bytes
    return Workload(name=name, buffers=buffers, ranges=ranges, heads=heads, outputs=tuple(outputs), tokens=tokens,
                    flops=flops, bytes=nbytes)


def config3(batch=16, T=512, P=128, H=4, hd=32):
    """Local-encoder cross-attention: patch queries over the bytes of their own patch."""
    E = H * hd
    q = synth.normal(synth.seed_for(3, synth.S_Q), (batch, P, E))
    k = synth.normal(synth.seed_for(3, synth.S_K), (batch, T, E))
    v = synth.normal(synth.seed_for(3, synth.S_V), (batch, T, E))
    out = np.zeros((batch, P, E), dtype=np.float32)
    lo = np.zeros((batch, P), dtype=np.uint32)
    hi = np.zeros((batch, P), dtype=np.uint32)
    patches = []
    for b in range(batch):
        starts, lens = synth.patch_lengths(synth.seed_for(3, synth.S_PATCH) + 0x10 * b, P, T)
        patches.append((starts, lens))
        lo[b] = starts
        hi[b] = starts + lens
    scale = float(np.float32(1.0) / np.sqrt(np.float32(hd)))
    heads = []
    for b in range(batch):
        for h in range(H):
            heads.append(Head(q=("q", b * P * E + h * hd, E), k=("k", b * T * E + h * hd, E),
                              v=("v", b * T * E + h * hd, E), out=("out", b * P * E, E, h * hd),
                              nq=P, nk=T, hd=hd, scale=scale, mask="range", mask_ref=("lo", "hi", b * P), seq=b))
    pairs = batch * H * T
    ids_bytes = batch * (T + P) * 8
    return Workload(name="c3_encoder_cross", buffers={"q": q.reshape(-1), "k": k.reshape(-1), "v": v.reshape(-1),
                                                      "out": out.reshape(-1)},
                    ranges={"lo": lo.reshape(-1), "hi": hi.reshape(-1)}, heads=heads, tokens=batch * P,
                    flops=4.0 * hd * pairs, bytes=4.0 * (q.size + k.size + v.size + out.size) + ids_bytes,
                    meta=dict(batch=batch, T=T, P=P, H=H, hd=hd, E=E, patches=patches))


@dataclass
class KvWorkload:
    """KV-cache step workload: `steps` consecutive calls, n new rows per sequence each."""
    name: str
    cache_k: np.ndarray      # [batch*max_seq_len, E]
    cache_v: np.ndarray
    lens: np.ndarray         # [batch] valid rows before the first step
    q_new: np.ndarray        # [steps, batch*n, E]
    k_new: np.ndarray
    v_new: np.ndarray
    n: int
    steps: int
    kind: str                # "causal" | "block"
    commit: bool
    batch: int
    max_seq_len: int
    H: int
    hd: int
    window: int = 0
    rope_cos: np.ndarray = None   # [max_seq_len, hd/2] rotation tables: q_new / k_new are un-rotated
    rope_sin: np.ndarray = None
    tokens: int = 0          # query rows per step
    flops: float = 0.0       # per step (first step)
    bytes: float = 0.0

    @property
    def E(self):
        return self.H * self.hd


def rope_tables(positions, hd, theta=500000.0):
    """cos / sin of pos / theta^(2i/hd), [positions, hd/2] fp32 (the quantities
    blt_rope_precompute tabulates; computed in float64 here and rounded once, so
    the values are inputs of a workload, not a restatement of that function)."""
    i = np.arange(hd // 2, dtype=np.float64)
    freq = 1.0 / np.power(np.float64(theta), 2.0 * i / hd)
    angle = np.arange(positions, dtype=np.float64)[:, None] * freq[None, :]
    return np.cos(angle).astype(np.float32), np.sin(angle).astype(np.float32)


def _fill_cache(cfg_id, batch, max_seq_len, E, lens, period=None):
    """`period`: generate that many sequences and repeat them over the batch (large
    bandwidth workloads, where drawing every value would dominate the run time)."""
    gen = batch if not period else min(batch, period)
    k = synth.normal(synth.seed_for(cfg_id, synth.S_K), (gen, max_seq_len, E))
    v = synth.normal(synth.seed_for(cfg_id, synth.S_V), (gen, max_seq_len, E))
    if gen < batch:
        reps = (batch + gen - 1) // gen
        k = np.tile(k, (reps, 1, 1))[:batch].copy()
        v = np.tile(v, (reps, 1, 1))[:batch].copy()
    # rows past the valid length hold stale data in the reference too; keep them
    # finite but recognisable so that a kernel reading them would be caught
    for b in range(batch):
        k[b, lens[b]:] = 1.0e3
        v[b, lens[b]:] = -1.0e3
    return k.reshape(batch * max_seq_len, E), v.reshape(batch * max_seq_len, E)


def config4(batch=64, steps=256, H=4, hd=32, len_lo=1, len_hi=512, max_seq_len=None, cache_period=None,
            rope=False):
    """KV-cache decode: one new byte per sequence and step, appended before attending."""
    E = H * hd
    if max_seq_len is None:
        max_seq_len = len_hi + steps
    lens = synth.integers(synth.seed_for(4, synth.S_LEN), batch, len_lo, len_hi).astype(np.uint32)
    ck, cv = _fill_cache(4, batch, max_seq_len, E, lens, cache_period)
    q_new = synth.normal(synth.seed_for(4, synth.S_NEWQ), (steps, batch, E))
    k_new = synth.normal(synth.seed_for(4, synth.S_NEWK), (steps, batch, E))
    v_new = synth.normal(synth.seed_for(4, synth.S_NEWV), (steps, batch, E))
    nk0 = lens.astype(np.int64) + 1
    rc, rs = rope_tables(max_seq_len, hd) if rope else (None, None)
    return KvWorkload(name="c4_kv_decode", cache_k=ck, cache_v=cv, lens=lens, q_new=q_new, k_new=k_new, v_new=v_new,
                      n=1, steps=steps, kind="causal", commit=True, batch=batch, max_seq_len=max_seq_len, H=H, hd=hd,
                      rope_cos=rc, rope_sin=rs, tokens=batch, flops=4.0 * hd * H * float(nk0.sum()),
                      bytes=4.0 * (2 * E * float(nk0.sum()) + batch * (E + E + 2 * E)))


def config5(batch=64, B=4, H=4, hd=32, len_lo=64, len_hi=508, max_seq_len=None, steps=1, cache_period=None,
            rope=False):
    """BLT-D/DV block verify: B query rows per sequence see the cached prefix and the whole block."""
    E = H * hd
    if max_seq_len is None:
        max_seq_len = 768
    assert len_hi + B <= max_seq_len
    lens = synth.integers(synth.seed_for(5, synth.S_LEN), batch, len_lo, len_hi).astype(np.uint32)
    ck, cv = _fill_cache(5, batch, max_seq_len, E, lens, cache_period)
    q_new = synth.normal(synth.seed_for(5, synth.S_NEWQ), (steps, batch * B, E))
    k_new = synth.normal(synth.seed_for(5, synth.S_NEWK), (steps, batch * B, E))
    v_new = synth.normal(synth.seed_for(5, synth.S_NEWV), (steps, batch * B, E))
    nk = lens.astype(np.int64) + B
    rc, rs = rope_tables(max_seq_len, hd) if rope else (None, None)
    return KvWorkload(name="c5_block_verify_B%d" % B, cache_k=ck, cache_v=cv, lens=lens, q_new=q_new, k_new=k_new,
                      v_new=v_new, n=B, steps=steps, kind="block", commit=False, batch=batch,
                      max_seq_len=max_seq_len, H=H, hd=hd, rope_cos=rc, rope_sin=rs, tokens=batch * B,
                      flops=4.0 * hd * H * B * float(nk.sum()),
                      bytes=4.0 * (2 * E * float(nk.sum()) + batch * B * 2 * E))
