"""Seeded synthetic inputs for the five attention workloads.

The reference ships no generator for per-op attention inputs, so this is the
build's own definition, shared by the parity tests and the benchmark so that
the GPU path and the CPU checker always see the same bytes:

* integers: splitmix64 (the recurrence the reference uses for its own test
  draws, csrc/infer/block_generation.c:12-18): state += 0x9E3779B97F4A7C15,
  then the usual two xor-shift-multiply rounds;
* N(0,1): two 24-bit uniforms per pair -> Box-Muller in float64 -> float32;
* patch lengths: geometric with mean 4 (`1 + floor(ln(1-u)/ln(3/4))`), clipped
  to 1..16, then repaired so that exactly P patches tile T bytes.

Everything is vectorised numpy on uint64; there is no Python-level loop over
elements.
"""
import numpy as np

GOLDEN = np.uint64(0x9E3779B97F4A7C15)
SEED_BASE = 0xB17D0000
STREAM_STRIDE = 0x1000
# sub-stream ids
S_Q, S_K, S_V, S_LEN, S_PATCH, S_NEWQ, S_NEWK, S_NEWV, S_REPAIR = range(9)


def seed_for(config_id, stream):
    return SEED_BASE + config_id + STREAM_STRIDE * (stream + 1)


def _mix(z):
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def splitmix64(seed, n):
    """First n outputs of splitmix64 started at `seed`, as uint64."""
    with np.errstate(over="ignore"):
        idx = np.arange(1, n + 1, dtype=np.uint64)
        return _mix(np.uint64(seed) + idx * GOLDEN)


def uniform24(seed, n):
    """n uniforms in [0,1) with 24 random bits each (top bits of each draw)."""
    return (splitmix64(seed, n) >> np.uint64(40)).astype(np.float64) / float(1 << 24)


def normal(seed, shape):
    """float32 N(0,1) of `shape`; element 2t and 2t+1 come from draw pair t."""
    n = int(np.prod(shape))
    pairs = (n + 1) // 2
    u = uniform24(seed, 2 * pairs)
    u1 = 1.0 - u[0::2]  # (0,1]
    u2 = u[1::2]
    r = np.sqrt(-2.0 * np.log(u1))
    out = np.empty(2 * pairs, dtype=np.float64)
    out[0::2] = r * np.cos(2.0 * np.pi * u2)
    out[1::2] = r * np.sin(2.0 * np.pi * u2)
    return out[:n].astype(np.float32).reshape(shape)


def integers(seed, n, lo, hi):
    """n integers uniform in [lo, hi] (inclusive) as int64: next() % range."""
    span = np.uint64(hi - lo + 1)
    return (splitmix64(seed, n) % span).astype(np.int64) + lo


def patch_lengths(seed, num_patches, seq_len, mean=4.0, lo=1, hi=16):
    """Geometric patch lengths repaired to tile [0, seq_len) with num_patches."""
    assert num_patches * lo <= seq_len <= num_patches * hi
    u = uniform24(seed, num_patches)
    p = 1.0 - 1.0 / mean
    lens = 1 + np.floor(np.log(1.0 - u) / np.log(p)).astype(np.int64)
    lens = np.clip(lens, lo, hi)
    # deterministic repair: walk a second stream of indices, nudging entries
    picks = splitmix64(seed + 0x777, 64 * num_patches + 4 * seq_len) % np.uint64(num_patches)
    total = int(lens.sum())
    t = 0
    while total != seq_len:
        i = int(picks[t % len(picks)])
        t += 1
        if total > seq_len and lens[i] > lo:
            lens[i] -= 1
            total -= 1
        elif total < seq_len and lens[i] < hi:
            lens[i] += 1
            total += 1
    starts = np.concatenate(([0], np.cumsum(lens)[:-1])).astype(np.int64)
    return starts, lens
