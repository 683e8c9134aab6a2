"""Runs a fixed list of KV-cache step cases through blt_kv_attend_step_hip /
blt_kv_rope_attend_step_hip and checks each against the CPU checker.  Not
collected by pytest: test_gpu_parity.py starts it in a fresh process per
kernel (VALU or matrix-core), because the library reads BLT_HIP_BLOCK_KERNEL
once per process.

Outputs: |got - ref| <= 1e-5 + 1e-4 * |ref|; cache contents bit for bit.
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from fblt_amd import runner, workloads  # noqa: E402
from oracle import binding, runner as orunner  # noqa: E402


def chunked(n, rope, hd=32, window=0):
    """n new rows per sequence and step, causal within the chunk (prefill chunks)."""
    kw = workloads.config4(batch=9, steps=2, H=4 if hd == 32 else 2, hd=hd, len_hi=150, max_seq_len=150 + 2 * n,
                           rope=rope)
    rs = np.random.RandomState(n)
    kw.n = n
    kw.window = window
    kw.q_new, kw.k_new, kw.v_new = (rs.randn(kw.steps, kw.batch * n, kw.E).astype(np.float32) for _ in range(3))
    return kw


CASES = {
    "block4": lambda: workloads.config5(batch=9, B=4),
    "block16": lambda: workloads.config5(batch=9, B=16),
    "block32": lambda: workloads.config5(batch=9, B=32),
    "chunk3": lambda: chunked(3, False),
    "chunk12": lambda: chunked(12, False),
    "decode_rope": lambda: workloads.config4(batch=7, steps=4, len_hi=200, rope=True),
    "chunk3_rope": lambda: chunked(3, True),
    "chunk12_rope": lambda: chunked(12, True),
    "chunk20_rope_hd64": lambda: chunked(20, True, hd=64),
    "chunk6_rope_window": lambda: chunked(6, True, window=40),
    "chunk9_rope_hd64_window": lambda: chunked(9, True, hd=64, window=33),
    "chunk16": lambda: chunked(16, False),
    "chunk17": lambda: chunked(17, False),
    "chunk40_rope": lambda: chunked(40, True),                  # longer than one launch takes: 32 + 8 rows
    "chunk70_window_hd64": lambda: chunked(70, True, hd=64, window=50),
    "block8_rope": lambda: workloads.config5(batch=9, B=8, rope=True),
    "block16_rope_hd64": lambda: workloads.config5(batch=5, B=16, H=2, hd=64, rope=True),
    # the shapes around the all-at-once kernel's limits: caches of one or two rows (one cached tile and
    # the tile of new rows, four waves), a prefix of four tiles per wave, one past what it holds (the looping kernels
    # take over), a block of one row short of a tile at head width 64
    "block7_tiny_cache": lambda: workloads.config5(batch=6, B=7, len_lo=1, len_hi=2, max_seq_len=64),
    "block16_prefix_900": lambda: workloads.config5(batch=3, B=16, len_lo=700, len_hi=990, max_seq_len=1024),
    "block16_prefix_1100": lambda: workloads.config5(batch=3, B=16, len_lo=1000, len_hi=1100, max_seq_len=1200),
    "block15_hd64_prefix_400": lambda: workloads.config5(batch=4, B=15, H=2, hd=64, len_lo=100, len_hi=400, max_seq_len=512),
}


def main():
    orc = binding.load_oracle()
    for name, make in CASES.items():
        print("case", name, flush=True)
        kw = make()
        ref_out, ref_k, ref_v = orunner.run_kv(kw, lib=orc)
        d = runner.DeviceKvWorkload(kw)
        d.run()
        out, ck, cv, lens = d.results()
        if ck.tobytes() != ref_k.tobytes() or cv.tobytes() != ref_v.tobytes():
            print("FAIL %s: cache contents differ" % name)
            sys.exit(1)
        err = np.abs(out.astype(np.float64) - ref_out)
        if not (err <= 1e-5 + 1e-4 * np.abs(ref_out)).all():
            print("FAIL %s: max err %.3e" % (name, float(err.max())))
            sys.exit(1)
    print("OK")


if __name__ == "__main__":
    main()
