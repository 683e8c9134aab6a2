"""Randomly shaped strided batches of attention problems through libfblt_hip.so, checked against the
CPU checker.  Not collected by pytest: test_gpu_parity.py starts it in a fresh process per kernel
family / workgroup shape, because the library reads its routing hooks once per process.

usage: random_cases.py SEED [SEED ...]

Shapes per seed: 1..5 sequences x 1..4 heads, head widths 32 / 64 (sometimes 16, 48, 128), 1..260
query rows (most of them at most 128), causal with a moved diagonal and an optional sliding window,
or every key visible.  Tolerance: |got - ref| <= 1e-5 + 1e-4 * |ref| element-wise.
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from fblt_amd import api, runner, workloads  # noqa: E402
from oracle import binding, runner as orunner  # noqa: E402


def random_workload(rs):
    batch, H = int(rs.randint(1, 6)), int(rs.randint(1, 5))
    hd = int(rs.choice([32, 64])) if rs.rand() < 0.8 else int(rs.choice([16, 48, 128]))
    nq = int(rs.randint(1, 129)) if rs.rand() < 0.7 else int(rs.randint(129, 261))
    causal = rs.rand() < 0.6
    if causal:
        extra = 0 if rs.rand() < 0.5 else int(rs.randint(1, 200))
        nk = nq + extra
        window = 0 if rs.rand() < 0.6 else int(rs.randint(1, nk + 1))
        w = workloads.offset_causal(batch=batch, nq=nq, nk=nk, H=H, hd=hd, window=window,
                                    seed_cfg=int(rs.randint(1, 1000)))
        what = "causal nq=%d nk=%d window=%d" % (nq, nk, window)
    else:
        nk = int(rs.randint(1, 301))
        w = workloads.offset_causal(batch=batch, nq=nq, nk=nk, H=H, hd=hd, causal_offset=0,
                                    seed_cfg=int(rs.randint(1, 1000)))
        for h in w.heads:
            h.mask, h.causal_offset, h.window = "none", 0, 0
        what = "all keys nq=%d nk=%d" % (nq, nk)
    return w, "%d x %d heads of %d, %s" % (batch, H, hd, what)


def main():
    orc = binding.load_oracle()
    launched = set()
    for seed in (int(a) for a in sys.argv[1:]):
        rs = np.random.RandomState(seed)
        for case in range(12):
            w, what = random_workload(rs)
            print("seed %d case %d: %s" % (seed, case, what), flush=True)
            orunner.run(w, lib=orc)
            ref = w.buffers["out"].copy()
            w.buffers["out"][:] = 0
            d = runner.DeviceWorkload(w)
            try:
                for entry in ("batch", "plan"):
                    d.zero_outputs()
                    if entry == "batch":
                        d.run_batch("descriptor")
                    else:
                        plan = d.make_plan("descriptor")
                        d.lib.blt_hip_profile_begin()
                        d.lib.blt_attention_plan_run_hip(plan)
                        d.lib.blt_backend_pass_sync_hip()
                        launched.update(api.profile_end().keys())
                        d.lib.blt_attention_plan_destroy_hip(plan)
                    got = d.output("out")
                    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
                    bad = err > 1e-5 + 1e-4 * np.abs(ref)
                    if bad.any():
                        print("FAIL seed %d case %d (%s) %s: %d out of tolerance, max %.3e" % (
                            seed, case, what, entry, int(bad.sum()), float(err.max())))
                        sys.exit(1)
            finally:
                d.close()
    print("LAUNCHED", ",".join(sorted(launched)))
    print("OK")


if __name__ == "__main__":
    main()
