"""Runs a fixed list of attention cases through libfblt_hip.so and checks each
against the CPU checker.  Not collected by pytest: test_gpu_parity.py starts it
in a fresh process per kernel family, because the library reads the
BLT_HIP_ATTN_FAMILY hook once per process.

Tolerance: |got - ref| <= 1e-5 + 1e-4 * |ref| element-wise.
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from tests import lse_check  # noqa: E402
from fblt_amd import abi, api, runner, workloads  # noqa: E402
from oracle import binding, runner as orunner  # noqa: E402

def _nonfinite_keys():
    """Causal self-attention whose K holds a NaN, a +inf and a -inf: the scores against those
    keys are not finite and the reference drops such keys from the softmax."""
    w = workloads.config1(batch=1, T=160, H=2, hd=32)
    E = w.meta["E"]
    qkv = w.buffers["qkv"].reshape(160, 3 * E)
    qkv[5, E + 3] = np.nan
    qkv[70, E + 32] = np.inf
    qkv[100, E + 7] = -np.inf
    return w


CASES = {
    "nonfinite_keys": _nonfinite_keys,
    "c1_small": lambda: workloads.config1(batch=1, T=96, H=2, hd=32),
    "c1_ragged": lambda: workloads.config1(batch=2, T=77, H=2, hd=32),
    "c1_300": lambda: workloads.config1(batch=2, T=300, H=2, hd=64),
    "c1_129": lambda: workloads.config1(batch=3, T=129, H=1, hd=32),
    "c2_small": lambda: workloads.config2(batch=2, P=48, H=2, hd=64, T_bytes=192),
    "chunk_prefill": lambda: workloads.offset_causal(batch=2, nq=100, nk=228, H=2, hd=32),
    "window": lambda: workloads.offset_causal(batch=2, nq=200, nk=200, H=2, hd=64, window=40),
    "window_offset": lambda: workloads.offset_causal(batch=1, nq=150, nk=400, H=2, hd=32, window=70),
    "mixed_shapes": lambda: workloads.merged("mixed", [workloads.config1(batch=1, T=96, H=2, hd=32),
                                                       workloads.config1(batch=2, T=300, H=1, hd=32),
                                                       workloads.offset_causal(batch=1, nq=70, nk=200, H=3, hd=32)]),
    # short problems with a sliding window, with and without an offset of the diagonal
    "short_window": lambda: workloads.offset_causal(batch=2, nq=120, nk=120, H=2, hd=64, window=40),
    "short_window_offset": lambda: workloads.offset_causal(batch=2, nq=90, nk=250, H=2, hd=32, window=70),
    # 512 problems of 64 rows: more 32-row (and 16-row) tiles than the chip holds at once, in a
    # multiple that lets resident workgroups walk them
    "c2_many": lambda: workloads.config2(batch=64, P=64, H=8, hd=64, T_bytes=256),
    "c1_full": lambda: workloads.config1(),
    "c2_full": lambda: workloads.config2(),
}
ENTRIES = ("batch_descriptor", "batch_dense", "per_head_flag", "plan_lse")


def check(name, entry, got, ref):
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    bad = err > 1e-5 + 1e-4 * np.abs(ref)
    if bad.any():
        print("FAIL %s/%s: %d out of tolerance, max %.3e" % (name, entry, int(bad.sum()), float(err.max())))
        sys.exit(1)
    return float(err.max())


def main():
    import torch
    orc = binding.load_oracle()
    kernels = set()
    launched = set()  # names of the kernels the plans launched
    for name, make in CASES.items():
        w = make()
        orunner.run(w, lib=orc)
        ref = {n: w.buffers[n].copy() for n in w.outputs}
        for n in w.outputs:
            w.buffers[n][:] = 0
        d = runner.DeviceWorkload(w)
        try:
            for entry in ENTRIES:
                if entry == "per_head_flag" and any(h.causal_offset != 0 or h.window != 0 for h in w.heads):
                    continue  # the flag only describes plain causal problems
                print("case %s/%s" % (name, entry), flush=True)
                d.zero_outputs()
                if entry == "batch_descriptor":
                    d.run_batch("descriptor")
                elif entry == "batch_dense":
                    d.run_batch("dense")
                elif entry == "per_head_flag":
                    d.run_per_head("flag", with_weights=False)
                else:
                    lse = [torch.full((h.nq * 2,), 7.0, dtype=torch.float32, device="cuda") for h in w.heads]
                    arr = d.problems("descriptor", None, [t.data_ptr() for t in lse])
                    plan = d.lib.blt_attention_plan_create_hip(arr, len(w.heads))
                    kernels.add(d.lib.blt_attention_plan_kernel_hip(plan).decode())
                    d.lib.blt_hip_profile_begin()
                    d.lib.blt_attention_plan_run_hip(plan)
                    d.lib.blt_backend_pass_sync_hip()
                    launched.update(api.profile_end().keys())
                    d.lib.blt_attention_plan_destroy_hip(plan)
                    if name != "nonfinite_keys" and not name.endswith("_full") and name != "c2_many":
                        # the returned (max, sum) pairs rebuild the checker's weights
                        host_w = [np.zeros(h.nq * h.nk, dtype=np.float32) for h in w.heads]
                        keep = {n: w.buffers[n].copy() for n in w.outputs}
                        orunner.run(w, lib=orc, weights=host_w)
                        for n in w.outputs:
                            w.buffers[n][:] = keep[n]
                        cache = {}
                        lse_check.check_workload(w, [t.cpu().numpy() for t in lse], host_w,
                                                 lambda h: orunner._mask_for(orc, w, h, cache))
                    else:
                        for t in lse:
                            x = t.cpu().numpy().reshape(-1, 2)
                            assert np.isfinite(x).all() and (x[:, 1] >= 1.0 - 1e-4).all(), "lse"
                for n in w.outputs:
                    check(name, entry + ":" + n, d.output(n), ref[n])
        finally:
            d.close()
    print("case lse pairs, single-head calls", flush=True)
    lse_check.run_single_head_cases(api.load(), orc, api, abi, binding)
    print("KERNELS", ",".join(sorted(kernels)))
    print("LAUNCHED", ",".join(sorted(launched)))
    print("OK")


if __name__ == "__main__":
    main()
