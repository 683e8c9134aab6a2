"""A KV step whose device-side lengths outgrew the host's hint.  Not collected by pytest:
test_gpu_parity.py runs it in a process of its own, because the library ends the process with the
reference's fatal error once it sees the device's error word.

    python kv_guard_case.py hint|slab|tables|graph

One sequence of the batch is one row longer than the launch (hint), its slab (max_seq_len) or the
rotation tables allow.  Expected: every kernel exits normally; that sequence is left alone (no
write-through, no output rows, length not advanced); the other sequences are computed as usual;
"CHECKED" is printed; the next synchronising library call prints "exceeds cache capacity" and
exits with status 1.

graph: the committing step is recorded into a HIP graph with a tight hint and replayed until one
sequence outgrows it -- the lengths advance on the device, the host issues nothing but graph
launches.  The replay that is still inside the hint passes its synchronisation quietly; the one
past it leaves that sequence alone and the next synchronising call is the same fatal error.
"""
import ctypes as C
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from fblt_amd import api, runner, workloads  # noqa: E402
from oracle import binding, runner as orunner  # noqa: E402


def graph_case():
    import torch
    over = 1
    kw = workloads.config4(batch=3, steps=1, len_lo=20, len_hi=100, max_seq_len=200)
    kw.lens[over] = 126
    hint = 128
    lib = api.load()
    d = runner.DeviceKvWorkload(kw)
    E = kw.E

    def step():
        lib.blt_kv_attend_step_hip(C.byref(d.c), d.q_new[0].data_ptr(), E, d.k_new[0].data_ptr(), E,
                                   d.v_new[0].data_ptr(), E, d.out[0].data_ptr(), E, 1, api.BLT_KV_STEP_CAUSAL, 1, hint)
    step()                              # eager: 126 -> 127, scratch gets allocated
    lib.blt_backend_pass_sync_hip()
    lib.blt_hip_capture_begin()
    step()
    graph = lib.blt_hip_capture_end()
    lib.blt_hip_graph_launch(graph)     # 127 -> 128: the last step the captured launch holds
    lib.blt_backend_pass_sync_hip()     # quiet
    assert int(d.lens.cpu().numpy()[over]) == 128
    print("REPLAY 1 QUIET", flush=True)
    sentinel = 123.0
    d.out.fill_(sentinel)
    torch.cuda.synchronize()
    before_k = d.cache_k.cpu().numpy().copy()
    lib.blt_hip_graph_launch(graph)     # 129 keys: past the hint
    torch.cuda.synchronize()            # not a library call: the error word is not looked at yet
    out, ck, lens = (t.cpu().numpy() for t in (d.out, d.cache_k, d.lens))
    assert int(lens[over]) == 128, lens
    assert (out[0, over] == sentinel).all()
    lo, hi = over * kw.max_seq_len, (over + 1) * kw.max_seq_len
    assert ck[lo:hi].tobytes() == before_k[lo:hi].tobytes()
    for b in (0, 2):                    # the others went on as usual
        assert int(lens[b]) == int(kw.lens[b]) + 3 and (out[0, b] != sentinel).any()
    print("CHECKED", flush=True)
    lib.blt_backend_pass_sync_hip()     # reads the error word: fatal
    print("NOT REACHED", flush=True)


def main():
    import torch
    mode = sys.argv[1]
    if mode == "graph":
        return graph_case()
    over = 1                      # the sequence that is too long
    if mode == "hint":            # 3 sequences, hint 128 -> the launch covers 2 splits x 64 keys
        kw = workloads.config4(batch=3, steps=1, len_lo=20, len_hi=100, max_seq_len=200)
        kw.lens[over] = 128
        hint = 128
    elif mode == "slab":          # the slab holds 100 rows and is full
        kw = workloads.config4(batch=3, steps=1, len_lo=20, len_hi=90, max_seq_len=100)
        kw.lens[over] = 100
        hint = 100
    else:                         # rotation tables one row short of the slab
        kw = workloads.config4(batch=3, steps=1, len_lo=20, len_hi=90, max_seq_len=128, rope=True)
        kw.rope_cos, kw.rope_sin = kw.rope_cos[:120].copy(), kw.rope_sin[:120].copy()
        kw.lens[over] = 120
        hint = 120
    lib = api.load()
    d = runner.DeviceKvWorkload(kw)
    sentinel = 123.0
    d.out.fill_(sentinel)
    E = kw.E
    if d.rope is not None:
        lib.blt_kv_rope_attend_step_hip(C.byref(d.c), d.q_new[0].data_ptr(), E, d.k_new[0].data_ptr(), E,
                                        d.v_new[0].data_ptr(), E, d.rope[0].data_ptr(), d.rope[1].data_ptr(),
                                        d.rope[0].shape[0], d.out[0].data_ptr(), E, 1, api.BLT_KV_STEP_CAUSAL, 1, hint)
    else:
        lib.blt_kv_attend_step_hip(C.byref(d.c), d.q_new[0].data_ptr(), E, d.k_new[0].data_ptr(), E,
                                   d.v_new[0].data_ptr(), E, d.out[0].data_ptr(), E, 1, api.BLT_KV_STEP_CAUSAL, 1, hint)
    torch.cuda.synchronize()      # not a library call: the error word is not looked at yet
    out, ck, cv, lens = (t.cpu().numpy() for t in (d.out, d.cache_k, d.cache_v, d.lens))
    # the over-long sequence: untouched
    assert int(lens[over]) == int(kw.lens[over]), lens
    assert (out[0, over] == sentinel).all()
    lo, hi = over * kw.max_seq_len, (over + 1) * kw.max_seq_len
    assert ck[lo:hi].tobytes() == kw.cache_k[lo:hi].tobytes() and cv[lo:hi].tobytes() == kw.cache_v[lo:hi].tobytes()
    if over + 1 < kw.batch:       # nothing was stored past its slab either
        assert ck[hi:hi + 1].tobytes() == kw.cache_k[hi:hi + 1].tobytes()
    # the others: as the checker computes them
    good = [b for b in range(kw.batch) if b != over]
    kw.lens[over] = 5             # any length the checker can run; its rows are not compared
    ref_out, ref_k, ref_v = orunner.run_kv(kw, lib=binding.load_oracle())
    for b in good:
        err = np.abs(out[0, b].astype(np.float64) - ref_out[0, b])
        assert (err <= 1e-5 + 1e-4 * np.abs(ref_out[0, b])).all(), (b, float(err.max()))
        lo, hi = b * kw.max_seq_len, (b + 1) * kw.max_seq_len
        assert ck[lo:hi].tobytes() == ref_k[lo:hi].tobytes() and cv[lo:hi].tobytes() == ref_v[lo:hi].tobytes()
        assert int(lens[b]) == int(kw.lens[b]) + 1
    print("CHECKED", flush=True)
    lib.blt_backend_pass_sync_hip()   # reads the error word: fatal
    print("NOT REACHED", flush=True)


if __name__ == "__main__":
    main()
