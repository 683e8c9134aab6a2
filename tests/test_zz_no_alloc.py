"""blt_kv_attend_step_noalloc_hip against blt_kv_attend_step_hip: same arguments, same kernels, the
scratch in a fixed device array instead of allocated buffers.  Two calls in a row, the second with
a smaller input, each compared with the allocating entry point (outputs, cache rows and lengths
bit for bit: the kernels and their launch shapes are identical) and with the CPU checker (fp32
tolerance |got - ref| <= 1e-5 + 1e-4 |ref|; cache rows and lengths bit-exact)."""
import ctypes as C

import numpy as np
import pytest

from fblt_amd import api, workloads
from oracle import runner as orunner

pytestmark = pytest.mark.gpu


def _run(kw, entry):
    """All steps of a KV workload through `entry`; returns (out, cache_k, cache_v, lens)."""
    from fblt_amd import runner
    d = runner.DeviceKvWorkload(kw)
    fn = getattr(d.lib, entry)
    E = kw.E
    for s in range(kw.steps):
        fn(C.byref(d.c), d.q_new[s].data_ptr(), E, d.k_new[s].data_ptr(), E, d.v_new[s].data_ptr(), E,
           d.out[s].data_ptr(), E, kw.n, d.kind, 1 if kw.commit else 0, d.host_max_len + kw.n)
        if kw.commit:
            d.host_max_len += kw.n
    d.lib.blt_backend_pass_sync_hip()
    return d.results()


def _cases():
    # decode with the keys of a sequence split over workgroups (per-split records and tickets in use),
    # then a smaller decode, a block verify through the matrix-core kernel, and a long-prefix block
    # step whose keys are split over workgroups as well
    yield "decode_split", workloads.config4(batch=24, steps=4, len_lo=300, len_hi=700, max_seq_len=720)
    yield "decode_split_smaller", workloads.config4(batch=5, steps=3, len_lo=10, len_hi=200, max_seq_len=210)
    yield "c4_shape", workloads.config4(batch=64, steps=3)
    yield "block16", workloads.config5(batch=9, B=16)
    yield "block8_long_prefix", workloads.config5(batch=2, B=8, len_lo=2500, len_hi=3000, max_seq_len=3072)
    yield "block4_smaller", workloads.config5(batch=3, B=4)
    # 20 block rows at head width 16: the vector kernel in two launches of at most 16 rows that share the
    # fixed per-split records
    wide = workloads.config5(batch=4, B=20, H=4, hd=16, len_lo=600, len_hi=900, max_seq_len=1024)
    yield "block20_head16_two_launches", wide


def test_noalloc_entry_matches_the_allocating_one(oracle):
    for name, kw in _cases():
        ref_out, ref_k, ref_v = orunner.run_kv(kw, lib=oracle)
        got = _run(kw, "blt_kv_attend_step_noalloc_hip")
        want = _run(kw, "blt_kv_attend_step_hip")
        for g, w, what in zip(got, want, ("out", "cache_k", "cache_v", "lens")):
            assert g.tobytes() == w.tobytes(), "%s: %s differs from the allocating entry point" % (name, what)
        err = np.abs(got[0].astype(np.float64) - ref_out)
        assert (err <= 1e-5 + 1e-4 * np.abs(ref_out)).all(), "%s: max err %.3e" % (name, float(err.max()))
        assert got[1].tobytes() == ref_k.tobytes() and got[2].tobytes() == ref_v.tobytes(), name
        assert (got[3] == kw.lens.astype(np.int64) + (kw.steps * kw.n if kw.commit else 0)).all(), name


def test_noalloc_entry_replays_from_a_graph(oracle):
    """The entry's own use: recorded into a HIP graph (after one eager call, which looks up the fixed array's
    address) and replayed three times with eager work in between; every replay gives the allocating entry's bits."""
    import torch
    from fblt_amd import runner
    lib = api.load()
    kw = workloads.config4(batch=24, steps=1, len_lo=300, len_hi=700, max_seq_len=720)
    kw.commit = False
    want = _run(kw, "blt_kv_attend_step_hip")
    d = runner.DeviceKvWorkload(kw)
    E = kw.E

    def step():
        lib.blt_kv_attend_step_noalloc_hip(C.byref(d.c), d.q_new[0].data_ptr(), E, d.k_new[0].data_ptr(), E,
                                           d.v_new[0].data_ptr(), E, d.out[0].data_ptr(), E, kw.n, d.kind, 0,
                                           d.host_max_len + kw.n)
    step()
    lib.blt_backend_pass_sync_hip()
    lib.blt_hip_capture_begin()
    step()
    graph = lib.blt_hip_capture_end()
    other = workloads.config5(batch=3, B=4)
    for _ in range(3):
        d.out.zero_()
        torch.cuda.synchronize()
        lib.blt_hip_graph_launch(graph)
        lib.blt_backend_pass_sync_hip()
        got = d.results()
        for g, w, what in zip(got, want, ("out", "cache_k", "cache_v", "lens")):
            assert g.tobytes() == w.tobytes(), "replay: %s differs from the allocating entry point" % what
        _run(other, "blt_kv_attend_step_noalloc_hip")   # eager work on the same fixed array between replays
    lib.blt_hip_graph_destroy(graph)


def test_noalloc_entry_rejects_what_the_fixed_scratch_cannot_hold():
    """Beyond the fixed array's size the call ends with a message naming both figures (fatal: own process)."""
    import os
    import subprocess
    import sys
    code = r"""
import ctypes as C, sys
sys.path.insert(0, %r)
import torch
from fblt_amd import api
lib = api.load()
batch, E, H, L = 6000, 128, 4, 64
c = api.BltKvAttnCache()
k = torch.zeros((batch * L, E), device="cuda"); v = torch.zeros_like(k)
lens = torch.ones(batch, dtype=torch.int32, device="cuda")
c.self_k, c.self_v, c.self_len = k.data_ptr(), v.data_ptr(), lens.data_ptr()
c.batch, c.max_seq_len, c.embed_dim, c.num_heads, c.window = batch, L, E, H, 0
rows = torch.zeros((batch, E), device="cuda"); out = torch.zeros_like(rows)
lib.blt_kv_attend_step_noalloc_hip(C.byref(c), rows.data_ptr(), E, rows.data_ptr(), E, rows.data_ptr(), E,
                                   out.data_ptr(), E, 1, 0, 0, 2)
print("NOT REACHED")
""" % os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert p.returncode == 1 and "NOT REACHED" not in p.stdout, (p.returncode, p.stdout[-500:], p.stderr[-1500:])
    assert "fixed scratch holds" in p.stderr and "4096 sequences" in p.stderr, p.stderr[-1500:]
