"""Golden vectors written by tests/golden/make_golden.py from the reference's
own CPU ops.  CPU: the checker must reproduce every output bit for bit
(SHA-256 of the full output).  GPU: the HIP library must match the stored
samples within the fp32 tolerance, and cache contents bit for bit."""
import hashlib
import os

import numpy as np
import pytest

from tests.golden.make_golden import DENSE_CASES, KV_CASES
from oracle import runner as orunner

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attention_golden.npz"))


def sha(arr):
    return np.frombuffer(hashlib.sha256(np.ascontiguousarray(arr).tobytes()).digest(), dtype=np.uint8)


def check_samples(arr, key, exact):
    flat = np.ascontiguousarray(arr).reshape(-1)
    assert flat.size == int(GOLD[key + "/size"][0])
    got, want = flat[GOLD[key + "/idx"]].astype(np.float64), GOLD[key + "/val"].astype(np.float64)
    if exact:
        assert (got == want).all()
    else:
        assert (np.abs(got - want) <= 1e-5 + 1e-4 * np.abs(want)).all(), float(np.abs(got - want).max())


@pytest.mark.parametrize("name", list(DENSE_CASES))
def test_oracle_reproduces_reference_dense(name, oracle):
    w = DENSE_CASES[name]()
    orunner.run(w, lib=oracle)
    assert (sha(w.buffers["out"]) == GOLD[name + "/out/sha256"]).all()
    check_samples(w.buffers["out"], name + "/out", exact=True)


@pytest.mark.parametrize("name", list(KV_CASES))
def test_oracle_reproduces_reference_kv(name, oracle):
    out, ck, cv = orunner.run_kv(KV_CASES[name](), lib=oracle)
    assert (sha(out) == GOLD[name + "/out/sha256"]).all()
    assert (sha(ck) == GOLD[name + "/cache_k/sha256"]).all()
    assert (sha(cv) == GOLD[name + "/cache_v/sha256"]).all()


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(DENSE_CASES))
@pytest.mark.parametrize("entry", ["per_head_dense", "plan"])
def test_hip_matches_reference_dense(name, entry):
    from fblt_amd import runner
    d = runner.DeviceWorkload(DENSE_CASES[name]())
    try:
        d.zero_outputs()
        if entry == "per_head_dense":
            d.run_per_head("dense", with_weights=True)
        else:
            plan = d.make_plan("descriptor")
            d.lib.blt_attention_plan_run_hip(plan)
            d.lib.blt_backend_pass_sync_hip()
            d.lib.blt_attention_plan_destroy_hip(plan)
        check_samples(d.output("out"), name + "/out", exact=False)
    finally:
        d.close()


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(KV_CASES))
def test_hip_matches_reference_kv(name):
    from fblt_amd import runner
    d = runner.DeviceKvWorkload(KV_CASES[name]())
    d.run()
    out, ck, cv, lens = d.results()
    check_samples(out, name + "/out", exact=False)
    assert (sha(ck) == GOLD[name + "/cache_k/sha256"]).all()   # slot indexing + write-through: bit-exact
    assert (sha(cv) == GOLD[name + "/cache_v/sha256"]).all()
