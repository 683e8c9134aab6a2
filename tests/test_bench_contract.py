"""The benchmark's command-line contract: one GPU only, one JSON line with the agreed fields."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused():
    p = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert p.returncode != 0
    assert "one GPU" in (p.stdout + p.stderr)


def _record(name, bound="hbm", caller=True):
    """A per-workload record shaped like the ones bench.py measures, with awkward float values."""
    roof = lambda b: {"bound": b, "achieved": 1234.56789012345, "peak": 8000.0 if b == "hbm" else 157.3,
                      "unit": "GB/s" if b == "hbm" else "TFLOP/s", "frac": 0.123456789012345, "traffic": 16936934.2976}
    r = {"workload": name, "kernel": "kv_block16_mfma+kv_step+splitk_pair_cross_epilogue", "launches_per_step": 15.0,
         "tokens_per_step": 2048, "ms_per_step": 0.0123456789, "us_per_step": 12.3456789, "kernel_us_avg": 9.87654321,
         "kernel_us_p50": 9.54321098, "kernel_us_samples": 200, "kernel_us_percentiles": {"n": 200, "mean": 9.87654321, "p50": 9.5, "p90": 10.1, "p99": 12.0, "min": 9.0,
                                   "max": 13.0},
         "tokens_per_s": 212345678.9012345, "flops": 2.705e8, "bytes": 16777216.0, "roofline_hbm": roof("hbm"),
         "roofline_mfma": roof("mfma"),
         "cpu_baseline": {"value": 33123.456789, "unit": "tokens/s", "cores": 1, "kind": "reference",
                          "sample": "3 full passes of %s, 12.1 s, dense mask passed in" % name}}
    r["roofline"] = r["roofline_" + bound]
    if caller:
        r["reference_call_pattern"] = {"launches_per_pass": 144.0, "kernel_us_per_pass": 1234.56789,
                                       "wall_us_per_pass": 2345.678901, "per_kernel_us": {}, "tokens_per_s": 1.0e6}
    return r


def test_summary_line_stays_short_with_every_workload_present():
    """The driver keeps a bounded tail of stdout: the line that carries metric, value, roofline and
    cpu_baseline must fit it with every workload of a full run present."""
    import bench
    names = ["c1", "c3", "c4", "c4_host_lens", "c4_b128_L2048_host_lens", "draft_pass", "c4_rope", "c5_B4", "c5_B8", "c5_B16", "c5_B4_host_lens", "c5_B8_host_lens",
             "c5_B16_host_lens", "c5_chunk_causal_n16", "c1_x64", "c2_x8",
             "c1_T4096", "c2_P2048", "c4_b128_L2048", "c5_B16_b128_L2048", "mha_c1", "xattn_c3", "mha_c2",
             "matmul_8192x512x1536", "decode_layer", "decode_step", "decode_step_b1", "decode_step_prefill_512",
             "mask_c1_causal_512", "mask_c3_patch_groups_128x512", "mask_c5_block_infer_524", "mask_causal_window_4096"]
    # as in a real run: only the dense configurations carry the reference call pattern, the host-length
    # twins of the KV rows carry no CPU leg of their own
    others = {n: _record(n, "mfma" if n.startswith("c1") else "hbm", caller=n in ("c1", "c3")) for n in names}
    for n in names:
        if n.endswith("host_lens") or n == "c4_rope":
            del others[n]["cpu_baseline"]
    head = _record("c2_patch_block_causal")
    floor = {"event_us_mean": 4.012, "event_us_median": 3.92, "back_to_back_wall_us": 2.213}
    line = json.dumps(bench.compact_line(head, others, head["cpu_baseline"], 200, 20, "gpurun_out/bench_detail.json",
                                         floor))
    assert len(line) < 4096, len(line)
    d = json.loads(line)
    for key in ("metric", "value", "unit", "ms_per_step", "roofline", "cpu_baseline", "decode_us_per_step",
                "verify_tokens_per_s", "per_config"):
        assert d[key] is not None, key
    assert set(d["per_config"]) >= {"c1", "c2", "c3", "c4", "c5_B4", "c5_B8", "c5_B16"}
    assert d["per_config"]["c1"]["caller"][0] == 144.0 and d["per_config"]["c1"]["us"] > 0
    assert d["launch_floor"]["event_us_mean"] > d["launch_floor"]["back_to_back_wall_us"]


def test_traffic_figures_come_from_the_committed_counter_summary():
    import bench
    t = bench.measured_traffic()
    assert set(t) >= {"c2_patch_block_causal", "c1_local_decoder_causal", "c3_encoder_cross", "c4_kv_decode",
                      "c5_block_verify_B4", "c5_block_verify_B8", "c5_block_verify_B16"}
    assert all(1e5 < v < 1e9 for v in t.values())


@pytest.mark.gpu
def test_one_json_line_with_the_agreed_fields(tmp_path):
    """A full default-shaped run (every workload, short CPU legs): stdout is one line under 4 KB."""
    p = subprocess.run([sys.executable, BENCH, "--steps", "20", "--warmup", "5", "--cpu-seconds", "0.5", "--cpu-scale",
                        "0.1", "--detail", str(tmp_path / "detail.json")], capture_output=True, text=True, timeout=900)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    assert len(lines[0]) < 4096, len(lines[0])
    d = json.loads(lines[0])
    detail = json.load(open(tmp_path / "detail.json"))
    assert set(detail["workloads"]) >= {"c1", "c2", "c3", "c4", "c5_B4", "c5_B8", "c5_B16", "decode_step"}
    assert d["decode_us_per_step"] > 0 and set(d["verify_tokens_per_s"]) == {"c5_B4", "c5_B8", "c5_B16"}
    for k in ("c1", "c2", "c3"):
        assert d["per_config"][k]["caller"][0] > d["per_config"][k].get("launches", 1)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 20 and d["warmup"] == 5 and d["vs_baseline"] is None
    assert d["dtype"] == "f32" and "workload" in d["config"] and d["higher_is_better"] is True
    r = d["roofline"]
    assert r["bound"] in ("hbm", "mfma") and r["unit"] in ("GB/s", "TFLOP/s")
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-9 and r["peak"] in (8000.0, 157.3)
    c = d["cpu_baseline"]
    assert c["kind"] in ("reference", "port") and c["cores"] == 1 and c["value"] > 0 and c["sample"]
    assert d["cpu_cores"] == 1
    assert d["value"] > 0 and d["ms_per_step"] > 0
