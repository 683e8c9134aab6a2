#!/usr/bin/env python3
"""Attention hot-path benchmark on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only c2]

A "step" is one pass of the headline workload -- the patch-transformer
block-causal attention (batch 16, 128 patches, 8 heads of 64, fp32) -- through
the HIP library: one resident plan, one kernel launch per step, inputs already
in HBM.  The last line on stdout is ONE compact JSON object (a few KB): the
whole-job throughput of that workload, the roofline figures of its kernel
(duration from HIP events attached to every launch of the timed region), the
CPU baseline (the reference's own attention core where its build travelled
with the tree, else the checker under oracle/; one host core, bounded sample),
the other two parts of the composite metric (decode us/step, verify tokens/s)
and one summary row per attention shape under "per_config".  The full
per-workload records go to stderr as they are measured and, together, to the
file --detail names.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix, published

TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.md")
DETAIL_FILE = os.path.join(ROOT, "gpurun_out", "bench_detail.json")


def measured_traffic():
    """{workload name: HBM bytes per launch} from the committed counter summary: one table row per
    workload holding the FETCH_SIZE and WRITE_SIZE readings (KiB per dispatch, `rocprofv3 --pmc`, one
    counter per run) and the factors the same counters read for a plain copy of known size.  An
    absent file or row gives no figure (traffic: null), never a stale constant."""
    out = {}
    try:
        with open(TRAFFIC_FILE) as f:
            for line in f:
                cells = [c.strip().strip("`") for c in line.strip().strip("|").split("|")]
                if len(cells) < 5 or cells[0] in ("workload", "") or set(cells[0]) <= set("-: "):
                    continue
                try:
                    fetch, ffac, write, wfac = (float(c) for c in cells[1:5])
                except ValueError:
                    continue
                out[cells[0]] = (fetch * ffac + write * wfac) * 1024.0
    except OSError:
        pass
    return out


MEASURED_TRAFFIC_BYTES = measured_traffic()


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def roofline(bound, work, avg_s, traffic=None):
    """work = algorithmic bytes (hbm) or flops (mfma) per launch."""
    if bound == "hbm":
        achieved, peak, unit = work / avg_s / 1e9, HBM_PEAK_GBS, "GB/s"
    else:
        achieved, peak, unit = work / avg_s / 1e12, FP32_MFMA_PEAK_TFLOPS, "TFLOP/s"
    return {"bound": bound, "achieved": achieved, "peak": peak, "unit": unit, "frac": achieved / peak,
            "traffic": traffic}


MIN_SAMPLES = 200   # event-timed launches behind every kernel duration, whatever --steps says
WARM_MS = 100.0     # back-to-back work before anything at the BASELINE sizes is timed, whatever --warmup says


def sample_stats(samples_us):
    """mean / p50 / p90 / p99 / min / max of per-step device times in us (nearest-rank percentiles)."""
    import numpy as np
    a = np.sort(np.array(samples_us, dtype=np.float64))
    pick = lambda q: float(a[min(len(a) - 1, int(q * len(a)))])
    return {"n": len(a), "mean": float(a.mean()), "p50": pick(0.50), "p90": pick(0.90), "p99": pick(0.99),
            "min": float(a[0]), "max": float(a[-1])}


def per_step_us(launch_ms, steps):
    """Per-launch durations (ms, issue order) of `steps` equal steps -> device us per step."""
    per = len(launch_ms) // steps if steps and len(launch_ms) % steps == 0 else 0
    if per <= 1:
        return [v * 1e3 for v in launch_ms]
    return [sum(launch_ms[i * per:(i + 1) * per]) * 1e3 for i in range(steps)]


def warm_up(lib, one_call, calls, warm_ms=0.0):
    """`calls` untimed calls, then more until `warm_ms` of back-to-back work has passed: kernels
    that keep the matrix cores busy for 100 us and more run about 15 % slower in the first tens of
    milliseconds after an idle spell than they do sustained (the clocks of an idle GPU ramp up
    under load), so the workloads sized to leave the launch floor are timed in the sustained state."""
    for _ in range(calls):
        one_call()
    lib.blt_backend_pass_sync_hip()
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < warm_ms:
        for _ in range(10):
            one_call()
        lib.blt_backend_pass_sync_hip()


def time_plan(lib, api, plan, steps, warmup, warm_ms=WARM_MS):
    """Warm-up (`warmup` launches, then by time), then two regions of back-to-back launches:
    exactly `steps` plain launches bracketed by device syncs (the whole-job wall time), and
    max(steps, MIN_SAMPLES) launches with a start / stop event pair attached to each (the kernel's
    own durations).  Returns (wall seconds of the plain region, {tag: (launches, total_ms, min,
    max)} of one launch, per-launch durations in ms of the event-timed region, its wall seconds)."""
    run = lambda: lib.blt_attention_plan_run_hip(plan)
    warm_up(lib, run, warmup, warm_ms)
    lib.blt_hip_profile_begin()
    run()
    tags = api.profile_end()
    lib.blt_backend_pass_sync_hip()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    lib.blt_backend_pass_sync_hip()
    wall_plain = time.perf_counter() - t0
    n = max(steps, MIN_SAMPLES)
    lib.blt_hip_profile_begin()
    t0 = time.perf_counter()
    for _ in range(n):
        run()
    lib.blt_backend_pass_sync_hip()
    wall_events = time.perf_counter() - t0
    return wall_plain, tags, api.profile_end_list(), wall_events


def bench_dense(make, steps, warmup, bound, mask_mode="descriptor", warm_ms=WARM_MS, caller_path=False):
    from fblt_amd import api, runner
    lib = api.load()
    w = make()
    d = runner.DeviceWorkload(w)
    plan = d.make_plan(mask_mode)
    kernel = lib.blt_attention_plan_kernel_hip(plan).decode()
    wall_plain, tags, launch_ms, wall_events = time_plan(lib, api, plan, steps, warmup, warm_ms)
    lib.blt_attention_plan_destroy_hip(plan)
    caller = bench_caller_path(w, d, steps, warmup) if caller_path else None
    d.close()
    per_launch = sum(v[0] for v in tags.values())          # launches of one step
    samples = per_step_us(launch_ms, len(launch_ms) // per_launch)
    pct = sample_stats(samples)
    avg_s = pct["mean"] * 1e-6                               # device time of one step (all its launches)
    res = {
        "workload": w.name, "kernel": kernel, "launches_per_step": per_launch,
        "tokens_per_step": w.tokens, "ms_per_step": wall_plain / steps * 1e3,
        "ms_per_step_with_events": wall_events / len(samples) * 1e3,
        "kernel_us_avg": pct["mean"], "kernel_us_p50": pct["p50"], "kernel_us_min": pct["min"],
        "kernel_us_samples": pct["n"], "kernel_us_percentiles": pct,
        "tokens_per_s": w.tokens * steps / wall_plain,
        "tokens_per_s_kernel": w.tokens / avg_s,
        "flops": w.flops, "bytes": w.bytes,
        "roofline_hbm": roofline("hbm", w.bytes, avg_s, MEASURED_TRAFFIC_BYTES.get(w.name)),
        "roofline_mfma": roofline("mfma", w.flops, avg_s),
    }
    res["warmup_ms"] = warm_ms
    if caller:
        res["reference_call_pattern"] = caller
    res["roofline"] = res["roofline_" + bound]
    return res, w


def bench_caller_path(w, d, steps, warmup):
    """The same workload the way an unmodified reference caller issues it on this library's ops
    (csrc/models/attention.c:92-128, 197-202; cross_attention.c:70-96, 145-150): per sequence one
    dense mask built on the device arena by blt_build_attention_mask, then one
    blt_attention_head_core call per head with that mask and weights_out set.  Device time = the
    launches' own durations summed; wall time includes this script's ctypes call overhead (a C
    caller pays less per call)."""
    import ctypes as C
    import torch
    from fblt_amd import abi, api
    lib = api.load()
    seqs = {}
    for h in w.heads:
        seqs.setdefault(h.seq, []).append(h)
    scores = torch.empty(max(h.nq * h.nk for h in w.heads), dtype=torch.float32, device="cuda")
    arena = lib.blt_arena_create(64 << 20, abi.BLT_BACKEND_HIP)
    plan = []
    for seq, heads in seqs.items():
        cfg = d.mask_config(heads[0])
        args = [d.head_args(h, "none", weights_ptr=scores.data_ptr()) for h in heads]
        plan.append((cfg, args))
    t = abi.BltTensor()

    def one_pass():
        for cfg, args in plan:
            arena.contents.offset = 0
            lib.blt_build_attention_mask(C.byref(cfg), C.byref(t), arena)
            for a in args:
                a.mask = t.data
                lib.blt_attention_head_core(abi.BLT_BACKEND_HIP, C.byref(a))
    n = max(10, steps // 10)
    warm_up(lib, one_pass, max(2, warmup // 4), WARM_MS / 2)
    lib.blt_hip_profile_begin()
    for _ in range(n):
        one_pass()
    prof = api.profile_end()
    t0 = time.perf_counter()
    for _ in range(n):
        one_pass()
    lib.blt_backend_pass_sync_hip()
    wall = time.perf_counter() - t0
    lib.blt_arena_destroy(arena)
    return {"entry": "blt_build_attention_mask + one blt_attention_head_core per (sequence, head), dense mask, weights_out",
            "launches_per_pass": sum(v[0] for v in prof.values()) / n,
            "kernel_us_per_pass": sum(v[1] for v in prof.values()) * 1e3 / n,
            "per_kernel_us": {k: v[1] * 1e3 / n for k, v in prof.items()},
            "wall_us_per_pass": wall / n * 1e6, "tokens_per_s": w.tokens * n / wall}


def bench_kv(kw, steps, warmup, warm_ms=0.0, lens="device"):
    """KV-cache workloads: `steps` consecutive step calls after `warmup` calls.  A
    committing workload (decode) appends one row per call and needs kw.steps >=
    warmup + steps; a non-committing one (verify) repeats its single step (and can be
    warmed by time, see warm_up).  lens="host": the caller keeps the lengths, as the
    reference does, and the steps go through blt_kv_attend_step_lens_hip."""
    from fblt_amd import api, runner
    lib = api.load()
    d = runner.DeviceKvWorkload(kw, lens=lens)
    idx = (lambda s: s) if kw.commit else (lambda s: 0)

    def one_pass(profiled, count=steps):
        """reset, `warmup` steps, then `count` timed steps; (wall seconds, per-launch ms or None)"""
        d.reset()
        for s in range(warmup):
            d.step(idx(s))
        lib.blt_backend_pass_sync_hip()
        if profiled:
            lib.blt_hip_profile_begin()
        t0 = time.perf_counter()
        for s in range(warmup, warmup + count):
            d.step(idx(s))
        lib.blt_backend_pass_sync_hip()
        wall = time.perf_counter() - t0
        return wall, (api.profile_end_list() if profiled else None)

    # warm by time: a non-committing step repeats; a committing workload repeats whole passes
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < max(warm_ms, WARM_MS):
        one_pass(False)
    d.reset()
    lib.blt_hip_profile_begin()
    d.step(idx(0))
    tags = api.profile_end()
    wall_plain, _ = one_pass(False)
    # a committing workload has exactly `steps` steps to time; a repeating one gives as many samples as asked
    timed = steps if kw.commit else max(steps, MIN_SAMPLES)
    wall, launch_ms = one_pass(True, timed)
    per_launch = sum(v[0] for v in tags.values())
    samples = per_step_us(launch_ms, len(launch_ms) // per_launch)
    pct = sample_stats(samples)
    avg_s = pct["mean"] * 1e-6
    # algorithmic work of an average timed step: lengths grow by n per committed step
    E, n = kw.E, kw.n
    base = float(kw.lens.astype("int64").sum())
    grown = kw.batch * n * (warmup + (steps - 1) / 2.0) if kw.commit else 0.0
    mean_keys = base + grown + kw.batch * n            # sum over sequences of keys attended
    rows = kw.batch * n
    # K and V of every attended key, plus Q in / O out per row, plus the appended K/V rows (decode)
    bytes_step = 4.0 * (2 * E * mean_keys + rows * 2 * E + (rows * 2 * E if kw.commit else 0))
    flops_step = 4.0 * kw.hd * kw.H * n * mean_keys
    res = {
        "workload": kw.name, "kernel": "+".join(sorted(tags)), "launches_per_step": per_launch,
        "tokens_per_step": kw.tokens, "us_per_step": wall_plain / steps * 1e6,
        "us_per_step_with_events": wall / timed * 1e6, "kernel_us_avg": pct["mean"], "kernel_us_p50": pct["p50"],
        "kernel_us_min": pct["min"], "kernel_us_samples": pct["n"], "kernel_us_percentiles": pct,
        "tokens_per_s": kw.tokens * steps / wall_plain, "tokens_per_s_kernel": kw.tokens / avg_s,
        "flops": flops_step, "bytes": bytes_step,
        "roofline_hbm": roofline("hbm", bytes_step, avg_s, MEASURED_TRAFFIC_BYTES.get(kw.name)),
        "roofline_mfma": roofline("mfma", flops_step, avg_s),
        "entry": ("blt_kv_attend_step_lens_hip (lengths on the host, carried in the kernel arguments)"
                  if lens == "host" else "blt_kv_attend_step_hip / blt_kv_rope_attend_step_hip (lengths in device memory)"),
    }
    res["warmup_ms"] = max(warm_ms, WARM_MS)
    res["roofline"] = res["roofline_hbm"]
    return res, kw


def bench_block(name, T, E, H, steps, warmup, gemm_only=None, cross=None, warm_ms=0.0, hidden=None):
    """blt_multihead_attention (projection, rotation, all heads, projection) on random
    device tensors; with gemm_only=(m, k, n) one blt_matmul of that shape; with cross=P
    blt_cross_attention_forward of P patches over T bytes (T / P bytes per patch); with
    hidden=h the whole blt_transformer_forward block (RMSNorm, attention, gated feed-forward of
    width h, residuals) under a document-causal mask."""
    import ctypes as C
    import numpy as np
    import torch
    from fblt_amd import abi, api
    lib = api.load()
    view = lambda t: abi.tensor_view(t.data_ptr(), tuple(t.shape), abi.BLT_BACKEND_HIP)
    g = torch.Generator(device="cpu").manual_seed(1234)
    rnd = lambda *shape: torch.randn(*shape, generator=g, dtype=torch.float32)
    keep = []
    if gemm_only:
        m, k, n = gemm_only
        a, b, o = rnd(m, k).cuda(), (rnd(k, n) / k ** 0.5).cuda(), torch.zeros((m, n), device="cuda")
        va, vb, vo = view(a), view(b), view(o)
        run = lambda: lib.blt_matmul(C.byref(va), C.byref(vb), C.byref(vo))
        flops, nbytes, tokens = 2.0 * m * k * n, 4.0 * (m * k + k * n + m * n), m
    elif cross:
        P = cross
        xq, xkv, o = rnd(P, E).cuda(), rnd(T, E).cuda(), torch.zeros((P, E), device="cuda")
        ws = [(rnd(E, E) / E ** 0.5).cuda() for _ in range(4)]
        arena = lib.blt_arena_create(256 << 20, abi.BLT_BACKEND_HIP)
        mc = abi.BltMaskConfig()
        mc.seq_len_q, mc.seq_len_kv = P, T
        qg, kg = abi.size_array(list(range(P))), abi.size_array([i // (T // P) for i in range(T)])
        mc.query_group_ids, mc.kv_group_ids, mc.bidirectional_within_group = qg, kg, True
        vws = [view(w) for w in ws]
        wts = abi.BltCrossAttentionWeights(*(C.pointer(v) for v in vws))
        cc = abi.BltCrossAttentionConfig()
        cc.embed_dim, cc.num_heads, cc.head_dim, cc.mask_config = E, H, E // H, C.pointer(mc)
        vq, vkv, vo = view(xq), view(xkv), view(o)
        keep += [mc, qg, kg, vws, wts, ws]

        def run():
            arena.contents.offset = 0
            lib.blt_cross_attention_forward(C.byref(vq), C.byref(vkv), C.byref(wts), C.byref(vo), C.byref(cc), arena)
        flops = 2.0 * E * E * (2 * P + 2 * T) + 4.0 * (E // H) * H * T
        nbytes = 4.0 * (P * E + T * E + 4 * E * E + P * E)
        tokens = T
    else:
        hd = E // H
        x, wq, wp = rnd(T, E).cuda(), (rnd(E, 3 * E) / E ** 0.5).cuda(), (rnd(E, E) / E ** 0.5).cuda()
        o = torch.zeros((T, E), device="cuda")
        arena = lib.blt_arena_create(256 << 20, abi.BLT_BACKEND_HIP)
        cos = torch.zeros((T, hd // 2), device="cuda")
        sin = torch.zeros((T, hd // 2), device="cuda")
        vc, vs = view(cos), view(sin)
        rcfg = abi.BltRopeConfig(500000.0, hd)
        lib.blt_rope_precompute(T, C.byref(rcfg), C.byref(vc), C.byref(vs))
        mc = abi.BltMaskConfig()
        mc.seq_len_q = mc.seq_len_kv = T
        mc.is_causal = True
        ac = abi.BltAttentionConfig()
        ac.embed_dim, ac.num_heads, ac.head_dim = E, H, hd
        ac.use_rope, ac.rope_theta = True, 500000.0
        ac.rope_cos_cache, ac.rope_sin_cache, ac.mask_config = C.pointer(vc), C.pointer(vs), C.pointer(mc)
        vx, vq, vp, vo = view(x), view(wq), view(wp), view(o)
        keep += [cos, sin, vc, vs, mc]

        def run():
            arena.contents.offset = 0
            lib.blt_multihead_attention(C.byref(vx), C.byref(vq), C.byref(vp), C.byref(vo), C.byref(ac), arena)
        pairs = H * (T * (T + 1) // 2)
        flops = 2.0 * T * E * 3 * E + 4.0 * hd * pairs + 2.0 * T * E * E
        nbytes = 4.0 * (T * E + 3 * E * E + E * E + T * E)
        tokens = T
        if hidden:
            docs = abi.size_array([T // 3, (2 * T) // 3])
            mc.doc_boundaries, mc.num_docs = docs, 3
            n1, n2 = torch.ones(E, device="cuda"), torch.ones(E, device="cuda")
            up, gate = (rnd(E, hidden) / E ** 0.5).cuda(), (rnd(E, hidden) / E ** 0.5).cuda()
            down = (rnd(hidden, E) / hidden ** 0.5).cuda()
            tv = [view(t) for t in (n1, wq, wp, n2, up, gate, down)]
            wt = abi.BltTransformerWeights()
            wt.norm1_weight, wt.attn_qkv_w, wt.attn_proj_w, wt.norm2_weight = (C.pointer(v) for v in tv[:4])
            wt.ffn_up_w, wt.ffn_gate_w, wt.ffn_down_w = (C.pointer(v) for v in tv[4:])
            tc = abi.BltTransformerConfig()
            tc.attn_config = ac
            tc.hidden_dim, tc.norm_type, tc.activation_type = hidden, abi.BLT_NORM_RMSNORM, abi.BLT_ACTIVATION_SWIGLU
            keep += [docs, n1, n2, up, gate, down, tv, wt]

            def run():
                arena.contents.offset = 0
                lib.blt_transformer_forward(C.byref(vx), C.byref(wt), C.byref(vo), C.byref(tc), arena)
            flops += 2.0 * T * E * hidden * 3
            nbytes += 4.0 * 3 * E * hidden
    warm_up(lib, run, warmup, warm_ms)
    lib.blt_hip_profile_begin()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    lib.blt_backend_pass_sync_hip()
    wall = time.perf_counter() - t0
    prof = api.profile_end()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    lib.blt_backend_pass_sync_hip()
    wall_plain = time.perf_counter() - t0
    if not gemm_only:
        lib.blt_arena_destroy(arena)
    avg_s = sum(v[1] for v in prof.values()) / 1e3 / steps
    res = {"workload": name, "kernel": "+".join(sorted(prof)), "launches_per_step": sum(v[0] for v in prof.values()) / steps,
           "tokens_per_step": tokens, "ms_per_step": wall_plain / steps * 1e3,
           "ms_per_step_with_events": wall / steps * 1e3, "kernel_us_avg": avg_s * 1e6,
           "kernel_us_min": min(v[2] for v in prof.values()) * 1e3,
           "per_kernel_us": {k: v[1] * 1e3 / steps for k, v in prof.items()},
           "tokens_per_s": tokens * steps / wall_plain, "tokens_per_s_kernel": tokens / avg_s, "flops": flops,
           "bytes": nbytes, "roofline_hbm": roofline("hbm", nbytes, avg_s), "roofline_mfma": roofline("mfma", flops, avg_s)}
    if warm_ms:
        res["warmup_ms"] = warm_ms
    res["roofline"] = res["roofline_mfma"]
    return res


def bench_masks(steps, warmup, cpu):
    """The device mask builders (blt_build_attention_mask / blt_build_block_diffusion_mask on a device
    arena) at the shapes their callers use, and one large fill; per call: the fill kernel(s) by
    events, the whole call by the host clock (it ends with the blocking read-back of the empty-row
    check).  Algorithmic bytes = the mask written once.  `cpu`: time the restated builder beside it."""
    import ctypes as C
    import numpy as np
    from fblt_amd import abi, api, synth
    lib = api.load()
    out = {}

    def group_ids(P, T):
        _, lens = synth.patch_lengths(synth.seed_for(3, synth.S_LEN), P, T)
        return np.repeat(np.arange(P), lens)

    cases = []
    c1 = abi.BltMaskConfig(); c1.seq_len_q = c1.seq_len_kv = 512; c1.is_causal = True
    cases.append(("mask_c1_causal_512", "attention", c1, None, 512 * 512))
    c3 = abi.BltMaskConfig(); c3.seq_len_q, c3.seq_len_kv = 128, 512
    qg, kg = abi.size_array(range(128)), abi.size_array(group_ids(128, 512).tolist())
    c3.query_group_ids, c3.kv_group_ids, c3.bidirectional_within_group = qg, kg, True
    cases.append(("mask_c3_patch_groups_128x512", "attention", c3, (qg, kg), 128 * 512))
    c5 = abi.BltBlockDiffusionConfig(); c5.mode, c5.seq_len, c5.num_clean = abi.BLT_BDM_INFER, 524, 508
    cases.append(("mask_c5_block_infer_524", "block", c5, None, 524 * 524))
    big = abi.BltMaskConfig(); big.seq_len_q = big.seq_len_kv = 4096; big.is_causal = True; big.sliding_window = 1024
    cases.append(("mask_causal_window_4096", "attention", big, None, 4096 * 4096))

    arena = lib.blt_arena_create(160 << 20, abi.BLT_BACKEND_HIP)
    mark = arena.contents.offset
    for name, kind, cfg, keep, cells in cases:
        t = abi.BltTensor()
        fn = lib.blt_build_attention_mask if kind == "attention" else lib.blt_build_block_diffusion_mask

        def run():
            arena.contents.offset = mark
            fn(C.byref(cfg), C.byref(t), arena)
        n = max(10, steps // 4)
        warm_up(lib, run, max(3, warmup // 4))
        lib.blt_hip_profile_begin()
        t0 = time.perf_counter()
        for _ in range(n):
            run()
        lib.blt_backend_pass_sync_hip()
        wall = time.perf_counter() - t0
        prof = api.profile_end()
        fill = {k: v for k, v in prof.items() if k != "mask_row_check"}
        avg_s = sum(v[1] for v in fill.values()) / 1e3 / n
        nbytes = 4.0 * cells
        res = {"workload": name, "kernel": "+".join(sorted(prof)), "launches_per_step": sum(v[0] for v in prof.values()) / n,
               "us_per_call": wall / n * 1e6, "kernel_us_avg": avg_s * 1e6,
               "per_kernel_us": {k: v[1] * 1e3 / n for k, v in prof.items()}, "bytes": nbytes,
               "roofline": roofline("hbm", nbytes, avg_s)}
        if cpu:
            from oracle import binding
            orc = binding.load_oracle()
            buf = np.empty(cells, dtype=np.float32)
            ofn = orc.orc_build_attention_mask if kind == "attention" else orc.orc_build_block_diffusion_mask
            reps, spent = 0, 0.0
            while reps < 1 or (spent < 1.0 and reps < 50):
                t0 = time.perf_counter()
                assert ofn(C.byref(cfg), binding.fptr(buf)) == 0
                spent += time.perf_counter() - t0
                reps += 1
            res["cpu_baseline"] = {"value": spent / reps * 1e6, "unit": "us/call", "cores": 1, "kind": "port",
                                   "sample": "%d calls, %.2f s" % (reps, spent)}
        out[name] = res
    lib.blt_arena_destroy(arena)
    return out


def bench_decode_layer(steps, warmup, batch=64, H=4, hd=32, hidden=512, len_hi=512):
    """blt_kv_decode_layer_hip: one decoder layer (self-attention block with fused RoPE and
    write-through, feed-forward block) for `batch` sequences, one new row each, per step."""
    import ctypes as C
    import numpy as np
    import torch
    from fblt_amd import abi, api, synth
    lib = api.load()
    E, half = H * hd, hd // 2
    total = warmup + steps
    max_len = len_hi + 2 * total + 2
    lens = synth.integers(synth.seed_for(4, synth.S_LEN), batch, 1, len_hi).astype(np.int32)
    g = torch.Generator(device="cpu").manual_seed(99)
    rnd = lambda *shape: torch.randn(*shape, generator=g, dtype=torch.float32)
    ck, cv = rnd(batch * max_len, E).cuda(), rnd(batch * max_len, E).cuda()
    Wt = {k: (rnd(*shape) / shape[0] ** 0.5).cuda() for k, shape in
          dict(qkv=(E, 3 * E), proj=(E, E), up=(E, hidden), gate=(E, hidden), down=(hidden, E)).items()}
    n1, n2 = torch.ones(E, device="cuda"), torch.ones(E, device="cuda")
    view = lambda t: abi.tensor_view(t.data_ptr(), tuple(t.shape), abi.BLT_BACKEND_HIP)
    views = {k: view(v) for k, v in Wt.items()}
    vn1, vn2 = view(n1), view(n2)
    w = abi.BltTransformerWeights()
    w.norm1_weight, w.norm2_weight = C.pointer(vn1), C.pointer(vn2)
    w.attn_qkv_w, w.attn_proj_w = C.pointer(views["qkv"]), C.pointer(views["proj"])
    w.ffn_up_w, w.ffn_gate_w, w.ffn_down_w = C.pointer(views["up"]), C.pointer(views["gate"]), C.pointer(views["down"])
    cos, sin = torch.zeros((max_len, half), device="cuda"), torch.zeros((max_len, half), device="cuda")
    vc, vs = view(cos), view(sin)
    rcfg = abi.BltRopeConfig(500000.0, hd)
    lib.blt_rope_precompute(max_len, C.byref(rcfg), C.byref(vc), C.byref(vs))
    tl0 = torch.from_numpy(lens).cuda()
    tl = tl0.clone()
    c = api.BltKvAttnCache()
    c.self_k, c.self_v, c.self_len = ck.data_ptr(), cv.data_ptr(), tl.data_ptr()
    c.batch, c.max_seq_len, c.embed_dim, c.num_heads, c.window = batch, max_len, E, H, 0
    x, o = rnd(batch, E).cuda(), torch.zeros((batch, E), device="cuda")
    arena = lib.blt_arena_create(64 << 20, abi.BLT_BACKEND_HIP)
    hint0 = int(lens.max())

    def run(count, first, commit=1):
        for s in range(count):
            arena.contents.offset = 0
            lib.blt_kv_decode_layer_hip(C.byref(c), C.byref(w), x.data_ptr(), o.data_ptr(), cos.data_ptr(),
                                        sin.data_ptr(), max_len, 1, api.BLT_KV_STEP_CAUSAL, commit,
                                        hint0 + first + s + 1, arena)
    run(warmup, 0)
    lib.blt_backend_pass_sync_hip()
    lib.blt_hip_profile_begin()
    t0 = time.perf_counter()
    run(steps, warmup)
    lib.blt_backend_pass_sync_hip()
    wall = time.perf_counter() - t0
    prof = api.profile_end()
    tl.copy_(tl0)
    torch.cuda.synchronize()
    run(warmup, 0)
    lib.blt_backend_pass_sync_hip()
    t0 = time.perf_counter()
    run(steps, warmup)
    lib.blt_backend_pass_sync_hip()
    wall_plain = time.perf_counter() - t0
    # the same layer step recorded once into a HIP graph (no commit: a replay repeats the step at
    # the lengths reached above) against the same step issued eagerly
    lib.blt_backend_pass_sync_hip()
    t0 = time.perf_counter()
    run(steps, warmup + steps - 1, commit=0)
    lib.blt_backend_pass_sync_hip()
    wall_eager_fixed = time.perf_counter() - t0
    per_graph = 6   # as many layer steps per graph as a 6-layer decoder issues per token
    lib.blt_hip_capture_begin()
    for _ in range(per_graph):
        run(1, warmup + steps - 1, commit=0)
    graph = lib.blt_hip_capture_end()
    for _ in range(warmup):
        lib.blt_hip_graph_launch(graph)
    lib.blt_backend_pass_sync_hip()
    replays = max(1, steps // per_graph)
    t0 = time.perf_counter()
    for _ in range(replays):
        lib.blt_hip_graph_launch(graph)
    lib.blt_backend_pass_sync_hip()
    wall_graph = (time.perf_counter() - t0) * steps / (replays * per_graph)
    lib.blt_hip_graph_destroy(graph)
    lib.blt_arena_destroy(arena)
    avg_s = sum(v[1] for v in prof.values()) / 1e3 / steps
    mean_keys = float(lens.astype("int64").sum()) + batch * (warmup + (steps - 1) / 2.0) + batch
    flops = batch * 2.0 * (E * 3 * E + E * E + 3 * E * hidden) + 4.0 * hd * H * mean_keys
    nbytes = 4.0 * (2 * E * mean_keys + 3 * E * E + E * E + 3 * E * hidden)
    res = {"workload": "decoder layer step: %d sequences, E=%d, H=%d, hidden=%d, cached 1..%d" % (batch, E, H, hidden, len_hi),
           "kernel": "+".join(sorted(prof)), "launches_per_step": sum(v[0] for v in prof.values()) / steps,
           "tokens_per_step": batch, "us_per_step": wall_plain / steps * 1e6,
           "us_per_step_fixed_length_eager": wall_eager_fixed / steps * 1e6,
           "us_per_step_fixed_length_graph_replay": wall_graph / steps * 1e6,   # 6 layer steps (30 kernels) per graph
           "us_per_step_with_events": wall / steps * 1e6, "kernel_us_avg": avg_s * 1e6,
           "kernel_us_min": min(v[2] for v in prof.values()) * 1e3,
           "per_kernel_us": {k: v[1] * 1e3 / steps for k, v in prof.items()},
           "tokens_per_s": batch * steps / wall_plain, "tokens_per_s_kernel": batch / avg_s, "flops": flops,
           "bytes": nbytes, "roofline_hbm": roofline("hbm", nbytes, avg_s), "roofline_mfma": roofline("mfma", flops, avg_s)}
    res["roofline"] = res["roofline_hbm"]
    return res


def cpu_decode_layer(budget_s, batch=64, H=4, hd=32, hidden=512, len_hi=512):
    """The restated decoder layer on one host core, one sequence at a time as the reference runs it."""
    import numpy as np
    from fblt_amd import synth
    from oracle import binding
    lib = binding.load_oracle()
    E, half = H * hd, hd // 2
    max_len = len_hi + 64
    rs = np.random.RandomState(5)
    lens = synth.integers(synth.seed_for(4, synth.S_LEN), batch, 1, len_hi)
    ck, cv = rs.randn(batch * max_len, E).astype(np.float32), rs.randn(batch * max_len, E).astype(np.float32)
    W = {k: (rs.randn(*shape) / np.sqrt(shape[0])).astype(np.float32) for k, shape in
         dict(qkv=(E, 3 * E), proj=(E, E), up=(E, hidden), gate=(E, hidden), down=(hidden, E)).items()}
    ones = np.ones(E, dtype=np.float32)
    cos, sin = np.empty(max_len * half, dtype=np.float32), np.empty(max_len * half, dtype=np.float32)
    lib.orc_rope_precompute(max_len, 500000.0, hd, binding.fptr(cos), binding.fptr(sin))
    x, o = rs.randn(batch, E).astype(np.float32), np.zeros((batch, E), dtype=np.float32)
    fp = lambda a: binding.fptr(a.reshape(-1))
    steps, spent = 0, 0.0
    while steps < 1 or (spent < budget_s and steps < 32):
        t0 = time.perf_counter()
        for b in range(batch):
            rc = lib.orc_kv_decode_layer(fp(ck), fp(cv), max_len, E, H, b, int(lens[b]) + steps, 1, 0, fp(ones),
                                         fp(W["qkv"]), fp(W["proj"]), fp(ones), fp(W["up"]), fp(W["gate"]),
                                         fp(W["down"]), hidden, fp(cos), fp(sin), max_len, fp(x[b:b + 1]),
                                         fp(o[b:b + 1]))
            assert rc == 0
        spent += time.perf_counter() - t0
        steps += 1
    return {"value": spent / steps * 1e6, "unit": "us/step", "cores": 1, "kind": "port",
            "sample": "%d layer steps of %d sequences, %.1f s" % (steps, batch, spent)}


def _decode_step_setup(batch, L, E, H, hidden, V, len_hi, total_steps, seed=17):
    """Seeded decoder weights, per-sequence lengths and patch tables (4 bytes per patch) of the
    batched decoder-step workload."""
    import numpy as np
    from fblt_amd import decoder, synth
    max_len = len_hi + total_steps + 8
    max_len += (-max_len) % 4
    lens = synth.integers(synth.seed_for(4, synth.S_LEN), batch, 1, len_hi).astype(np.int64)
    weights = decoder.random_weights(E, hidden, L, V, seed)
    tables = [decoder.patch_table([4] * (max_len // 4)) for _ in range(batch)]
    return max_len, lens, weights, tables


def bench_decode_step(steps, warmup, batch=64, L=2, E=128, H=4, hidden=512, V=256, len_hi=512, n=1):
    """blt_kv_decode_step_batched_hip: the whole incremental decoder step (per layer the cross block
    over the tier-2 cache and the self-attention / feed-forward layer, then the LM head) for `batch`
    sequences, one new row each, per step."""
    import ctypes as C
    import numpy as np
    import torch
    from fblt_amd import abi, api, decoder
    lib = api.load()
    hd, half = E // H, E // H // 2
    # n = 1: consecutive steps, the sequences grow; n > 1 (a prompt chunk): every call starts again from
    # the same cached lengths
    max_len, lens, weights, tables = _decode_step_setup(batch, L, E, H, hidden, V, len_hi,
                                                        2 * (warmup + steps) if n == 1 else n)
    view = lambda t: abi.tensor_view(t.data_ptr(), tuple(t.shape), abi.BLT_BACKEND_HIP)
    cos, sin = torch.zeros((max_len, half), device="cuda"), torch.zeros((max_len, half), device="cuda")
    vc, vs = view(cos), view(sin)
    rcfg = abi.BltRopeConfig(500000.0, hd)
    lib.blt_rope_precompute(max_len, C.byref(rcfg), C.byref(vc), C.byref(vs))
    bound = decoder.bind(weights, cos.cpu().numpy(), sin.cpu().numpy(), abi.BLT_BACKEND_HIP, decoder.device_place,
                         E, H, H, hidden, V, max_len)
    arena = lib.blt_arena_create(1 << 30, abi.BLT_BACKEND_HIP)
    cache = lib.blt_kv_cache_create_batched(arena, bound.ptr, max_len, batch)
    g = torch.Generator(device="cpu").manual_seed(7)
    P = max_len // 4
    for l in range(L):   # cached rows: random content, as after a prefill
        for name in ("self_k", "self_v"):
            t = torch.randn(batch * max_len, E, generator=g, dtype=torch.float32)
            lib.blt_hip_memcpy_h2d(getattr(cache.contents, name)[l].data, t.data_ptr(), t.numel() * 4)
            lib.blt_backend_pass_sync_hip()
    for b in range(batch):
        pin = torch.randn(P, E, generator=g, dtype=torch.float32).cuda()
        vp = view(pin)
        lib.blt_kv_cache_refresh_cross_seq_hip(cache, b, C.byref(vp), tables[b], P, 0, arena)
    lib.blt_backend_pass_sync_hip()
    mark = arena.contents.offset
    table_ptrs = (C.POINTER(abi.BltPatchInfo) * batch)(*(C.cast(t, C.POINTER(abi.BltPatchInfo)) for t in tables))
    num = abi.size_array([P] * batch)
    x = torch.randn(batch * n, E, generator=g, dtype=torch.float32).cuda()
    logits = torch.zeros((batch * n, V), device="cuda")
    vx, vl = view(x), view(logits)
    self_len = abi.size_array(lens.tolist())

    def run(count):
        for _ in range(count):
            arena.contents.offset = mark
            if n > 1:
                for b in range(batch):
                    self_len[b] = int(lens[b])
            lib.blt_kv_decode_step_batched_hip(cache, self_len, table_ptrs, num, None, C.byref(vx), C.byref(vl), arena)
    run(warmup)
    lib.blt_backend_pass_sync_hip()
    lib.blt_hip_profile_begin()
    t0 = time.perf_counter()
    run(steps)
    lib.blt_backend_pass_sync_hip()
    wall = time.perf_counter() - t0
    prof = api.profile_end()
    run(warmup)
    lib.blt_backend_pass_sync_hip()
    t0 = time.perf_counter()
    run(steps)
    lib.blt_backend_pass_sync_hip()
    wall_plain = time.perf_counter() - t0
    lib.blt_kv_cache_destroy(cache)
    lib.blt_arena_destroy(arena)
    avg_s = sum(v[1] for v in prof.values()) / 1e3 / steps
    rows = batch * n
    if n == 1:
        mean_keys = float(lens.sum()) + batch * (warmup + (steps - 1) / 2.0) + batch   # keys attended per step
        read_keys = mean_keys
    else:
        mean_keys = n * float(lens.sum()) + batch * n * (n + 1) / 2.0                  # (row, key) pairs per call
        read_keys = float(lens.sum()) + rows
    per_layer_w = E * E * 2 + E * 3 * E + E * E + 3 * E * hidden   # cross q / proj, qkv, proj, up / gate / down
    flops = L * (rows * 2.0 * per_layer_w + 4.0 * hd * H * mean_keys + 4.0 * E * rows) + rows * 2.0 * E * V
    nbytes = 4.0 * (L * (2 * E * read_keys + per_layer_w + 2 * E * rows) + E * V)
    res = {"workload": "decoder step: %d sequences x %d new rows, %d layers (cross block in each), E=%d, H=%d, "
                       "hidden=%d, V=%d, cached 1..%d" % (batch, n, L, E, H, hidden, V, len_hi),
           "kernel": "+".join(sorted(prof)), "launches_per_step": sum(v[0] for v in prof.values()) / steps,
           "tokens_per_step": rows, "us_per_step": wall_plain / steps * 1e6,
           "us_per_step_with_events": wall / steps * 1e6, "kernel_us_avg": avg_s * 1e6,
           "kernel_us_min": min(v[2] for v in prof.values()) * 1e3,
           "per_kernel_us": {k: v[1] * 1e3 / steps for k, v in prof.items()},
           "tokens_per_s": rows * steps / wall_plain, "tokens_per_s_kernel": rows / avg_s, "flops": flops,
           "bytes": nbytes, "roofline_hbm": roofline("hbm", nbytes, avg_s), "roofline_mfma": roofline("mfma", flops, avg_s)}
    res["roofline"] = res["roofline_hbm"]
    return res


def bench_encoder(steps, warmup, cpu_budget_s):
    """The local encoder's forward (csrc/models/local_encoder.c:193-281) at C3's caller size -- 512
    bytes in about 128 patches, E = 128, 4 heads, 2 layers with a cross block each, three hashed
    n-gram tables: this library's blt_local_encoder_forward, and the restated forward on one host
    core beside it."""
    import ctypes as C
    import numpy as np
    import torch
    from fblt_amd import abi, api, decoder, encoder
    lib = api.load()
    c = dict(T=512, E=128, H=4, XH=4, L=2, hidden=256, ngrams=(3, 4, 5), vocab=2048)
    rs = np.random.RandomState(31)
    lengths = []
    while sum(lengths) < c["T"]:
        lengths.append(int(min(c["T"] - sum(lengths), rs.poisson(3) + 1)))
    P = len(lengths)
    data = rs.randint(0, 256, size=c["T"]).astype(np.uint8)
    weights = encoder.random_weights(c["E"], c["hidden"], c["L"], c["ngrams"], c["vocab"], 37)
    hd = c["E"] // c["H"]
    view = lambda t, dt=abi.BLT_DTYPE_FP32: abi.tensor_view(t.data_ptr(), tuple(t.shape), abi.BLT_BACKEND_HIP, dtype=dt)
    cos, sin = torch.zeros((c["T"], hd // 2), device="cuda"), torch.zeros((c["T"], hd // 2), device="cuda")
    vc, vs = view(cos), view(sin)
    rcfg = abi.BltRopeConfig(500000.0, hd)
    lib.blt_rope_precompute(c["T"], C.byref(rcfg), C.byref(vc), C.byref(vs))
    tables = (cos.cpu().numpy(), sin.cpu().numpy())
    args = (c["E"], c["H"], c["XH"], c["hidden"], c["T"], c["ngrams"], c["vocab"], 1000003)
    dev = encoder.bind(weights, *tables, abi.BLT_BACKEND_HIP, decoder.device_place, *args)
    patches = decoder.patch_table(lengths)
    tbytes = torch.from_numpy(data).cuda()
    p_out, h_out = torch.zeros((P, c["E"]), device="cuda"), torch.zeros((c["T"], c["E"]), device="cuda")
    vb, vp, vh = view(tbytes, abi.BLT_DTYPE_UINT8), view(p_out), view(h_out)
    arena = lib.blt_arena_create(256 << 20, abi.BLT_BACKEND_HIP)

    def timed(entry):
        def run(count):
            for _ in range(count):
                arena.contents.offset = 0
                entry(dev.ptr, C.byref(vb), patches, P, None, 0, C.byref(vp), C.byref(vh), arena)
        run(warmup)
        lib.blt_backend_pass_sync_hip()
        lib.blt_hip_profile_begin()
        run(steps)
        lib.blt_backend_pass_sync_hip()
        prof = api.profile_end()
        t0 = time.perf_counter()
        run(steps)
        lib.blt_backend_pass_sync_hip()
        wall = (time.perf_counter() - t0) / steps
        return {"launches_per_pass": sum(v[0] for v in prof.values()) / steps,
                "kernel_us_per_pass": sum(v[1] for v in prof.values()) * 1e3 / steps, "wall_us_per_pass": wall * 1e6,
                "per_kernel_us": {k: v[1] * 1e3 / steps for k, v in prof.items()}}

    steps = max(10, steps // 5)
    mine = timed(lib.blt_local_encoder_forward)
    lib.blt_arena_destroy(arena)
    avg_s = mine["kernel_us_per_pass"] * 1e-6
    E, T, hidden, L = c["E"], c["T"], c["hidden"], c["L"]
    per_layer_w = E * 3 * E + E * E + 3 * E * hidden + 4 * E * E
    flops = L * (2.0 * T * (E * 3 * E + E * E + 3 * E * hidden) + 4.0 * hd * c["H"] * T * (T + 1) / 2 +
                 2.0 * (P * 2 * E * E + T * 2 * E * E) + 4.0 * E * T)
    nbytes = 4.0 * (L * (per_layer_w + 6 * T * E) + T * E * (1 + len(c["ngrams"])))
    res = {"workload": "local encoder forward: %d bytes, %d patches, %d layers (cross block in each), E=%d, H=%d, "
                       "hidden=%d, %d hashed n-gram tables" % (T, P, L, E, c["H"], hidden, len(c["ngrams"])),
           "entry": "blt_local_encoder_forward", "kernel": "+".join(sorted(mine["per_kernel_us"])),
           "launches_per_step": mine["launches_per_pass"], "tokens_per_step": T, "us_per_step": mine["wall_us_per_pass"],
           "kernel_us_avg": mine["kernel_us_per_pass"], "kernel_us_min": min(mine["per_kernel_us"].values()),
           "per_kernel_us": mine["per_kernel_us"], "tokens_per_s": T / (mine["wall_us_per_pass"] * 1e-6), "flops": flops,
           "bytes": nbytes, "roofline_hbm": roofline("hbm", nbytes, avg_s), "roofline_mfma": roofline("mfma", flops, avg_s)}
    res["roofline"] = res["roofline_mfma"]
    if cpu_budget_s > 0:
        from oracle import binding
        orc = binding.load_oracle()
        host = encoder.bind(weights, *tables, abi.BLT_BACKEND_CPU, decoder.host_place, *args)
        po, ho = np.zeros((P, E), dtype=np.float32), np.zeros((T, E), dtype=np.float32)
        t0, passes = time.perf_counter(), 0
        while passes == 0 or time.perf_counter() - t0 < cpu_budget_s:
            assert orc.orc_local_encoder_forward(host.ptr, data.ctypes.data_as(C.POINTER(C.c_uint8)), T, patches, P, None,
                                                 0, binding.fptr(po.reshape(-1)), binding.fptr(ho.reshape(-1))) == 0
            passes += 1
        dt = (time.perf_counter() - t0) / passes
        res["cpu_baseline"] = {"value": T / dt, "unit": "tokens/s", "cores": 1, "kind": "port",
                               "sample": "%d passes of the restated forward, %.1f s" % (passes, dt * passes),
                               "ms_per_pass": dt * 1e3}
    return res


def bench_decoder_forward(steps, warmup, cpu_budget_s, T=512, L=2, E=128, H=4, hidden=512, V=256):
    """The local decoder's plain forward in its inference form (csrc/models/local_decoder.c:233-351:
    D_0 = the encoder's rows, cross block and byte block per layer, LM head) at C1's caller size:
    this library's blt_local_decoder_forward_ext, and the restated forward on one host core."""
    import ctypes as C
    import numpy as np
    import torch
    from fblt_amd import abi, api, decoder
    lib = api.load()
    hd, half = E // H, E // H // 2
    rs = np.random.RandomState(41)
    lengths = []
    while sum(lengths) < T:
        lengths.append(int(min(T - sum(lengths), rs.poisson(3) + 1)))
    P = len(lengths)
    weights = decoder.random_weights(E, hidden, L, V, 43)
    view = lambda t: abi.tensor_view(t.data_ptr(), tuple(t.shape), abi.BLT_BACKEND_HIP)
    cos, sin = torch.zeros((T, half), device="cuda"), torch.zeros((T, half), device="cuda")
    vc, vs = view(cos), view(sin)
    rcfg = abi.BltRopeConfig(500000.0, hd)
    lib.blt_rope_precompute(T, C.byref(rcfg), C.byref(vc), C.byref(vs))
    tables = (cos.cpu().numpy(), sin.cpu().numpy())
    args = (E, H, H, hidden, V, T)
    dev = decoder.bind(weights, *tables, abi.BLT_BACKEND_HIP, decoder.device_place, *args)
    patches = decoder.patch_table(lengths)
    hidden_in = rs.randn(T, E).astype(np.float32)
    latents = rs.randn(P, E).astype(np.float32)
    th, tp = torch.from_numpy(hidden_in).cuda(), torch.from_numpy(latents).cuda()
    tl = torch.zeros((T, V), device="cuda")
    vh, vp, vl = view(th), view(tp), view(tl)
    arena = lib.blt_arena_create(256 << 20, abi.BLT_BACKEND_HIP)

    def run(count):
        for _ in range(count):
            arena.contents.offset = 0
            lib.blt_local_decoder_forward_ext(dev.ptr, C.byref(vh), C.byref(vp), patches, P, None, None, None, 0, None, 0,
                                              C.byref(vl), None, arena)
    steps = max(10, steps // 5)
    run(warmup)
    lib.blt_backend_pass_sync_hip()
    lib.blt_hip_profile_begin()
    run(steps)
    lib.blt_backend_pass_sync_hip()
    prof = api.profile_end()
    t0 = time.perf_counter()
    run(steps)
    lib.blt_backend_pass_sync_hip()
    wall = (time.perf_counter() - t0) / steps
    lib.blt_arena_destroy(arena)
    per_kernel = {k: v[1] * 1e3 / steps for k, v in prof.items()}
    kernel_us = sum(per_kernel.values())
    flops = L * (2.0 * T * (E * 3 * E + E * E + 3 * E * hidden) + 4.0 * E * T * (T + 1) / 2 +
                 2.0 * (T * 2 * E * E + P * 2 * E * E) + 4.0 * E * T) + 2.0 * T * E * V
    nbytes = 4.0 * (L * (E * 3 * E + E * E + 3 * E * hidden + 4 * E * E + 6 * T * E) + E * V + T * V)
    res = {"workload": "local decoder forward: %d bytes, %d patches, %d layers (cross block in each), E=%d, H=%d, "
                       "hidden=%d, V=%d" % (T, P, L, E, H, hidden, V),
           "entry": "blt_local_decoder_forward_ext", "kernel": "+".join(sorted(per_kernel)),
           "launches_per_step": sum(v[0] for v in prof.values()) / steps, "tokens_per_step": T, "us_per_step": wall * 1e6,
           "kernel_us_avg": kernel_us, "kernel_us_min": min(per_kernel.values()), "per_kernel_us": per_kernel,
           "tokens_per_s": T / wall, "flops": flops, "bytes": nbytes,
           "roofline_hbm": roofline("hbm", nbytes, kernel_us * 1e-6), "roofline_mfma": roofline("mfma", flops, kernel_us * 1e-6)}
    res["roofline"] = res["roofline_mfma"]
    if cpu_budget_s > 0:
        from oracle import binding
        orc = binding.load_oracle()
        host = decoder.bind(weights, *tables, abi.BLT_BACKEND_CPU, decoder.host_place, *args)
        out = np.zeros((T, V), dtype=np.float32)
        t0, passes = time.perf_counter(), 0
        while passes == 0 or time.perf_counter() - t0 < cpu_budget_s:
            assert orc.orc_local_decoder_forward(host.ptr, binding.fptr(hidden_in.reshape(-1)), T,
                                                 binding.fptr(latents.reshape(-1)), patches, P, None, 0, 0,
                                                 binding.fptr(out.reshape(-1))) == 0
            passes += 1
        dt = (time.perf_counter() - t0) / passes
        res["cpu_baseline"] = {"value": T / dt, "unit": "tokens/s", "cores": 1, "kind": "port",
                               "sample": "%d passes of the restated forward, %.1f s" % (passes, dt * passes),
                               "ms_per_pass": dt * 1e3}
    return res


def bench_draft_pass(steps, warmup, cpu_budget_s, N=400, B=8, L=2, E=128, H=4, hidden=512, V=256):
    """One denoising pass of the reference's draft loop (csrc/infer/block_generation.c:156-266: one
    sequence, N clean bytes, a block of B [MASK] rows on the last latent) three ways: the reference's
    call blt_local_decoder_forward_diffusion_infer (the whole [N + B] forward again on every pass),
    blt_kv_block_step_hip over a cache that holds the prefix (the block rows only), and the restated
    dense forward on one host core."""
    import ctypes as C
    import numpy as np
    import torch
    from fblt_amd import abi, api, decoder
    lib = api.load()
    hd, half = E // H, E // H // 2
    max_len = N + 32 + (-(N + 32)) % 4
    weights = decoder.random_weights(E, hidden, L, V, 23)
    view = lambda t: abi.tensor_view(t.data_ptr(), tuple(t.shape), abi.BLT_BACKEND_HIP)
    cos, sin = torch.zeros((max_len, half), device="cuda"), torch.zeros((max_len, half), device="cuda")
    vc, vs = view(cos), view(sin)
    rcfg = abi.BltRopeConfig(500000.0, hd)
    lib.blt_rope_precompute(max_len, C.byref(rcfg), C.byref(vc), C.byref(vs))
    tables = (cos.cpu().numpy(), sin.cpu().numpy())
    bound = decoder.bind(weights, *tables, abi.BLT_BACKEND_HIP, decoder.device_place, E, H, H, hidden, V, max_len)
    lengths = [4] * (N // 4)
    P = len(lengths)
    patches = decoder.patch_table(lengths)
    rs = np.random.RandomState(29)
    hidden_rows, latents = rs.randn(N, E).astype(np.float32), rs.randn(P, E).astype(np.float32)
    batch = decoder.BlockBatch(N, B, P)
    th, tp = torch.from_numpy(hidden_rows).cuda(), torch.from_numpy(latents).cuda()
    full, block = torch.zeros((N + B, V), device="cuda"), torch.zeros((B, V), device="cuda")
    vh, vp, vf, vb = view(th), view(tp), view(full), view(block)
    arena = lib.blt_arena_create(1 << 30, abi.BLT_BACKEND_HIP)
    cache = lib.blt_kv_cache_create(arena, bound.ptr, max_len)
    lib.blt_kv_cache_refresh_cross(cache, C.byref(vp), patches, P, 0, arena)
    prefix = torch.zeros((N, V), device="cuda")
    vpre = view(prefix)
    lib.blt_kv_decode_step(cache, C.byref(vp), patches, P, C.byref(vh), 1, C.byref(vpre), arena)
    lib.blt_backend_pass_sync_hip()
    mark = arena.contents.offset

    def timed(call):
        def run(count):
            for _ in range(count):
                arena.contents.offset = mark
                call()
        run(warmup)
        lib.blt_backend_pass_sync_hip()
        lib.blt_hip_profile_begin()
        run(steps)
        lib.blt_backend_pass_sync_hip()
        prof = api.profile_end()
        t0 = time.perf_counter()
        run(steps)
        lib.blt_backend_pass_sync_hip()
        wall = (time.perf_counter() - t0) / steps
        return {"launches_per_pass": sum(v[0] for v in prof.values()) / steps,
                "kernel_us_per_pass": sum(v[1] for v in prof.values()) * 1e3 / steps, "wall_us_per_pass": wall * 1e6,
                "per_kernel_us": {k: v[1] * 1e3 / steps for k, v in prof.items()}}

    dense = timed(lambda: lib.blt_local_decoder_forward_diffusion_infer(
        bound.ptr, C.byref(vh), C.byref(vp), patches, P, batch.ptr, abi.BLT_D0_LEARNED, C.byref(vf), arena))
    cached = timed(lambda: lib.blt_kv_block_step_hip(cache, P, batch.ptr, abi.BLT_D0_LEARNED, C.byref(vb), arena))
    lib.blt_backend_pass_sync_hip()
    agree = float((full[N:] - block).abs().max().item())
    lib.blt_kv_cache_destroy(cache)
    lib.blt_arena_destroy(arena)
    avg_s = cached["kernel_us_per_pass"] * 1e-6
    per_layer_w = E * E * 2 + E * 3 * E + E * E + 3 * E * hidden
    nbytes = 4.0 * (L * (2 * E * (N + B) + per_layer_w + 2 * E * B) + E * V)
    flops = L * (B * 2.0 * per_layer_w + 4.0 * hd * H * B * (N + B)) + B * 2.0 * E * V
    res = {"workload": "draft pass: 1 sequence, %d clean bytes, block of %d rows, %d layers (cross block in each), "
                       "E=%d, H=%d, hidden=%d, V=%d" % (N, B, L, E, H, hidden, V),
           "entry": "blt_kv_block_step_hip over the cached prefix",
           "kernel": "+".join(sorted(cached["per_kernel_us"])), "launches_per_step": cached["launches_per_pass"],
           "tokens_per_step": B, "us_per_step": cached["wall_us_per_pass"], "kernel_us_avg": cached["kernel_us_per_pass"],
           "kernel_us_min": min(cached["per_kernel_us"].values()), "per_kernel_us": cached["per_kernel_us"],
           "tokens_per_s": B / (cached["wall_us_per_pass"] * 1e-6), "flops": flops, "bytes": nbytes,
           "roofline_hbm": roofline("hbm", nbytes, avg_s), "roofline_mfma": roofline("mfma", flops, avg_s),
           "reference_call": dict(dense, entry="blt_local_decoder_forward_diffusion_infer (prefix recomputed per pass)"),
           "block_rows_max_abs_difference_between_the_two": agree}
    res["roofline"] = res["roofline_hbm"]
    if cpu_budget_s > 0:
        from oracle import binding
        orc = binding.load_oracle()
        host = decoder.bind(weights, *tables, abi.BLT_BACKEND_CPU, decoder.host_place, E, H, H, hidden, V, max_len)
        out = np.zeros((N + B, V), dtype=np.float32)
        fp = lambda a: binding.fptr(a.reshape(-1))
        t0, passes = time.perf_counter(), 0
        while passes == 0 or time.perf_counter() - t0 < cpu_budget_s:
            assert orc.orc_local_decoder_forward_diffusion_infer(host.ptr, fp(hidden_rows), fp(latents), patches, P,
                                                                 batch.ptr, abi.BLT_D0_LEARNED, fp(out)) == 0
            passes += 1
        dt = (time.perf_counter() - t0) / passes
        res["cpu_baseline"] = {"value": B / dt, "unit": "tokens/s", "cores": 1, "kind": "port",
                               "sample": "%d dense passes of the restated forward, %.1f s" % (passes, dt * passes),
                               "ms_per_pass": dt * 1e3}
    return res


def cpu_decode_step(budget_s, batch=64, L=2, E=128, H=4, hidden=512, V=256, len_hi=512, n=1):
    """The restated decoder step on one host core, one sequence at a time as the reference runs it."""
    import numpy as np
    from fblt_amd import abi, decoder
    from oracle import binding
    lib = binding.load_oracle()
    hd, half = E // H, E // H // 2
    max_len, lens, weights, tables = _decode_step_setup(batch, L, E, H, hidden, V, len_hi, 40 if n == 1 else n)
    cos, sin = np.empty(max_len * half, dtype=np.float32), np.empty(max_len * half, dtype=np.float32)
    lib.orc_rope_precompute(max_len, 500000.0, hd, binding.fptr(cos), binding.fptr(sin))
    bound = decoder.bind(weights, cos.reshape(max_len, half), sin.reshape(max_len, half), abi.BLT_BACKEND_CPU,
                         decoder.host_place, E, H, H, hidden, V, max_len)
    cache = decoder.HostCache(bound, max_len, batch)
    rs = np.random.RandomState(3)
    P = max_len // 4
    for name in ("self_k", "self_v"):
        for l in range(L):
            cache.tiers[name][l][:] = rs.randn(batch * max_len, E).astype(np.float32)
    for b in range(batch):
        pin = rs.randn(P, E).astype(np.float32)
        assert lib.orc_kv_cache_refresh_cross(cache.ptr, b, binding.fptr(pin.reshape(-1)), P, 0) == 0
    x, o = rs.randn(batch * n, E).astype(np.float32), np.zeros((batch * n, V), dtype=np.float32)
    fp = lambda a: binding.fptr(a.reshape(-1))
    steps, spent = 0, 0.0
    while steps < 1 or (spent < budget_s and steps < 16):
        t0 = time.perf_counter()
        for b in range(batch):
            base = int(lens[b]) + (steps if n == 1 else 0)
            assert lib.orc_kv_decode_step(cache.ptr, b, base, tables[b], P, fp(x[b * n:(b + 1) * n]), n, 0,
                                          fp(o[b * n:(b + 1) * n])) == 0
        spent += time.perf_counter() - t0
        steps += 1
    return {"value": spent / steps * 1e6, "unit": "us/step", "cores": 1, "kind": "port",
            "sample": "%d decoder steps of %d sequences, %.1f s" % (steps, batch, spent)}


def cpu_dense(w, budget_s):
    """One host core over the same workload; repeated whole passes up to the budget.  Through the
    reference's own attention core where its build is present (kind "reference"), else through the
    restatement (kind "port"); the two are bit-identical and compiled with the same flags."""
    from oracle import binding, runner as orunner
    lib = binding.load_oracle()
    ref = binding.load_ref()
    passes, spent = 0, 0.0
    while passes < 1 or (spent < budget_s and passes < 200):
        spent += orunner.run_ref(w, ref, lib=lib, timed=True) if ref else orunner.run(w, lib=lib, timed=True)
        passes += 1
    return {"value": w.tokens * passes / spent, "unit": "tokens/s", "cores": 1, "kind": "reference" if ref else "port",
            "sample": "%d full passes of %s, %.1f s, dense mask passed in, one core call per (sequence, head)"
                      % (passes, w.name, spent), "ms_per_pass": spent / passes * 1e3}


def _chunk_causal(kw):
    """The block-verify workload with causal rows: row r of a chunk sees the prefix and rows <= r."""
    import dataclasses
    n, E = kw.n, kw.E
    pairs = float(kw.lens.astype("int64").sum()) * n + kw.batch * n * (n + 1) / 2.0
    return dataclasses.replace(kw, name="c5_chunk_causal_n%d" % n, kind="causal",
                               flops=4.0 * kw.hd * kw.H * pairs)


def cpu_kv(kw, budget_s, max_steps):
    from oracle import binding, runner as orunner
    lib = binding.load_oracle()
    steps = 1
    out = orunner.run_kv(kw, lib=lib, steps=1, timed=True)
    per = out[3]
    steps = int(max(1, min(max_steps, budget_s / max(per, 1e-6))))
    out = orunner.run_kv(kw, lib=lib, steps=steps, timed=True)
    spent = out[3]
    return {"value": kw.tokens * steps / spent, "unit": "tokens/s", "cores": 1, "kind": "port",
            "sample": "first %d steps of %s, %.1f s, write-through then one core call per (sequence, head)"
                      % (steps, kw.name, spent), "us_per_step": spent / steps * 1e6}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--only", default="", help="comma list of c1,c2,c3,c4,c5 (c2 always runs)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU budget of the headline workload")
    ap.add_argument("--cpu-scale", type=float, default=1.0, help="scales the CPU budgets of the other workloads")
    ap.add_argument("--detail", default=DETAIL_FILE, help="file the full per-workload records are written to")
    ap.add_argument("--probe-copy-mib", type=int, default=0,
                    help="only run the plain streaming copy of this many MiB --steps times (counter yardstick)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (the workload shards by sequence "
                 "with no exchange step; run one process per GPU on its own sequences). Use --gpus 1.")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU: the HIP attention backend has no CPU path")
    from fblt_amd import workloads

    if args.probe_copy_mib:
        from fblt_amd import probes
        lib = probes.load()
        nbytes = args.probe_copy_mib << 20
        src = torch.ones(nbytes // 4, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            lib.blt_probe_stream_copy(dst.data_ptr(), src.data_ptr(), nbytes)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        print(json.dumps({"probe": "stream_copy", "bytes_in": nbytes, "bytes_out": nbytes, "launches": args.steps,
                          "GBps_read_plus_write": 2.0 * nbytes * args.steps / dt / 1e9}), flush=True)
        return

    only = set(x for x in args.only.split(",") if x)
    want = lambda c: not only or c in only
    K, W = args.steps, args.warmup
    cs = args.cpu_scale

    from fblt_amd import probes
    floor = _sig(probes.launch_floor(300))
    log("launch_floor", json.dumps(floor))
    head, w2 = bench_dense(workloads.config2, K, W, "hbm", caller_path=True)
    log("c2", json.dumps(head))
    others = {}
    if want("c1"):
        others["c1"], w1 = bench_dense(workloads.config1, K, W, "mfma", caller_path=True)
        log("c1", json.dumps(others["c1"]))
    if want("c3"):
        others["c3"], w3 = bench_dense(workloads.config3, K, W, "hbm", caller_path=True)
        log("c3", json.dumps(others["c3"]))
    if want("c4"):
        others["c4"], k4 = bench_kv(workloads.config4(steps=W + 256, max_seq_len=512 + W + 256), 256, W)
        log("c4", json.dumps(others["c4"]))
        # the same steps with the lengths where the reference keeps them (on the host)
        others["c4_host_lens"], _ = bench_kv(workloads.config4(steps=W + 256, max_seq_len=512 + W + 256), 256, W,
                                             lens="host")
        log("c4_host_lens", json.dumps(others["c4_host_lens"]))
        # the same steps with the rotation of the new Q/K rows fused in (un-rotated inputs + tables)
        others["c4_rope"], _ = bench_kv(workloads.config4(steps=W + 256, max_seq_len=512 + W + 256, rope=True), 256,
                                        W)
        others["c4_rope"]["workload"] = "c4_kv_decode + fused RoPE of new rows"
        log("c4_rope", json.dumps(others["c4_rope"]))
    if want("c5"):
        for B in (4, 8, 16):
            others["c5_B%d" % B], k5 = bench_kv(workloads.config5(B=B), K, W)
            log("c5_B%d" % B, json.dumps(others["c5_B%d" % B]))
            # the same block with the lengths where the reference keeps them (on the host,
            # csrc/infer/kv_cache.h:56-60; csrc/infer/block_generation.c:156-266)
            others["c5_B%d_host_lens" % B], _ = bench_kv(workloads.config5(B=B), K, W, lens="host")
            log("c5_B%d_host_lens" % B, json.dumps(others["c5_B%d_host_lens" % B]))
        # the sibling shape the reference's KV path really runs: a chunk-causal block of 16 new rows
        # over the cached prefix (a prefill chunk, kv_cache.c:229-236), not committed so that it repeats
        others["c5_chunk_causal_n16"], _ = bench_kv(_chunk_causal(workloads.config5(B=16)), K, W)
        others["c5_chunk_causal_n16"]["roofline_hbm"]["traffic"] = None
        log("c5_chunk_causal_n16", json.dumps(others["c5_chunk_causal_n16"]))
    # batch-swept prefill: the same kernels away from the launch floor
    if want("sweep"):
        for name, make in (("c1_x64", lambda: workloads.config1(batch=64)),
                           ("c2_x8", lambda: workloads.config2(batch=128)),
                           ("c1_T4096", lambda: workloads.config1(batch=8, T=4096)),
                           ("c2_P2048", lambda: workloads.config2(batch=8, P=2048, T_bytes=8192))):
            others[name], _ = bench_dense(make, max(10, K // 10), 3, "mfma", warm_ms=100.0)
            others[name]["roofline_hbm"]["traffic"] = None   # counters were read at the BASELINE sizes only
            log(name, json.dumps(others[name]))

        # decode and block verify with enough cached keys to leave the launch floor
        big = workloads.config4(batch=128, steps=3 + 20, len_lo=1024, len_hi=2048, max_seq_len=2048 + 32,
                               cache_period=8)
        others["c4_b128_L2048"], _ = bench_kv(big, 20, 3)
        others["c4_b128_L2048"]["roofline_hbm"]["traffic"] = None
        log("c4_b128_L2048", json.dumps(others["c4_b128_L2048"]))
        others["c4_b128_L2048_host_lens"], _ = bench_kv(big, 20, 3, lens="host")
        others["c4_b128_L2048_host_lens"]["roofline_hbm"]["traffic"] = None
        log("c4_b128_L2048_host_lens", json.dumps(others["c4_b128_L2048_host_lens"]))
        bigv = workloads.config5(batch=128, B=16, len_lo=1024, len_hi=2032, max_seq_len=2048, cache_period=8)
        others["c5_B16_b128_L2048"], _ = bench_kv(bigv, 20, 3, warm_ms=100.0)
        others["c5_B16_b128_L2048"]["roofline_hbm"]["traffic"] = None
        log("c5_B16_b128_L2048", json.dumps(others["c5_B16_b128_L2048"]))
        others["c5_B16_b128_L2048_host_lens"], _ = bench_kv(bigv, 20, 3, warm_ms=100.0, lens="host")
        others["c5_B16_b128_L2048_host_lens"]["roofline_hbm"]["traffic"] = None
        log("c5_B16_b128_L2048_host_lens", json.dumps(others["c5_B16_b128_L2048_host_lens"]))

    # the callers either side of the core: the whole attention block and its projection
    if want("block"):
        others["mha_c1"] = bench_block("blt_multihead_attention T=512 E=128 H=4 rope causal", 512, 128, 4, K, W)
        log("mha_c1", json.dumps(others["mha_c1"]))
        others["xattn_c3"] = bench_block("blt_cross_attention_forward P=128 T=512 E=128 H=4 patch mask", 512, 128, 4,
                                         K, W, cross=128)
        log("xattn_c3", json.dumps(others["xattn_c3"]))
        others["mha_c2"] = bench_block("blt_multihead_attention T=128 E=512 H=8 rope causal", 128, 512, 8, K, W)
        log("mha_c2", json.dumps(others["mha_c2"]))
        # a whole layer of the patch transformer (C2's caller once more removed) and of the local encoder
        others["layer_c2"] = bench_block("blt_transformer_forward T=128 E=512 H=8 hidden=2048 rope document-causal",
                                         128, 512, 8, K, W, hidden=2048)
        log("layer_c2", json.dumps(others["layer_c2"]))
        others["layer_c1"] = bench_block("blt_transformer_forward T=512 E=128 H=4 hidden=512 rope document-causal",
                                         512, 128, 4, K, W, hidden=512)
        log("layer_c1", json.dumps(others["layer_c1"]))
        others["matmul_8192x512x1536"] = bench_block("blt_matmul 8192x512x1536", 0, 0, 0, max(10, K // 10), 3,
                                                     gemm_only=(8192, 512, 1536), warm_ms=100.0)
        log("matmul", json.dumps(others["matmul_8192x512x1536"]))
        others["decode_layer"] = bench_decode_layer(K, W)
        if not args.no_cpu:
            others["decode_layer"]["cpu_baseline"] = cpu_decode_layer(2.0 * cs)
        log("decode_layer", json.dumps(others["decode_layer"]))
        others["decode_step"] = bench_decode_step(K, W)
        if not args.no_cpu:
            others["decode_step"]["cpu_baseline"] = cpu_decode_step(2.0 * cs)
        log("decode_step", json.dumps(others["decode_step"]))
        # the reference's own use of the step: one sequence, one new row per call
        others["decode_step_b1"] = bench_decode_step(K, W, batch=1)
        if not args.no_cpu:
            others["decode_step_b1"]["cpu_baseline"] = cpu_decode_step(2.0 * cs, batch=1)
        log("decode_step_b1", json.dumps(others["decode_step_b1"]))
        # a 512-byte prompt through the same entry point in one call (time to the first token)
        others["decode_step_prefill_512"] = bench_decode_step(max(10, K // 10), 3, batch=1, len_hi=1, n=512)
        if not args.no_cpu:
            others["decode_step_prefill_512"]["cpu_baseline"] = cpu_decode_step(2.0 * cs, batch=1, len_hi=1, n=512)
        log("decode_step_prefill_512", json.dumps(others["decode_step_prefill_512"]))
        # BLT-D drafting: one denoising pass over a 400-byte prefix, block of 8
        others["draft_pass"] = bench_draft_pass(K, W, 0.0 if args.no_cpu else 2.0 * cs)
        log("draft_pass", json.dumps(others["draft_pass"]))
        others["encoder"] = bench_encoder(K, W, 0.0 if args.no_cpu else 2.0 * cs)
        log("encoder", json.dumps(others["encoder"]))
        others["decoder_forward"] = bench_decoder_forward(K, W, 0.0 if args.no_cpu else 2.0 * cs)
        log("decoder_forward", json.dumps(others["decoder_forward"]))

    # the dense-mask builders the callers still use
    if want("masks"):
        for name, res in bench_masks(K, W, not args.no_cpu).items():
            others[name] = res
            log(name, json.dumps(res))

    cpu_head = None
    if not args.no_cpu:
        cpu_head = cpu_dense(w2, args.cpu_seconds)
        log("cpu c2", json.dumps(cpu_head))
        if want("c1"):
            others["c1"]["cpu_baseline"] = cpu_dense(w1, 2.0 * cs)
        if want("c3"):
            others["c3"]["cpu_baseline"] = cpu_dense(w3, 2.0 * cs)
        if want("c4"):
            others["c4"]["cpu_baseline"] = cpu_kv(workloads.config4(steps=64), 3.0 * cs, 64)
        if want("c5"):
            for B in (4, 8, 16):
                others["c5_B%d" % B]["cpu_baseline"] = cpu_kv(workloads.config5(B=B, steps=1), 1.0 * cs, 1)
            others["c5_chunk_causal_n16"]["cpu_baseline"] = cpu_kv(_chunk_causal(workloads.config5(B=16, steps=1)), 1.0 * cs, 1)

    head["cpu_baseline"] = cpu_head
    detail = dict(others)
    detail["c2"] = head
    detail_path = None
    try:
        os.makedirs(os.path.dirname(args.detail) or ".", exist_ok=True)
        with open(args.detail, "w") as f:
            json.dump({"steps": K, "warmup": W, "workloads": detail}, f, indent=1)
        detail_path = os.path.relpath(args.detail, ROOT)
    except OSError as e:
        log("detail file not written:", e)
    print(json.dumps(compact_line(head, others, cpu_head, K, W, detail_path, floor)), flush=True)


def _sig(x, digits=4):
    """Floats cut to a few significant digits: the summary line stays short."""
    if isinstance(x, float):
        return float("%.*g" % (digits, x))
    if isinstance(x, dict):
        return {k: _sig(v, digits) for k, v in x.items()}
    return x


def compact_line(head, others, cpu_head, K, W, detail_path, floor=None):
    """The one JSON object printed last on stdout: headline figures in full precision, one short
    summary row per attention shape (kernel, its device microseconds, fraction of the binding
    roofline, the reference call pattern beside it, CPU figure)."""
    def row(r):
        """kernel, device us per step (mean and median of the event samples), bound and fraction of its
        roofline, tokens/s; where measured: HBM traffic over algorithmic bytes, the reference's call pattern
        on this library's ops as [launches, device us, wall us] per pass, the CPU figure."""
        if r is None:
            return None
        c_dense = "reference_call_pattern" in r   # the dense configurations: tokens/s of the KV rows are lifted to the top
        o = {"kernel": r["kernel"][:24], "us": r["kernel_us_avg"], "p50": r.get("kernel_us_p50"),
             "bound": r["roofline"]["bound"], "frac": r["roofline"]["frac"]}
        if c_dense:
            o["tok_s"] = r["tokens_per_s"]
        if r["launches_per_step"] != 1:
            o["launches"] = r["launches_per_step"]
        if r.get("roofline_hbm", {}).get("traffic"):
            o["traffic_x"] = r["roofline_hbm"]["traffic"] / r["bytes"]   # measured HBM bytes over algorithmic bytes
        c = r.get("reference_call_pattern")
        if c:
            o["caller"] = [c["launches_per_pass"], _sig(c["kernel_us_per_pass"]), _sig(c["wall_us_per_pass"])]
        b = r.get("cpu_baseline")
        if b:
            o["cpu"] = [_sig(b["value"]), b["unit"]]
        return _sig(o)
    per = {"c2": row(head)}
    for k in ("c1", "c3", "c4", "c4_host_lens", "c4_rope", "c5_B4", "c5_B4_host_lens", "c5_B8", "c5_B8_host_lens",
              "c5_B16", "c5_B16_host_lens"):
        if k in others:
            per[k] = row(others[k])
    # the same kernels away from the launch floor: [kernel us, binding roofline, fraction of it]
    scaled = {k: [_sig(others[k]["kernel_us_avg"]), others[k]["roofline"]["bound"], _sig(others[k]["roofline"]["frac"])]
              for k in ("c1_x64", "c2_x8", "c1_T4096", "c2_P2048", "c4_b128_L2048", "c4_b128_L2048_host_lens",
                        "c5_B16_b128_L2048", "c5_B16_b128_L2048_host_lens") if k in others}
    return {
        "metric": "attn_tokens_per_s", "value": head["tokens_per_s"], "unit": "tokens/s",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "patch-transformer block-causal attention: batch 16, P=128 patches, 8 heads, "
                               "head_dim 64, fp32, seeded N(0,1) (BASELINE configs[1])",
                   "entry": "blt_attention_plan_run_hip, causal descriptor, one launch per step",
                   "kernel": head["kernel"], "tokens_per_step": head["tokens_per_step"]},
        "kernel_us_avg": head["kernel_us_avg"],
        "kernel_us_p50": head["kernel_us_percentiles"]["p50"],
        "kernel_us_samples": head["kernel_us_samples"],
        # an empty kernel timed the same way (events on the dispatch) and by the host clock back to back: an
        # event-timed duration includes dispatch overhead that overlaps the previous kernel in a back-to-back
        # loop, so kernel_us can exceed ms_per_step for kernels close to the floor
        "launch_floor": floor,
        "roofline": head["roofline"],
        "roofline_mfma": head["roofline_mfma"],
        "cpu_baseline": cpu_head,
        "cpu_cores": cpu_head["cores"] if cpu_head else None,
        # the other parts of the composite headline metric (decode us/step, verify tokens/s), when they ran
        # decode: wall microseconds per step of the 256 consecutive steps; the lengths on the host as in the
        # reference's blt_kv_decode_step (the device-length entry, which graphs can replay, is beside it)
        "decode_us_per_step": others["c4_host_lens"]["us_per_step"] if "c4_host_lens" in others else None,
        "decode_us_per_step_device_lens": others["c4"]["us_per_step"] if "c4" in others else None,
        # verify: query rows per second of the block step, lengths on the host as the reference keeps them
        "verify_tokens_per_s": {k[:-10]: others[k]["tokens_per_s"] for k in
                                ("c5_B4_host_lens", "c5_B8_host_lens", "c5_B16_host_lens") if k in others} or None,
        "per_config": per,
        "at_scale": scaled or None,
        "detail": detail_path,
    }


if __name__ == "__main__":
    main()
