"""Runs a workload through libfblt_hip.so with device buffers owned by torch.

torch is plumbing here: it allocates device memory and copies results back.
All compute goes through the C-ABI on the HIP null stream, so callers must not
switch torch to another stream around these calls.
"""
import ctypes as C

import numpy as np

from . import abi, api


def _torch():
    import torch
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU visible: the HIP attention backend has no CPU path")
    return torch


def sync():
    api.load().blt_backend_pass_sync_hip()


class DeviceWorkload:
    """Device-resident copy of a workloads.Workload plus problem builders."""

    def __init__(self, w):
        torch = _torch()
        self.w = w
        self.lib = api.load()
        self.dev = {n: torch.from_numpy(np.ascontiguousarray(a)).cuda() for n, a in w.buffers.items()}
        self.rng = {n: torch.from_numpy(a.astype(np.int32)).cuda() for n, a in w.ranges.items()}
        self._keep = []
        self.arena = None
        self._mask_cache = {}

    # ---- helpers -------------------------------------------------------
    def ptr(self, name, off=0):
        return self.dev[name].data_ptr() + 4 * off

    def zero_outputs(self):
        for n in self.w.outputs:
            self.dev[n].zero_()
        _torch().cuda.synchronize()

    def output(self, name="out"):
        _torch().cuda.synchronize()
        return self.dev[name].cpu().numpy()

    def _arena(self):
        if self.arena is None:
            self.arena = self.lib.blt_arena_create(256 << 20, abi.BLT_BACKEND_HIP)
        return self.arena

    def close(self):
        if self.arena is not None:
            self.lib.blt_backend_pass_sync_hip()
            self.lib.blt_arena_destroy(self.arena)
            self.arena = None

    def mask_config(self, h):
        """The blt_mask_config a reference caller would fill for head h's sequence (index arrays
        on the host, as the reference passes them): causal (+ offset, window) for the
        self-attention blocks (csrc/models/local_common.c:110, global_transformer.c:19-28), patch
        groups for the cross block (csrc/models/local_encoder.c:56-74)."""
        cfg = abi.BltMaskConfig()
        cfg.seq_len_q, cfg.seq_len_kv = h.nq, h.nk
        if h.mask == "causal":
            cfg.is_causal = True
            cfg.causal_offset = h.causal_offset
            cfg.sliding_window = h.window
        elif h.mask == "range":
            lo_name, hi_name, off = h.mask_ref
            lo = self.w.ranges[lo_name][off:off + h.nq]
            hi = self.w.ranges[hi_name][off:off + h.nq]
            kv = np.full(h.nk, h.nq, dtype=np.uint64)
            for i in range(h.nq):
                kv[lo[i]:hi[i]] = i
            qg, kg = abi.size_array(range(h.nq)), abi.size_array(kv)
            self._keep += [qg, kg]
            cfg.query_group_ids, cfg.kv_group_ids = qg, kg
            cfg.bidirectional_within_group = True
        else:
            raise ValueError(h.mask)
        return cfg

    def dense_mask_ptr(self, h):
        """Device address of the dense additive mask of head h, built by the
        device mask builder in the arena (the reference's flow)."""
        if h.mask == "none":
            return None
        if h.mask == "causal":
            key = ("causal", h.nq, h.nk, h.causal_offset, h.window)
        elif h.mask == "range":
            key = ("range", h.mask_ref, h.nq, h.nk)
        else:
            raise ValueError(h.mask)
        if key in self._mask_cache:
            return self._mask_cache[key]
        cfg = self.mask_config(h)
        t = abi.BltTensor()
        self.lib.blt_build_attention_mask_hip(C.byref(cfg), C.byref(t), self._arena())
        self._mask_cache[key] = t.data
        return t.data

    def head_args(self, h, mode, weights_ptr=None, lse_ptr=None, scratch_ptr=None):
        """mode: 'flag' (is_causal / no mask), 'dense' (device dense mask), 'none' (no mask fields)."""
        mask = None
        causal = False
        if mode == "dense":
            mask = self.dense_mask_ptr(h)
        elif mode == "flag":
            causal = h.mask == "causal"
        a = api.head_args(self.ptr(h.q[0], h.q[1]), self.ptr(h.k[0], h.k[1]), self.ptr(h.v[0], h.v[1]),
                          self.ptr(h.out[0], h.out[1]), h.nq, h.nk, h.hd, h.scale, h.q[2], h.k[2], h.v[2], h.out[2],
                          h.out[3], weights=weights_ptr, scratch=scratch_ptr, lse=lse_ptr, mask=mask, causal=causal)
        return a

    def problems(self, mask_mode="descriptor", weights_ptrs=None, lse_ptrs=None):
        """ctypes array of blt_attention_problem for every head.
        mask_mode: 'descriptor' (causal / row-range descriptors), 'dense', 'flag'."""
        probs = []
        for t, h in enumerate(self.w.heads):
            wp = None if weights_ptrs is None else weights_ptrs[t]
            lp = None if lse_ptrs is None else lse_ptrs[t]
            if mask_mode == "descriptor" and h.mask == "causal":
                a = self.head_args(h, "none", wp, lp)
                probs.append(api.problem(a, api.BLT_ATTN_MASK_CAUSAL, h.causal_offset, h.window))
            elif mask_mode == "descriptor" and h.mask == "range":
                a = self.head_args(h, "none", wp, lp)
                lo_name, hi_name, off = h.mask_ref
                probs.append(api.problem(a, api.BLT_ATTN_MASK_ROW_RANGE,
                                         row_lo=self.rng[lo_name].data_ptr() + 4 * off,
                                         row_hi=self.rng[hi_name].data_ptr() + 4 * off))
            else:
                a = self.head_args(h, "dense" if mask_mode == "dense" else "flag", wp, lp)
                probs.append(api.problem(a))
        return api.problem_array(probs)

    # ---- ways to run ---------------------------------------------------
    def run_per_head(self, mode="dense", with_weights=True):
        """The reference's caller loop: one blt_attention_head_core_hip call per head."""
        torch = _torch()
        max_scores = max(h.nq * h.nk for h in self.w.heads)
        buf = torch.empty(max_scores, dtype=torch.float32, device="cuda")
        for h in self.w.heads:
            a = self.head_args(h, mode, weights_ptr=buf.data_ptr() if with_weights else None,
                               scratch_ptr=None if with_weights else buf.data_ptr())
            self.lib.blt_attention_head_core_hip(abi.BLT_BACKEND_HIP, C.byref(a))
        self.lib.blt_backend_pass_sync_hip()

    def run_batch(self, mask_mode="descriptor"):
        arr = self.problems(mask_mode)
        self.lib.blt_attention_batch_hip(arr, len(self.w.heads))
        self.lib.blt_backend_pass_sync_hip()

    def make_plan(self, mask_mode="descriptor"):
        arr = self.problems(mask_mode)
        return self.lib.blt_attention_plan_create_hip(arr, len(self.w.heads))


class DeviceKvWorkload:
    """Device-resident KV-cache workload driving blt_kv_attend_step_hip, or
    blt_kv_rope_attend_step_hip when the workload carries rotation tables.  With
    lens="host" the lengths stay on the host (as the reference keeps them) and single-row
    steps go through blt_kv_attend_step_lens_hip; the device copy of the lengths is then
    not used."""

    def __init__(self, kw, lens="device"):
        torch = _torch()
        self.kw = kw
        self.lens_mode = lens
        self.host_lens = kw.lens.astype(np.uint32)  # the caller's own lengths (lens="host")
        self._host_lens_p = self.host_lens.ctypes.data_as(C.POINTER(C.c_uint32))
        self.lib = api.load()
        self.cache_k = torch.from_numpy(kw.cache_k).cuda()
        self.cache_v = torch.from_numpy(kw.cache_v).cuda()
        self.lens0 = torch.from_numpy(kw.lens.astype(np.int32)).cuda()
        self.lens = self.lens0.clone()
        self.q_new = torch.from_numpy(kw.q_new).cuda()
        self.k_new = torch.from_numpy(kw.k_new).cuda()
        self.v_new = torch.from_numpy(kw.v_new).cuda()
        self.rope = None
        if kw.rope_cos is not None:
            self.rope = (torch.from_numpy(kw.rope_cos).cuda(), torch.from_numpy(kw.rope_sin).cuda())
        self.out = torch.zeros((kw.steps, kw.batch * kw.n, kw.E), dtype=torch.float32, device="cuda")
        self.host_max_len = int(kw.lens.max())
        self.c = api.BltKvAttnCache()
        self.c.self_k = self.cache_k.data_ptr()
        self.c.self_v = self.cache_v.data_ptr()
        self.c.self_len = self.lens.data_ptr()
        self.c.batch, self.c.max_seq_len = kw.batch, kw.max_seq_len
        self.c.embed_dim, self.c.num_heads, self.c.window = kw.E, kw.H, kw.window
        self.kind = api.BLT_KV_STEP_CAUSAL if kw.kind == "causal" else api.BLT_KV_STEP_BLOCK
        # addresses of every step's rows, taken once: slicing a tensor per step costs more host
        # time than the step's launch
        self._rows = [tuple(t[s].data_ptr() for t in (self.q_new, self.k_new, self.v_new, self.out))
                      for s in range(kw.steps)]
        self._cache_ref = C.byref(self.c)
        self._rope_args = ((self.rope[0].data_ptr(), self.rope[1].data_ptr(), self.rope[0].shape[0])
                           if self.rope is not None else (None, None, 0))

    def reset(self):
        """Lengths back to the start; cache rows past them are dead by contract."""
        self.lens.copy_(self.lens0)
        self.host_max_len = int(self.kw.lens.max())
        self.host_lens[:] = self.kw.lens
        _torch().cuda.synchronize()

    def step(self, s):
        kw = self.kw
        E = kw.E
        hint = self.host_max_len + kw.n
        q, k, v, out = self._rows[s]
        cos, sin, rows = self._rope_args
        if self.lens_mode == "host":
            self.lib.blt_kv_attend_step_lens_hip(self._cache_ref, self._host_lens_p, q, E, k, E, v, E, cos, sin, rows,
                                                 out, E, kw.n, self.kind)
            if kw.commit:  # the caller advances its lengths, as the reference does after a step
                self.host_lens += np.uint32(kw.n)
        elif self.rope is not None:
            self.lib.blt_kv_rope_attend_step_hip(self._cache_ref, q, E, k, E, v, E, cos, sin, rows, out, E, kw.n,
                                                 self.kind, 1 if kw.commit else 0, hint)
        else:
            self.lib.blt_kv_attend_step_hip(self._cache_ref, q, E, k, E, v, E, out, E, kw.n, self.kind,
                                            1 if kw.commit else 0, hint)
        if kw.commit:
            self.host_max_len += kw.n

    def run(self, steps=None):
        steps = self.kw.steps if steps is None else steps
        for s in range(steps):
            self.step(s)
        self.lib.blt_backend_pass_sync_hip()

    def results(self):
        _torch().cuda.synchronize()
        lens = (self.host_lens.astype(np.int32) if self.lens_mode == "host"
                else self.lens.cpu().numpy())
        return self.out.cpu().numpy(), self.cache_k.cpu().numpy(), self.cache_v.cpu().numpy(), lens
