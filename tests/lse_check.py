"""Pins the (row max, row sum) pair the attention kernels return in lse_out.

Contract (csrc/ops/attn_core.h:35, csrc/ops/attn_core.cu:266-274): lse_out[i] =
(m_i, l_i) with m_i the maximum of x_ij = scale * dot(q_i, k_j) + mask_ij over
the row's finite entries in NATURAL units and l_i = sum_j exp(x_ij - m_i), so
that the post-softmax weights are exp(x_ij - m_i) / l_i.  A row without a
finite entry returns (-inf, 0).

The check rebuilds the weights from the returned pair and an independent
float64 evaluation of x, and compares them with the CPU checker's weights; it
also compares m with the float64 row maximum.  A maximum kept in another unit
(log2), a sum taken against another maximum, or swapped slots all fail it.

Shared by tests/test_gpu_parity.py and tests/family_cases.py; not collected.
"""
import ctypes as C

import numpy as np

ATOL, RTOL = 1e-5, 1e-4


def scores64(q, k, scale, mask=None, causal=False, causal_offset=0, window=0):
    """x[i, j] in float64 for 2-D q [nq, hd], k [nk, hd]; masked entries are -inf."""
    x = (q.astype(np.float64) @ k.astype(np.float64).T) * float(np.float32(scale))
    nq, nk = x.shape
    if mask is not None:
        x = x + mask.reshape(nq, nk).astype(np.float64)
    elif causal:
        i = np.arange(nq)[:, None] + causal_offset
        j = np.arange(nk)[None, :]
        dead = j > i
        if window:
            dead |= (i - j) >= window
        x = np.where(dead, -np.inf, x)
    return x


def check_pair(lse, x, ref_weights, what):
    """lse [nq, 2] from the device, x [nq, nk] float64 scores, ref_weights [nq, nk] from the checker."""
    lse = np.asarray(lse, dtype=np.float64).reshape(-1, 2)
    nq, nk = x.shape
    assert lse.shape[0] == nq, what
    finite = np.isfinite(x)
    alive = finite.any(axis=1)
    m, l = lse[:, 0], lse[:, 1]
    # rows without a finite entry
    assert (m[~alive] == -np.inf).all() and (l[~alive] == 0).all(), "%s: dead rows must return (-inf, 0)" % what
    if not alive.any():
        return
    xmax = np.where(finite, x, -np.inf).max(axis=1)
    err = np.abs(m[alive] - xmax[alive])
    assert (err <= ATOL + RTOL * np.abs(xmax[alive])).all(), "%s: row maximum off by %.3e (natural units expected)" % (
        what, float(err.max()))
    assert (l[alive] >= 1.0 - 1e-4).all() and np.isfinite(l[alive]).all(), "%s: row sum" % what
    with np.errstate(invalid="ignore", over="ignore"):
        rebuilt = np.where(finite & alive[:, None], np.exp(x - m[:, None]) / l[:, None], 0.0)
    ref = np.asarray(ref_weights, dtype=np.float64).reshape(nq, nk)
    bad = np.abs(rebuilt - ref) > ATOL + RTOL * np.abs(ref)
    assert not bad.any(), "%s: weights rebuilt from (m, l) differ from the checker's: %d cells, max %.3e" % (
        what, int(bad.sum()), float(np.abs(rebuilt - ref).max()))


def head_views(w, h):
    """2-D float32 views (q [nq, hd], k [nk, hd]) of one head of a workloads.Workload."""
    def rows(spec, n):
        buf, off, stride = w.buffers[spec[0]], spec[1], spec[2]
        idx = off + np.arange(n)[:, None] * stride + np.arange(h.hd)[None, :]
        return buf[idx]
    return rows(h.q, h.nq), rows(h.k, h.nk)


def check_workload(w, lse_per_head, weights_per_head, mask_of):
    """Every head of a workload: mask_of(h) returns the dense additive mask [nq*nk] or None."""
    for t, h in enumerate(w.heads):
        q, k = head_views(w, h)
        mask = mask_of(h)
        x = scores64(q, k, h.scale, mask=mask)
        check_pair(lse_per_head[t], x, weights_per_head[t], "%s head %d" % (w.name, t))


def single_head_cases():
    """(name, nq, nk, hd, kind) of per-head calls that exercise dead rows, additive biases and the
    causal flag at sizes each kernel family takes."""
    return [("dense_dead_rows", 70, 130, 32, "dense"), ("dense_bias", 37, 70, 64, "bias"),
            ("causal_flag", 96, 96, 32, "causal"), ("no_mask", 33, 200, 64, "none"),
            ("small_rows", 3, 40, 32, "dense"), ("wide_dense", 160, 256, 64, "dense")]


def run_single_head_cases(lib, oracle, api, abi, binding):
    """Runs the cases through blt_attention_head_core_hip with lse_out only (the output mode the
    reference's BLT_FLASH_ATTN switch uses, csrc/models/attention.c:111-119) and with lse_out +
    weights_out; checks both against the checker."""
    import torch
    for name, nq, nk, hd, kind in single_head_cases():
        rs = np.random.RandomState(len(name) * 131 + nq)
        q, k, v = (rs.randn(n, hd).astype(np.float32) for n in (nq, nk, nk))
        scale = float(np.float32(1.0) / np.sqrt(np.float32(hd)))
        mask = None
        if kind in ("dense", "bias"):
            mask = np.where(rs.rand(nq, nk) < 0.45, -np.inf, 0.0).astype(np.float32)
            if kind == "bias":
                mask = np.where(np.isfinite(mask), (rs.randn(nq, nk) * 2).astype(np.float32), mask).astype(np.float32)
            mask[0, :] = -np.inf
            mask[nq - 1, :] = -np.inf
        out_ref = np.zeros((nq, hd), dtype=np.float32)
        w_ref = np.zeros((nq, nk), dtype=np.float32)
        a = binding.head_args(q.reshape(-1), k.reshape(-1), v.reshape(-1), out_ref.reshape(-1), nq, nk, hd, scale, hd,
                              hd, hd, hd, 0, weights=w_ref.reshape(-1), mask=None if mask is None else mask.reshape(-1),
                              causal=kind == "causal")
        assert oracle.orc_attention_head_core(C.byref(a)) == 0
        x = scores64(q, k, scale, mask=mask, causal=kind == "causal")
        tq, tk, tv = (torch.from_numpy(t).cuda() for t in (q, k, v))
        tm = torch.from_numpy(mask).cuda() if mask is not None else None
        for with_weights in (False, True):
            out = torch.zeros((nq, hd), dtype=torch.float32, device="cuda")
            lse = torch.full((nq, 2), 7.0, dtype=torch.float32, device="cuda")
            wts = torch.full((nq, nk), 9.0, dtype=torch.float32, device="cuda")
            d = api.head_args(tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), out.data_ptr(), nq, nk, hd, scale, hd, hd,
                              hd, hd, 0, weights=wts.data_ptr() if with_weights else None, lse=lse.data_ptr(),
                              mask=tm.data_ptr() if tm is not None else None, causal=kind == "causal")
            lib.blt_attention_head_core_hip(abi.BLT_BACKEND_HIP, C.byref(d))
            lib.blt_backend_pass_sync_hip()
            what = "%s (weights_out %s)" % (name, "set" if with_weights else "NULL")
            got = out.cpu().numpy()
            err = np.abs(got.astype(np.float64) - out_ref)
            assert (err <= ATOL + RTOL * np.abs(out_ref)).all(), "%s: output max err %.3e" % (what, float(err.max()))
            check_pair(lse.cpu().numpy(), x, w_ref, what)
            if with_weights:
                # Deliberate difference from the reference's flash kernel, which clears the score buffer
                # when lse_out is set (attn_core.cu:268-272; no reference caller passes both): here
                # weights_out still receives the post-softmax weights.
                gw = wts.cpu().numpy()
                werr = np.abs(gw.astype(np.float64) - w_ref)
                assert (werr <= ATOL + RTOL * np.abs(w_ref)).all(), "%s: weights_out" % what
            else:
                assert (wts == 9.0).all().item(), "%s: a buffer that was not passed was written" % what
