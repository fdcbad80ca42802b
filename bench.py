#!/usr/bin/env python3
"""Benchmark of the fused layer-op path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config I]
                    [--workload-only] [--no-cpu] [--iters N] [--detail PATH]

A step is one forward + backward pass of every op of the workload configuration
(default --config 5: the Llama-3-8B-width shape with bf16 I/O, the largest
configuration that fits one GPU) over one batch of synthetic data already resident
in HBM.

Output: one JSON line per configuration with its per-op table (every op and
direction timed on its own with HIP events on the library's stream over rotating
buffer sets, so the working set exceeds the 256 MB Infinity Cache; copy_us /
vs_copy compare with a plain copy kernel moving the same number of bytes the same
way), the same tables as one file (--detail; by default bench_per_op.json in the run's output folder),
and as the LAST line one compact JSON object:

  value / unit     whole-step algorithmic GB/s (sum of the ops' algorithmic bytes
                   / wall-clock step time, synchronised on both sides)
  tokens_per_s     B*T / step time
  roofline         the dominant kernel of the step (largest share of time);
                   traffic = HBM bytes per launch of that kernel from the committed
                   counter summary profiles/hbm_traffic.json
  cpu_baseline     the numpy restatement of the reference's CPU kernels, timed
                   on this host with the reference's protocol (2 warm-up + >= 5
                   timed passes, timing_ops.py:76-100) on a bounded number of rows
  min_frac         per configuration, the op and direction furthest below the
                   8 TB/s roofline and its fraction

All device calls go through the C ABI (autograd_amd/capi.py).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import platform
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

from autograd_amd import capi  # noqa: E402
from autograd_amd.configs import CONFIGS, op_bytes  # noqa: E402
from autograd_amd.utils import f32_array_to_bf16_bits  # noqa: E402

METRIC = "HBM GB/s (% of 8 TB/s) + tokens/s for fused norm/act/RoPE/embed fwd+bwd"
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of each kernel, per configuration, from two `rocprofv3 --pmc`
# runs of this file (FETCH_SIZE, then WRITE_SIZE), each scaled by what the counter
# reads for the 64 MiB copy of spin_up(); the commands are recorded in the file.
TRAFFIC_FILE = ROOT / "profiles" / "hbm_traffic.json"
ROTATE_BYTES = 768 << 20      # cycle at least this much distinct memory per op
MAX_SETS = 8
FOLD_EVERY = 24               # norm backward calls whose column sums one batched fold takes (a 12-layer network has 25)


def vp(d, off=0):
    return None if d is None else C.c_void_p(d.ptr + off)


class Pool:
    """Device buffers; large ones are filled by tiling a 16 MiB chunk of N(0,1)
    samples on the device, so multi-GB operands need no multi-GB host arrays."""

    def __init__(self, ctx, seed):
        self.ctx = ctx
        rng = np.random.default_rng(seed)
        chunk = rng.standard_normal(4 << 20, dtype=np.float32)
        self.src = {"f32": ctx.upload(chunk), "bf16": ctx.upload(f32_array_to_bf16_bits(chunk))}
        self.bufs = []

    def _new(self, numel, np_dtype):
        d = self.ctx.empty((int(numel),), np_dtype)
        self.bufs.append(d)
        return d

    def normal(self, numel, dtype):
        d = self._new(numel, np.uint16 if dtype == "bf16" else np.float32)
        src = self.src[dtype]
        off = 0
        while off < d.nbytes:
            n = min(src.nbytes, d.nbytes - off)
            self.ctx.call("agrad_copy", vp(src), vp(d, off), n)
            off += n
        return d

    def empty(self, numel, dtype):
        return self._new(numel, np.uint16 if dtype == "bf16" else np.float32)

    def raw(self, nbytes):
        return self._new(nbytes, np.uint8)

    def upload(self, arr):
        d = self.ctx.upload(arr)
        self.bufs.append(d)
        return d

    def release(self):
        self.ctx.synchronize()
        for d in self.bufs:
            d.free()
        for d in self.src.values():
            d.free()
        self.bufs = []


class Case:
    def __init__(self, op, direction, nbytes, nsets, launch, kernel, in_step=None):
        self.op, self.direction, self.nbytes, self.nsets = op, direction, nbytes, nsets
        self.launch, self.kernel = launch, kernel
        self.us = None
        # part of the wall-clock step?  by default every forward and backward row is
        self.in_step = direction in ("fwd", "bwd") if in_step is None else in_step


def n_sets(working_bytes):
    return int(max(1, min(MAX_SETS, -(-ROTATE_BYTES // max(working_bytes, 1)))))


def token_ids(cfg, rng, n):
    if cfg.embed_dist.startswith("zipf"):
        s = float(cfg.embed_dist[4:])
        p = np.arange(1, cfg.V + 1, dtype=np.float64) ** (-s)
        p /= p.sum()
        return rng.choice(cfg.V, size=n, p=p).astype(np.int32)
    return rng.integers(0, cfg.V, size=n, dtype=np.int32)


def build_cases(ctx, cfg, pool):
    """every op of the config, forward and backward, as launchable cases"""
    rng = np.random.default_rng(cfg.seed)
    ids0 = token_ids(cfg, rng, cfg.N) if cfg.embed else None
    distinct = int(np.unique(ids0).size) if ids0 is not None else None
    nbytes = op_bytes(cfg, distinct)
    cases = []
    # one builder per op family: each keeps its buffers in its own scope
    for builder in (_embed_cases, _norm_cases, _act_cases, _rope_cases, _layout_cases, _primitive_cases, _loss_cases,
                    _opt_cases):
        cases += builder(ctx, cfg, pool, rng, nbytes, ids0)
    return cases


def _embed_cases(ctx, cfg, pool, rng, nbytes, ids0):
    dt = capi.BF16 if cfg.dtype == "bf16" else capi.F32
    N, Cw, e = cfg.N, cfg.C, cfg.esize
    cases = []
    if cfg.embed:
        name = cfg.embed
        k = n_sets(2 * N * Cw * e)
        W = pool.normal(cfg.V * Cw, cfg.dtype)
        wpe = pool.normal(cfg.T * Cw, cfg.dtype) if name == "gather_sum" else None
        ids = [pool.upload(ids0 if i == 0 else token_ids(cfg, rng, N)) for i in range(k)]
        out = [pool.empty(N * Cw, cfg.dtype) for _ in range(k)]
        dY = [pool.normal(N * Cw, cfg.dtype) for _ in range(k)]
        dW = pool.empty(cfg.V * Cw, cfg.dtype)
        dwpe = pool.empty(cfg.T * Cw, cfg.dtype) if wpe is not None else None
        # the forward call also orders the ids (one launch: the ordering runs beside the
        # bandwidth-bound gather); the backward call consumes that order.  Same results
        # as agrad_gather_forward + agrad_embedding_backward.
        order = [pool.raw(4 * (6 * N + 128)) for _ in range(k)]
        sort_ws_bytes = ctx.lib.agrad_embedding_sort_workspace_bytes(N, cfg.V)
        sort_ws = pool.raw(sort_ws_bytes)
        ws_bytes = ctx.lib.agrad_embedding_backward_sorted_workspace_bytes(N, Cw)
        ws = pool.raw(ws_bytes)
        ctx.call("agrad_fill", dW.ptr, 0, 0, 1, dW.nbytes)

        def fwd(i):
            ctx.call("agrad_gather_forward_sorted", dt, vp(ids[i]), vp(W), vp(wpe), vp(out[i]), N, cfg.T, Cw, cfg.V,
                     vp(order[i]), vp(sort_ws), sort_ws_bytes)

        def bwd(i):
            # the position table's gradient, when there is one, rides in the same launch
            ctx.call("agrad_embedding_backward_sorted", dt, vp(order[i]), vp(dY[i]), vp(dW), vp(dwpe), vp(ws), ws_bytes,
                     N, cfg.T, Cw, cfg.V, 0)

        for i in range(k):
            fwd(i)          # every set's order exists before backward is timed on its own

        def zero(i):
            ctx.call("agrad_fill", dW.ptr, 0, 0, 1, dW.nbytes)

        # Where the id ordering rides.  It is needed by the backward call only, and takes 8 us alone at
        # 16384 ids (latency, not bytes).  "fwd" is the one launch that gathers and orders (what the
        # step and Runtime use); "fwd-plain" the gather without it; "id_ordering" the ordering alone;
        # "..._grad_zero_fill+order" the ordering at the front of the gradient table's zero fill instead
        # (agrad_embedding_order), beside the plain fill: the fill runs best with few waves on a CU and
        # is the worse host of the two.
        def fwd_plain(i):
            ctx.call("agrad_gather_forward", dt, vp(ids[i]), vp(W), vp(wpe), vp(out[i]), N, cfg.T, Cw, cfg.V)

        def order_alone(i):
            ctx.call("agrad_embedding_order", vp(ids[i]), N, cfg.V, vp(order[i]), vp(sort_ws), sort_ws_bytes, None, 0)

        def zero_and_order(i):
            ctx.call("agrad_embedding_order", vp(ids[i]), N, cfg.V, vp(order[i]), vp(sort_ws), sort_ws_bytes, vp(dW), dW.nbytes)

        # "..._grad_row_reset": the table gradient brought back to zero by clearing the rows of the last
        # pass's ids (agrad_embedding_grad_reset, what Runtime.zero_grad does after the first step) --
        # N*C items written instead of the fill's V*C.
        def row_reset(i):
            ctx.call("agrad_embedding_grad_reset", dt, vp(ids[i]), N, vp(dW), Cw, cfg.V)

        cases.append(Case(name, "fwd", nbytes[name][0], k, fwd, "gather_sort_kernel"))
        cases.append(Case(name, "fwd-plain", nbytes[name][0], k, fwd_plain, "gather_", in_step=False))
        cases.append(Case(name, "bwd", nbytes[name][1], k, bwd, "emb_row_sum_kernel"))
        cases.append(Case("id_ordering", "aux", 4 * N + 4 * (6 * N + 128), k, order_alone, "emb_group_sort_kernel"))
        cases.append(Case(name + "_grad_zero_fill", "aux", cfg.V * Cw * e, 1, zero, "fill16_kernel"))
        cases.append(Case(name + "_grad_row_reset", "aux", N * Cw * e, k, row_reset, "zero_rows16_kernel"))
        cases.append(Case(name + "_grad_zero_fill+order", "aux", cfg.V * Cw * e, k, zero_and_order, "fill_order_kernel"))
    return cases


def _norm_cases(ctx, cfg, pool, rng, nbytes, ids0):
    dt = capi.BF16 if cfg.dtype == "bf16" else capi.F32
    N, Cw, e = cfg.N, cfg.C, cfg.esize
    cases = []
    if cfg.norm:
        name = ("add+" if cfg.norm_residual else "") + cfg.norm + "norm"
        kind = capi.NORM_LAYER if cfg.norm == "layer" else capi.NORM_RMS
        k = n_sets(4 * N * Cw * e)
        gamma = pool.upload((1 + 0.02 * rng.standard_normal(Cw)).astype(np.float32)) if cfg.norm_affine \
            else pool.upload(np.ones(Cw, np.float32))
        beta = None
        if cfg.norm == "layer":
            beta = pool.upload((0.02 * rng.standard_normal(Cw)).astype(np.float32) if cfg.norm_affine
                               else np.zeros(Cw, np.float32))
        a = [pool.normal(N * Cw, cfg.dtype) for _ in range(k)]     # x   / saved h
        b = [pool.normal(N * Cw, cfg.dtype) for _ in range(k)]     # r   / incoming residual grad
        c = [pool.normal(N * Cw, cfg.dtype) for _ in range(k)]     # h   / dy
        d = [pool.empty(N * Cw, cfg.dtype) for _ in range(k)]      # y   / dx
        dgamma = pool.empty(Cw, "f32")
        dbeta = pool.empty(Cw, "f32") if beta is not None else None
        ws_bytes = ctx.lib.agrad_norm_backward_workspace_bytes(N, Cw, dt)
        ws = pool.raw(ws_bytes)
        res = cfg.norm_residual

        def fwd(i):
            ctx.call("agrad_norm_forward", kind, dt, vp(a[i]), vp(b[i]) if res else None, vp(gamma), vp(beta),
                     vp(c[i]) if res else None, vp(d[i]), N, Cw, cfg.norm_eps)

        def bwd(i):
            ctx.call("agrad_norm_backward", kind, dt, vp(a[i]), vp(c[i]), vp(gamma), vp(b[i]) if res else None,
                     vp(d[i]), None, vp(dgamma), vp(dbeta), vp(ws), ws_bytes, N, Cw, cfg.norm_eps, 0)

        # The same backward call with its dgamma / dbeta fold left pending (AGRAD_DEFER_PARAM_GRAD) and ONE
        # launch folding FOLD_EVERY calls' sums, the way Runtime.backward_graph ends a pass over a network
        # with that many norms; every pending call has its own workspace and gradient rows.
        d_ws = [pool.raw(ws_bytes) for _ in range(FOLD_EVERY)]
        d_dgamma = [pool.empty(Cw, "f32") for _ in range(FOLD_EVERY)]
        d_dbeta = [pool.empty(Cw, "f32") if beta is not None else None for _ in range(FOLD_EVERY)]
        calls = [0]

        def bwd_deferred(i):
            j = calls[0] % FOLD_EVERY
            ctx.call("agrad_norm_backward", kind, dt, vp(a[i]), vp(c[i]), vp(gamma), vp(b[i]) if res else None,
                     vp(d[i]), None, vp(d_dgamma[j]), vp(d_dbeta[j]), vp(d_ws[j]), ws_bytes, N, Cw, cfg.norm_eps,
                     capi.DEFER_PARAM_GRAD)
            calls[0] += 1
            if calls[0] % FOLD_EVERY == 0:
                ctx.call("agrad_finalize_param_grads")

        cases.append(Case(name, "fwd", nbytes[name][0], k, fwd, "norm_fwd_kernel"))
        cases.append(Case(name, "bwd", nbytes[name][1], k, bwd, "norm_bwd_kernel"))
        cases.append(Case(name, f"bwd-fold/{FOLD_EVERY}", nbytes[name][1], k, bwd_deferred, "norm_bwd_kernel"))
    return cases


def _act_cases(ctx, cfg, pool, rng, nbytes, ids0):
    dt = capi.BF16 if cfg.dtype == "bf16" else capi.F32
    N, e = cfg.N, cfg.esize
    cases = []
    if cfg.act:
        H = cfg.act_width
        rows = N
        if cfg.act == "swiglu":
            k = n_sets(5 * rows * H * e)
            gu = [pool.normal(rows * 2 * H, cfg.dtype) for _ in range(k)]
            h = [pool.normal(rows * H, cfg.dtype) for _ in range(k)]
            dgu = [pool.empty(rows * 2 * H, cfg.dtype) for _ in range(k)]

            def fwd(i):
                ctx.call("agrad_swiglu_forward", dt, vp(gu[i]), vp(h[i]), rows, H)

            def bwd(i):
                ctx.call("agrad_swiglu_backward", dt, vp(gu[i]), vp(h[i]), vp(dgu[i]), rows, H, 0)

            cases.append(Case("swiglu", "fwd", nbytes["swiglu"][0], k, fwd, "swiglu_fwd_kernel"))
            cases.append(Case("swiglu", "bwd", nbytes["swiglu"][1], k, bwd, "swiglu_bwd_kernel"))
        else:
            n = rows * H
            k = n_sets(3 * n * e)
            x = [pool.normal(n, cfg.dtype) for _ in range(k)]
            y = [pool.normal(n, cfg.dtype) for _ in range(k)]
            dx = [pool.empty(n, cfg.dtype) for _ in range(k)]
            f_name, b_name = f"agrad_{cfg.act}_forward", f"agrad_{cfg.act}_backward"

            def fwd(i):
                ctx.call(f_name, dt, vp(x[i]), vp(dx[i]), n)

            def bwd(i):
                ctx.call(b_name, dt, vp(x[i]), vp(y[i]), vp(dx[i]), n, 0)

            functor = {"gelu": "Gelu", "relu2": "Relu2"}[cfg.act]
            cases.append(Case(cfg.act, "fwd", nbytes[cfg.act][0], k, fwd, f"ew_kernel {functor}Fwd"))
            cases.append(Case(cfg.act, "bwd", nbytes[cfg.act][1], k, bwd, f"ew_kernel {functor}Bwd"))
    return cases


def _layout_cases(ctx, cfg, pool, rng, nbytes, ids0):
    """layout changes beside the hot path: q from [B,T,H,D] to [B,H,T,D] (rows kernel)
    and the [N, C] activation transposed to [C, N] (tile kernel); 2 * numel * e bytes"""
    import ctypes as C
    dt = capi.BF16 if cfg.dtype == "bf16" else capi.F32
    e = cfg.esize
    cases = []

    def add(name, dense_shape, dims):
        numel = int(np.prod(dense_shape))
        k = n_sets(numel * e)
        src = [pool.normal(numel, cfg.dtype) for _ in range(k)]
        dst = [pool.empty(numel, cfg.dtype) for _ in range(k)]
        base = np.cumprod((1,) + tuple(dense_shape[::-1]))[:-1][::-1]
        shape = (C.c_uint32 * len(dims))(*[dense_shape[d] for d in dims])
        strides = (C.c_uint64 * len(dims))(*[int(base[d]) for d in dims])

        def run(i):
            ctx.call("agrad_strided_copy", dt, vp(src[i]), vp(dst[i]), len(dims), shape, strides, 0)

        cases.append(Case(name, "layout", 2 * numel * e, k, run, "strided_"))

    if cfg.rope:
        Hq, _, D, _, _ = cfg.rope
        add("permute_bthd_bhtd", (cfg.B, cfg.T, Hq, D), (0, 2, 1, 3))
    if cfg.norm:
        add("transpose_nc_cn", (cfg.N, cfg.C), (1, 0))
    return cases


def _primitive_cases(ctx, cfg, pool, rng, nbytes, ids0):
    """the primitive ops beside the hot path: softmax over attention-shaped rows
    [B*H*T, T] (2 / 3 passes of n*e bytes) and x[N, C] * gamma[C] with both gradients
    (2*n*e forward; backward reads g and x and writes dx: 3*n*e)"""
    dt = capi.BF16 if cfg.dtype == "bf16" else capi.F32
    e = cfg.esize
    cases = []
    if cfg.rope:
        Hq = cfg.rope[0]
        rows = cfg.B * Hq * cfg.T
        V = cfg.T
        while rows * V * e > (1 << 30):       # keep the score matrix at a size one layer of one micro-batch has
            rows //= 2
        n = rows * V
        k = n_sets(2 * n * e)
        x = [pool.normal(n, cfg.dtype) for _ in range(k)]
        y = [pool.empty(n, cfg.dtype) for _ in range(k)]
        g = [pool.normal(n, cfg.dtype) for _ in range(k)]
        dx = [pool.empty(n, cfg.dtype) for _ in range(k)]

        def sm_fwd(i):
            ctx.call("agrad_softmax_forward", dt, vp(x[i]), vp(y[i]), rows, V)

        def sm_bwd(i):
            ctx.call("agrad_softmax_backward", dt, vp(y[i]), vp(g[i]), vp(dx[i]), rows, V, 0)

        for i in range(k):
            sm_fwd(i)
        cases.append(Case(f"softmax[{rows}x{V}]", "prim-fwd", 2 * n * e, k, sm_fwd, "softmax_fwd_kernel"))
        cases.append(Case(f"softmax[{rows}x{V}]", "prim-bwd", 3 * n * e, k, sm_bwd, "softmax_bwd_kernel"))
    if cfg.norm:
        # (own names throughout: the softmax closures above still read theirs)
        N, Cw = cfg.N, cfg.C
        m_n = N * Cw
        m_k = n_sets(2 * m_n * e)
        m_x = [pool.normal(m_n, cfg.dtype) for _ in range(m_k)]
        m_out = [pool.empty(m_n, cfg.dtype) for _ in range(m_k)]
        gam = pool.normal(Cw, cfg.dtype)
        dgam = pool.empty(Cw, cfg.dtype)
        ws_bytes = ctx.lib.agrad_mul_backward_workspace_bytes(capi.MUL_ROW, N, Cw)
        ws = pool.raw(max(ws_bytes, 256))

        def mul_fwd(i):
            ctx.call("agrad_mul_forward", dt, capi.MUL_ROW, vp(m_x[i]), vp(gam), vp(m_out[i]), N, Cw)

        def mul_bwd(i):        # m_out[i] plays the upstream gradient, the next set's m_out receives dx
            ctx.call("agrad_mul_backward", dt, capi.MUL_ROW, vp(m_out[i]), vp(m_x[i]), vp(gam), vp(m_out[(i + 1) % m_k]),
                     vp(dgam), vp(ws), ws_bytes, N, Cw, 0)

        cases.append(Case("mul_row", "prim-fwd", 2 * m_n * e, m_k, mul_fwd, "bcast_mul_kernel"))
        if m_k > 1:
            cases.append(Case("mul_row", "prim-bwd", 3 * m_n * e, m_k, mul_bwd, "bcast_mul_kernel"))
    if cfg.act == "gelu":
        # GELU(h + b) on the MLP's hidden tensor [N, 4C]: forward reads h, writes y (2*n*e);
        # backward reads dy and h, writes dh (3*n*e) and leaves the bias gradient beside it
        bg_rows, bg_C = cfg.N, cfg.act_width
        bg_n = bg_rows * bg_C
        bg_k = n_sets(3 * bg_n * e)
        bg_h = [pool.normal(bg_n, cfg.dtype) for _ in range(bg_k)]
        bg_dy = [pool.normal(bg_n, cfg.dtype) for _ in range(bg_k)]
        bg_out = [pool.empty(bg_n, cfg.dtype) for _ in range(bg_k)]
        bg_b = pool.normal(bg_C, cfg.dtype)
        bg_db = pool.empty(bg_C, cfg.dtype)
        bg_ws_bytes = ctx.lib.agrad_gelu_bias_backward_workspace_bytes(bg_rows, bg_C)
        bg_ws = pool.raw(max(bg_ws_bytes, 256))

        def bias_gelu_fwd(i):
            ctx.call("agrad_gelu_bias_forward", dt, vp(bg_h[i]), vp(bg_b), vp(bg_out[i]), bg_rows, bg_C)

        def bias_gelu_bwd(i):
            ctx.call("agrad_gelu_bias_backward", dt, vp(bg_dy[i]), vp(bg_h[i]), vp(bg_b), vp(bg_out[i]), vp(bg_db),
                     vp(bg_ws), bg_ws_bytes, bg_rows, bg_C, 0)

        cases.append(Case("bias_gelu", "prim-fwd", 2 * bg_n * e, bg_k, bias_gelu_fwd, "gelu_bias_kernel"))
        cases.append(Case("bias_gelu", "prim-bwd", 3 * bg_n * e, bg_k, bias_gelu_bwd, "colsum_partial_kernel"))
    return cases


def _rope_cases(ctx, cfg, pool, rng, nbytes, ids0):
    dt = capi.BF16 if cfg.dtype == "bf16" else capi.F32
    N = cfg.N
    cases = []
    if cfg.rope:
        Hq, Hkv, D, theta, sign = cfg.rope
        k = n_sets(nbytes["rope"][0] // 2)
        pos = np.arange(cfg.T, dtype=np.float32)[:, None]
        inv = np.float32(theta) ** (-np.arange(0, D, 2, dtype=np.float32)[None, :] / np.float32(D))
        cos = pool.upload(np.cos(pos * inv).astype(np.float32))
        sin = pool.upload(np.sin(pos * inv).astype(np.float32))
        q = [pool.normal(N * Hq * D, cfg.dtype) for _ in range(k)]
        kk = [pool.normal(N * Hkv * D, cfg.dtype) for _ in range(k)]

        def fwd(i):
            ctx.call("agrad_rope_qk", dt, vp(q[i]), vp(kk[i]), vp(cos), vp(sin), cfg.B, cfg.T, Hq, Hkv, D, sign, 0)

        def bwd(i):
            ctx.call("agrad_rope_qk", dt, vp(q[i]), vp(kk[i]), vp(cos), vp(sin), cfg.B, cfg.T, Hq, Hkv, D, sign, 1)

        cases.append(Case("rope", "fwd", nbytes["rope"][0], k, fwd, "rope_kernel"))
        cases.append(Case("rope", "bwd", nbytes["rope"][1], k, bwd, "rope_kernel"))
    return cases


def _loss_cases(ctx, cfg, pool, rng, nbytes, ids0):
    """cross-entropy over logits [N, V]: forward reads the logits once, backward
    reads them and writes the gradient (the forward pass leaves the row
    log-sum-exp).  Reported beside the step, not part of it."""
    if not cfg.embed:
        return []
    dt = capi.BF16 if cfg.dtype == "bf16" else capi.F32
    N, V, e = cfg.N, cfg.V, cfg.esize
    k = n_sets(2 * N * V * e)
    logits = [pool.normal(N * V, cfg.dtype) for _ in range(k)]
    dlogits = [pool.empty(N * V, cfg.dtype) for _ in range(k)]
    labels = pool.upload(rng.integers(0, V, N, dtype=np.int32))
    loss, lse, dloss = pool.empty(N, "f32"), pool.empty(N, "f32"), pool.normal(N, "f32")

    def fwd(i):
        ctx.call("agrad_cross_entropy_forward", dt, vp(logits[i]), vp(labels), vp(loss), vp(lse), N, V)

    def bwd(i):
        ctx.call("agrad_cross_entropy_backward", dt, vp(logits[i]), vp(labels), vp(dloss), vp(lse), vp(dlogits[i]), N, V, 0)

    def fused(i):
        # loss and gradient in one launch, in place: reads the row once, writes it once (the gradient a
        # call leaves is the next call's logits: any finite values time alike)
        ctx.call("agrad_cross_entropy_fused", dt, vp(logits[i]), vp(labels), vp(loss), vp(lse), None, N, V, 0, 1.0 / N, 1)

    fwd(0)   # lse for the backward timing
    return [Case("cross_entropy", "loss-fwd", N * V * e + 12 * N, k, fwd, "ce_fwd_kernel"),
            Case("cross_entropy", "loss-bwd", 2 * N * V * e + 12 * N, k, bwd, "ce_bwd_kernel"),
            Case("cross_entropy_fused", "loss-both", 2 * N * V * e + 12 * N, k, fused, "ce_fused_")]


def _opt_cases(ctx, cfg, pool, rng, nbytes, ids0):
    """AdamW over the embedding table's slab (the consumer of the gradients above)
    and the gradient-norm partial sums; fp32 parameters and moments, gradients in
    the configuration's I/O type.  Reported beside the step, not part of it."""
    if not cfg.embed:
        return []
    n = cfg.V * cfg.C
    gdt = capi.BF16 if cfg.dtype == "bf16" else capi.F32
    per_elem = 24 + cfg.esize                # read p, m, v (12) and g; write p, m, v (12)
    k = n_sets(per_elem * n)
    sets = []
    for _ in range(k):
        sets.append((pool.normal(n, "f32"), pool.normal(n, cfg.dtype), pool.empty(n, "f32"), pool.empty(n, "f32")))
        ctx.call("agrad_fill", sets[-1][2].ptr, 0, 0, 4, n)
        ctx.call("agrad_fill", sets[-1][3].ptr, 0, 0, 4, n)
    groups = ctx.lib.agrad_grad_norm_groups(n)
    partial = pool.empty(groups, "f32")
    lr, b1, b2 = 1e-3, 0.9, 0.999

    def step(i):
        p, g, m, v = sets[i]
        ctx.call("agrad_adamw_step", gdt, vp(p), vp(g), vp(m), vp(v), n, n, lr * 0.01, b1, 1.0 - b1, b2, 1.0 - b2,
                 1e-8, lr, 1.0, 1.0)

    def norm(i):
        ctx.call("agrad_grad_norm_sq", gdt, vp(sets[i][1]), vp(partial), n)

    # the same step with 8-bit moments: p read and written (8), g, one code byte of each
    # moment read and written (4), one scale pair per 256 elements
    from autograd_amd.optimizer import build_dynamic_map
    per_elem8 = 12 + cfg.esize
    q_n = n
    q_k = n_sets(per_elem8 * q_n)
    q_sets = []
    for _ in range(q_k):
        q_sets.append((pool.normal(q_n, "f32"), pool.normal(q_n, cfg.dtype), pool.raw(q_n), pool.raw(q_n),
                       pool.empty(groups, "f32"), pool.empty(groups, "f32")))
    map_m, map_v = ctx.upload(build_dynamic_map(True)), ctx.upload(build_dynamic_map(False))
    q_first = [True] * q_k

    def step8(i):
        p8, g8, qm, qv, am, av = q_sets[i]
        ctx.call("agrad_adamw8bit_step", gdt, vp(p8), vp(g8), vp(qm), vp(qv), vp(am), vp(av), vp(map_m), vp(map_v),
                 q_n, q_n, 1.0 - lr * 0.01, lr, b1, b2, 1e-8, 1.0, 1.0, int(q_first[i]))
        q_first[i] = False

    return [Case("adamw", "opt", per_elem * n, k, step, "adamw_vec_kernel"),
            Case("adamw_8bit", "opt", per_elem8 * q_n + 16 * groups, q_k, step8, "adamw8bit_kernel"),
            Case("grad_norm_sq", "opt", cfg.esize * n + 4 * groups, k, norm, "grad_norm_sq_kernel")]


def spin_up(ctx, seconds=0.25):
    """keep the GPU busy for a moment so that clocks have left their idle state
    before anything is timed"""
    n = 64 << 20
    a, b = ctx.empty((n,), np.uint8), ctx.empty((n,), np.uint8)
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(50):
            ctx.call("agrad_copy", vp(a), vp(b), n)
        ctx.synchronize()
    a.free()
    b.free()


def time_case(ctx, case, iters, exact=False):
    # at least `iters` launches and at least ~2 ms of GPU time (exactly `iters`
    # launches when exact: a counter-collection run pays per dispatch), timed as
    # up to five back-to-back groups; the figure is the median group's average
    for i in range(min(case.nsets, 3)):
        case.launch(i)
    ctx.synchronize()
    ctx.timer_start()
    for it in range(8):
        case.launch(it % case.nsets)
    probe_us = ctx.timer_stop() * 1e3 / 8
    if not exact:
        iters = int(max(iters, min(2000, 2000.0 / max(probe_us, 0.5))))
    groups = 1 if exact else min(5, max(1, iters // 6))
    per = -(-iters // groups)
    samples, it = [], 0
    for _ in range(groups):
        ctx.timer_start()
        for _ in range(per):
            case.launch(it % case.nsets)
            it += 1
        samples.append(ctx.timer_stop() * 1e3 / per)
    ctx.synchronize()
    case.us = float(np.median(samples))
    return case.us


def time_copy_of(ctx, nbytes, iters, exact=False):
    """What a plain 16-byte-per-lane copy kernel needs to move the same number of
    bytes (half read, half written) over the same rotation of buffer sets: the
    practical ceiling of this GPU for a stream of that size, launch ramp included."""
    half = max(16, (nbytes // 2) // 16 * 16)
    k = n_sets(nbytes)
    bufs = [(ctx.empty((half,), np.uint8), ctx.empty((half,), np.uint8)) for _ in range(k)]
    try:
        case = Case("copy", "ref", 2 * half, k,
                    lambda i: ctx.call("agrad_copy", vp(bufs[i][0]), vp(bufs[i][1]), half), "copy16_kernel")
        return time_case(ctx, case, iters, exact)
    finally:
        ctx.synchronize()
        for a, b in bufs:
            a.free()
            b.free()


def case_row(case):
    gbps = case.nbytes / (case.us * 1e-6) / 1e9
    row = {"op": case.op, "dir": case.direction, "MB": round(case.nbytes / 1e6, 2), "us": round(case.us, 2),
           "GBps": round(gbps, 1), "frac_hbm": round(gbps / HBM_PEAK_GBS, 4), "sets": case.nsets,
           "kernel": case.kernel}
    if getattr(case, "copy_us", None):
        row["copy_us"] = round(case.copy_us, 2)          # same bytes through the plain copy kernel
        row["vs_copy"] = round(case.copy_us / case.us, 3)
    return row


def run_config(ctx, cfg, iters):
    pool = Pool(ctx, cfg.seed)
    try:
        cases = build_cases(ctx, cfg, pool)
        for case in cases:
            time_case(ctx, case, iters)
    finally:
        pool.release()
    for case in cases:
        case.copy_us = time_copy_of(ctx, case.nbytes, iters)
    return [case_row(c) for c in cases]


def run_workload(ctx, cfg, steps, warmup, iters, exact=False):
    pool = Pool(ctx, cfg.seed)
    try:
        cases = build_cases(ctx, cfg, pool)
        step_cases = [c for c in cases if c.in_step and c.direction.startswith("fwd")] + \
                     [c for c in reversed(cases) if c.in_step and c.direction == "bwd"]
        step_bytes = sum(c.nbytes for c in step_cases)

        def step(s):
            for c in step_cases:
                c.launch(s % c.nsets)

        for s in range(warmup):
            step(s)
        ctx.synchronize()
        t0 = time.perf_counter()
        for s in range(steps):
            step(warmup + s)
        ctx.synchronize()
        wall = time.perf_counter() - t0
        for case in cases:
            time_case(ctx, case, iters, exact)
    finally:
        pool.release()
    for case in cases:
        case.copy_us = time_copy_of(ctx, case.nbytes, iters, exact)
    return cases, step_bytes, wall


def graph_replay(ctx, cfg, iters=200):
    """The launch-bound chain (a few MB per op): every op of `cfg` forward then
    backward, launched one by one and replayed from a recorded graph."""
    pool = Pool(ctx, cfg.seed)
    try:
        cases = [c for c in build_cases(ctx, cfg, pool) if c.in_step]
        chain = [c for c in cases if c.direction.startswith("fwd")] + [c for c in reversed(cases) if c.direction == "bwd"]

        def step():
            for c in chain:
                c.launch(0)

        for _ in range(3):
            step()
        ctx.synchronize()
        ctx.call("agrad_graph_begin")
        step()
        gid = C.c_uint64(0)
        ctx.call("agrad_graph_end", C.byref(gid))
        out = {}
        for name, fn in (("eager_us", step), ("graph_us", lambda: ctx.call("agrad_graph_launch", gid.value))):
            for _ in range(5):
                fn()
            ctx.synchronize()
            ctx.timer_start()
            for _ in range(iters):
                fn()
            out[name] = round(ctx.timer_stop() * 1e3 / iters, 2)
        ctx.synchronize()
        ctx.call("agrad_graph_destroy", gid.value)
        out["workload"] = f"configs[{cfg.index}] {cfg.name}: {len(chain)} ops forward then backward, one set of buffers"
        out["speedup"] = round(out["eager_us"] / out["graph_us"], 2)
        return out
    finally:
        pool.release()


# ---------------------------------------------------------------------------------
# The same ops through the host path the reference's trainers use: Tensor -> Op -> Backend
# -> Device -> Runtime (runtime.py:802-854), launched eagerly node by node and replayed
# from a recorded graph, beside the C-ABI figures of the per-op table.
# ---------------------------------------------------------------------------------
def runtime_path(cfg, per_op_rows, steps=20, ctx=None):
    """One training-step's worth of this configuration's ops as Runtime graphs on the "hip"
    device: ids -> embedding -> (add +) norm as one chain, the activation on its own input.
    (Rotary is left out: its two outputs have no common consumer without the attention GEMMs.)
    A step is the reference's timing protocol (timing_ops.py:76-100): zero_grad, forward, fill
    the upstream gradient, backward_graph, with the pass synchronisations those calls make.
    Returns microseconds per step -- eager by that protocol, through Runtime.execute (one pass), and
    execute replayed from a recorded graph -- and the sum of the same kernels' C-ABI times beside them."""
    from autograd_amd import op as O
    from autograd_amd.runtime import Runtime
    from autograd_amd.tensor import Tensor
    from autograd_amd.utils import BF16

    dt = BF16 if cfg.dtype == "bf16" else np.float32
    rng = np.random.default_rng(cfg.seed)

    def leaf(shape, grad, val, dtype=dt):
        return Tensor(shape=tuple(shape), dtype=dtype, device="hip", requires_grad=grad, init_val=val)

    roots = []
    if cfg.embed and cfg.norm:
        ids = leaf((cfg.B, cfg.T), False, token_ids(cfg, rng, cfg.N).reshape(cfg.B, cfg.T), np.int32)
        W = leaf((cfg.V, cfg.C), True, 0.02)
        if cfg.embed == "gather_sum":
            x0 = O.EmbeddingSumOp()(ids, W, leaf((cfg.T, cfg.C), True, 0.01))
        else:
            x0 = O.GatherOp()(ids, W)
        gamma = leaf((cfg.C,), True, 1.0, np.float32)
        if cfg.norm == "layer":
            beta = leaf((cfg.C,), True, 0.0, np.float32)
            if cfg.norm_residual:
                _, y = O.AddLayerNormOp(eps=cfg.norm_eps)(x0, leaf((cfg.B, cfg.T, cfg.C), False, 0.5), gamma, beta)
            else:
                y = O.LayerNormOp(eps=cfg.norm_eps)(x0, gamma, beta)
        elif cfg.norm_residual:
            _, y = O.AddRMSNormOp(eps=cfg.norm_eps)(x0, leaf((cfg.B, cfg.T, cfg.C), False, 0.5), gamma)
        else:
            y = O.RMSNormOp(eps=cfg.norm_eps)(x0, gamma)
        roots.append(y)
    if cfg.act:
        H = cfg.act_width
        if cfg.act == "swiglu":
            roots.append(O.SwiGLUOp()(leaf((cfg.N, 2 * H), True, 0.5)))
        else:
            act = O.GELUOp() if cfg.act == "gelu" else O.ReLUSquaredOp()
            roots.append(act(leaf((cfg.N, H), True, 0.5)))
    rts = []
    for out in roots:
        rt = Runtime(device="hip")
        rt.loss = out
        rt.build_topo(out)
        rt.bind_memory()
        rts.append(rt)
    backend = rts[0].backend

    def step():
        for rt in rts:
            rt.zero_grad()
            rt.forward()
            rt.backend.fill(rt.loss.grad, 1.0)
            rt.backward_graph()

    try:
        for _ in range(3):
            step()
        backend.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        backend.synchronize()
        eager_us = (time.perf_counter() - t0) * 1e6 / steps
        # the same through Runtime.execute, which makes one pass (one wait) of a step
        for rt in rts:
            rt.execute()
        backend.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            for rt in rts:
                rt.execute()
        backend.synchronize()
        execute_us = (time.perf_counter() - t0) * 1e6 / steps
        # ... and without the wait at the end of each step (one wait after the last)
        t0 = time.perf_counter()
        for _ in range(steps):
            for rt in rts:
                rt.execute(wait=False)
        backend.synchronize()
        nowait_us = (time.perf_counter() - t0) * 1e6 / steps
        def execute_all():
            for rt in rts:
                rt.execute()

        graph = rts[0].capture(execute_all)
        for _ in range(3):
            graph.launch()
        backend.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.launch()
        backend.synchronize()
        replay_us = (time.perf_counter() - t0) * 1e6 / steps
        graph.destroy()
    finally:
        for rt in rts:
            rt.release()
    # the kernels Runtime.execute launches for these graphs, from the per-op table
    names = set()
    if cfg.embed and cfg.norm:
        names |= {cfg.embed, ("add+" if cfg.norm_residual else "") + cfg.norm + "norm"}
    if cfg.act:
        names.add(cfg.act)
    kernels = [r for r in per_op_rows if (r["op"] in names and r["dir"] in ("fwd", "bwd"))
               or r["op"] == cfg.embed + "_grad_row_reset"]     # (what zero_grad launches after the first step)
    c_abi_us = sum(r["us"] for r in kernels)
    # the protocol's own fills, through the C ABI as well: the upstream gradient of each graph's output
    fill_us = 0.0
    if ctx is not None:
        for out in roots:
            nb = out.numel * cfg.esize
            buf = ctx.empty((nb,), np.uint8)
            case = Case("upstream_fill", "aux", nb, 1, lambda i, b=buf, n=nb: ctx.call("agrad_fill", b.ptr, 0, 0, 1, n), "fill16_kernel")
            fill_us += time_case(ctx, case, 30)
            buf.free()
    c_abi_us += fill_us
    return {"workload": f"configs[{cfg.index}] {cfg.name}: embedding -> norm chain and the activation, forward + backward "
                        f"through Runtime(device='hip'), {len(rts)} graphs",
            "eager_us": round(eager_us, 1), "execute_us": round(execute_us, 1), "execute_nowait_us": round(nowait_us, 1), "replay_us": round(replay_us, 1), "c_abi_kernels_us": round(c_abi_us, 1),
            "eager_vs_c_abi": round(eager_us / c_abi_us, 3) if c_abi_us else None,
            "nowait_vs_c_abi": round(nowait_us / c_abi_us, 3) if c_abi_us else None,
            "replay_vs_c_abi": round(replay_us / c_abi_us, 3) if c_abi_us else None,
            "c_abi_rows": [f"{r['op']} {r['dir']}" for r in kernels] + [f"upstream fills {fill_us:.1f} us"]}


# ---------------------------------------------------------------------------------
# CPU baseline: the numpy restatement of the reference's CPU kernels (oracle/),
# imported here only, as the thing that is timed beside the GPU numbers.
# ---------------------------------------------------------------------------------
def cpu_baseline(cfg):
    from oracle import cpu_ops as K

    rng = np.random.default_rng(cfg.seed)
    rows = cfg.N if cfg.index <= 1 else min(cfg.N, 2048)
    B = max(1, rows // cfg.T)
    T = min(cfg.T, rows)
    rows = B * T
    Cw = cfg.C
    widen = (lambda a: K.round_bf16(a)) if cfg.dtype == "bf16" else (lambda a: a)
    work = []

    if cfg.embed:
        ids = token_ids(cfg, rng, rows).reshape(B, T)
        # the table at its full [V, C] size as untouched zero pages, with values only in
        # the rows these ids address: the CPU kernels touch nothing else, and drawing
        # (or even zero-filling) V*C samples on one core takes minutes at the large shapes
        W = np.zeros((cfg.V, Cw), np.float32)
        uniq = np.unique(ids)
        W[uniq] = widen((0.02 * rng.standard_normal((uniq.size, Cw), dtype=np.float32)).astype(np.float32))
        wpe = widen((0.02 * rng.standard_normal((T, Cw))).astype(np.float32)) if cfg.embed == "gather_sum" else None
        dY = rng.standard_normal((B, T, Cw), dtype=np.float32)
        dW = np.zeros((cfg.V, Cw), np.float32)
        dwpe = np.zeros_like(wpe) if wpe is not None else None

        def emb():
            if wpe is None:
                K.gather_forward(ids, W)
                K.gather_backward_into(ids, dY, dW)
            else:
                K.embedding_sum_forward(ids, W, wpe)
                K.embedding_sum_backward_into(ids, dY, dW, dwpe)
        work.append(emb)
    if cfg.norm:
        x = rng.standard_normal((rows, Cw), dtype=np.float32)
        r = rng.standard_normal((rows, Cw), dtype=np.float32)
        dy = rng.standard_normal((rows, Cw), dtype=np.float32)
        g = (1 + 0.02 * rng.standard_normal(Cw)).astype(np.float32)
        bta = (0.02 * rng.standard_normal(Cw)).astype(np.float32)
        dx, dg, db = np.zeros_like(x), np.zeros_like(g), np.zeros_like(g)

        def norm():
            h = K.add_forward(x, r) if cfg.norm_residual else x
            if cfg.norm == "layer":
                K.layernorm_forward(h, g, bta, cfg.norm_eps)
                K.layernorm_backward_into(h, g, dy, cfg.norm_eps, dx, dg, db)
            else:
                K.rmsnorm_forward(h, g, cfg.norm_eps)
                K.rmsnorm_backward_into(h, g, dy, cfg.norm_eps, dx, dg)
        work.append(norm)
    if cfg.act:
        H = cfg.act_width
        if cfg.act == "swiglu":
            gu = rng.standard_normal((rows, 2 * H), dtype=np.float32)
            dh = rng.standard_normal((rows, H), dtype=np.float32)
            work.append(lambda: (K.swiglu_forward(gu), K.swiglu_backward(gu, dh)))
        else:
            xa = rng.standard_normal((rows, H), dtype=np.float32)
            dya = rng.standard_normal((rows, H), dtype=np.float32)
            dxa = np.zeros_like(xa)
            f, bfn = (K.gelu_forward, K.gelu_backward_into) if cfg.act == "gelu" else (K.relu2_forward, K.relu2_backward_into)
            work.append(lambda: (f(xa), bfn(xa, dya, dxa)))
    if cfg.rope:
        Hq, Hkv, D, theta, sign = cfg.rope
        q = rng.standard_normal((B, T, Hq, D), dtype=np.float32)
        kk = rng.standard_normal((B, T, Hkv, D), dtype=np.float32)
        cos, sin = K.rope_tables(T, D, theta)
        work.append(lambda: (K.rope_signed(q, kk, cos, sin, sign, False), K.rope_signed(q, kk, cos, sin, sign, True)))

    def one_pass():
        for fn in work:
            fn()

    # the reference's protocol (timed_repeat: 2 warm-up + 5 timed passes,
    # timing_ops.py:76-100), continued until about 12 s of CPU work are on the clock
    for _ in range(2):
        one_pass()
    passes = 0
    t0 = time.perf_counter()
    while passes < 5 or (time.perf_counter() - t0 < 12.0 and passes < 2000):
        one_pass()
        passes += 1
    sec = (time.perf_counter() - t0) / passes
    scaled = LayerLike(cfg, B, T)
    distinct = int(np.unique(ids).size) if cfg.embed else None
    total = sum(f + b for f, b in op_bytes(scaled, distinct).values())
    return {"value": round(total / sec / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"numpy restatement of the CPU kernels, fwd+bwd of every op on rows {rows} of {cfg.N} "
                      f"(B={B} T={T}), 2 warm-up + {passes} timed passes, {sec * 1e3:.1f} ms/pass; "
                      f"os.cpu_count()={os.cpu_count()}, numpy {np.__version__}",
            "tokens_per_s": round(rows / sec, 1)}


def LayerLike(cfg, B, T):
    from dataclasses import replace
    return replace(cfg, B=B, T=T)


def measured_traffic(cfg, case):
    """HBM bytes per launch of the case's kernel from the committed counter summary:
    entries of this configuration whose kernel name contains every word of
    case.kernel; None when the summary has no such kernel (never a guess)"""
    try:
        table = json.loads(TRAFFIC_FILE.read_text())["configs"].get(str(cfg.index), {})
    except (OSError, ValueError, KeyError):
        return None, None
    words = case.kernel.split()
    hits = [(k, v) for k, v in table.items() if all(w in k for w in words)]
    if len(hits) != 1:
        return None, None
    name, row = hits[0]
    return name, int(round(row["read_bytes"] + row["written_bytes"]))


def min_frac(rows):
    """the op and direction of the step furthest below the roofline"""
    step = [r for r in rows if r["dir"] in ("fwd", "bwd")]
    worst = min(step, key=lambda r: r["frac_hbm"])
    return [f"{worst['op']} {worst['dir']}", worst["frac_hbm"]]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", type=int, default=5, help="index into autograd_amd.configs.CONFIGS")
    ap.add_argument("--iters", type=int, default=30, help="launches per op in the per-op timing")
    ap.add_argument("--workload-only", action="store_true", help="skip the per-op tables of the other configs")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--detail", default=str(ROOT / "gpurun_out" / "bench_per_op.json"),
                    help="file that receives the per-op tables of every configuration")
    ap.add_argument("--exact-iters", action="store_true",
                    help="time each op over exactly --iters launches and shorten the clock spin-up "
                         "(for rocprofv3 --pmc runs, which serialise every dispatch)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this build has no multi-GPU path (asked for --gpus {args.gpus}); "
              "every op is row-independent and would shard over rows with one all-reduce of the parameter grads",
              file=sys.stderr)
        return 2
    cfg = CONFIGS[args.config]
    ctx = capi.Context(0)
    spin_up(ctx, 0.02 if args.exact_iters else 0.25)
    cases, step_bytes, wall = run_workload(ctx, cfg, args.steps, args.warmup, args.iters, args.exact_iters)
    ms_per_step = wall * 1e3 / args.steps
    gbps = step_bytes * args.steps / wall / 1e9
    timed = [c for c in cases if c.in_step]
    dom = max(timed, key=lambda c: c.us)
    dom_gbps = dom.nbytes / (dom.us * 1e-6) / 1e9
    dom_kernel, dom_traffic = measured_traffic(cfg, dom)

    def title(c):
        return f"configs[{c.index}] {c.name} ({c.dtype})"

    tables = {title(cfg): [case_row(c) for c in cases]}
    print(json.dumps({"per_op": title(cfg), "rows": tables[title(cfg)]}), flush=True)
    detail = {"workload": title(cfg), "per_op": tables}
    if not args.workload_only:
        detail["graph_replay"] = graph_replay(ctx, CONFIGS[0])
        print(json.dumps({"graph_replay": detail["graph_replay"]}), flush=True)
        for other in CONFIGS:
            if other.index != cfg.index:
                tables[title(other)] = run_config(ctx, other, args.iters)
                print(json.dumps({"per_op": title(other), "rows": tables[title(other)]}), flush=True)
        # the host path beside the C ABI, at two small, a middle and the largest configuration
        detail["runtime_path"] = [runtime_path(CONFIGS[i], tables[title(CONFIGS[i])], ctx=ctx) for i in (1, 2, 4, 5)]
        print(json.dumps({"runtime_path": detail["runtime_path"]}), flush=True)
    ctx.synchronize()
    ctx.close()
    try:
        Path(args.detail).parent.mkdir(parents=True, exist_ok=True)
        Path(args.detail).write_text(json.dumps(detail, indent=1))
    except OSError as err:
        print(f"could not write {args.detail}: {err}", file=sys.stderr)

    result = {
        "metric": METRIC, "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 I/O, fp32 arithmetic" if cfg.dtype == "bf16" else "f32", "data": "synthetic",
        "config": {"workload": f"configs[{cfg.index}] {cfg.name}: B={cfg.B} T={cfg.T} C={cfg.C} V={cfg.V}, "
                               f"ops {'/'.join(dict.fromkeys(c.op for c in timed))} fwd+bwd",
                   "step_MB": round(step_bytes / 1e6, 1)},
        "tokens_per_s": round(cfg.N * args.steps / wall, 1),
        "pct_of_hbm_peak": round(100 * gbps / HBM_PEAK_GBS, 2),
        "roofline": {"bound": "hbm", "kernel": dom_kernel or dom.kernel, "op": f"{dom.op} {dom.direction}",
                     "achieved": round(dom_gbps, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(dom_gbps / HBM_PEAK_GBS, 4), "traffic": dom_traffic,
                     "launch_us": round(dom.us, 2), "algorithmic_bytes": dom.nbytes,
                     "same_bytes_copy_us": round(dom.copy_us, 2) if getattr(dom, "copy_us", None) else None},
        "min_frac": {t.split(" ")[0]: min_frac(rows) for t, rows in tables.items()},
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(cfg)
    line = json.dumps(result, separators=(",", ":"))
    if len(line) >= 1800:          # the compact line stays compact: the long free-text fields give way first
        result["cpu_baseline"]["sample"] = result.get("cpu_baseline", {}).get("sample", "")[:120] if "cpu_baseline" in result else ""
        result["config"]["workload"] = result["config"]["workload"][:160]
        result["roofline"]["kernel"] = str(result["roofline"]["kernel"])[:80]
        line = json.dumps(result, separators=(",", ":"))
    print(line, flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
