"""Parity at the full shapes of the benchmark configurations, through the C ABI.

The CPU restatement needs seconds per million elements, so at these sizes the
inputs are a seeded block of R rows repeated down the tensor (on the device),
which turns the oracle's answer on the block into the exact answer for the
whole tensor:

  * row-wise outputs (norm y / dx, activations, rotary) repeat with the block,
    and the first, a middle and the last repetition are compared with the oracle;
  * column sums are linear: d(gamma), d(beta) of the whole tensor are `reps`
    times the block's;
  * the embedding gradient is compared on sampled columns against the row-order
    loop over ALL N ids, plus the size-independent invariants (column checksum,
    untouched rows exactly zero, run-to-run determinism);
  * rotary: backward(forward(x)) returns x.

Token ids are drawn for the full N with each configuration's distribution.
"""
import ctypes as C

import numpy as np
import pytest

from autograd_amd import capi
from autograd_amd.configs import CONFIGS
from oracle import closed_form as cf
from oracle import cpu_ops as K

from tests.helpers import assert_bf16_close, assert_fp32_close, assert_fp32_parity, from_bf16_bits, to_bf16_bits

pytestmark = pytest.mark.gpu

BLOCK_ROWS = 1024
FULL = [c for c in CONFIGS if c.index >= 1]
IDS = [f"cfg{c.index}-{c.name}" for c in FULL]


def vp(d, off=0):
    return C.c_void_p(d.ptr + off) if d is not None else None


class Dev:
    """device buffers of one test, freed together"""

    def __init__(self, ctx, cfg):
        self.ctx, self.cfg, self.held = ctx, cfg, []
        self.bf16 = cfg.dtype == "bf16"
        self.dt = capi.BF16 if self.bf16 else capi.F32
        self.np_dt = np.uint16 if self.bf16 else np.float32
        self.e = cfg.esize

    def host(self, a):
        """fp32 values -> (storage array to upload, the fp32 values the device will see)"""
        a = np.ascontiguousarray(a, dtype=np.float32)
        if not self.bf16:
            return a, a
        bits = to_bf16_bits(a)
        return bits, from_bf16_bits(bits)

    def keep(self, d):
        self.held.append(d)
        return d

    def upload(self, a):
        return self.keep(self.ctx.upload(np.ascontiguousarray(a)))

    def empty(self, n_items, dtype=None):
        return self.keep(self.ctx.empty((int(n_items),), dtype or self.np_dt))

    def tiled(self, block, reps):
        """device tensor holding `block` repeated `reps` times along axis 0"""
        block = np.ascontiguousarray(block)
        src = self.upload(block)
        if reps == 1:
            return src
        dst = self.keep(self.ctx.empty((reps * block.size,), block.dtype))
        for r in range(reps):
            self.ctx.call("agrad_copy", vp(src), vp(dst, r * block.nbytes), block.nbytes)
        return dst

    def rows(self, d, first_row, n_rows, width, dtype=None):
        dtype = np.dtype(dtype or self.np_dt)
        out = np.empty((n_rows, width), dtype=dtype)
        self.ctx.call("agrad_copy_to_host", d.ptr, first_row * width * dtype.itemsize,
                      out.ctypes.data_as(C.c_void_p), out.nbytes)
        return out

    def values(self, a):
        return from_bf16_bits(a) if self.bf16 else a

    def close_enough(self, got, ref, what):
        if self.bf16:
            assert_bf16_close(self.values(got), ref, what)
        else:
            assert_fp32_close(got, ref, what)

    def release(self):
        self.ctx.synchronize()
        for d in self.held:
            d.free()
        self.held = []


def sample_blocks(reps):
    return sorted({0, reps // 2, reps - 1})


def token_ids(cfg, rng):
    if cfg.embed_dist.startswith("zipf"):
        s = float(cfg.embed_dist[4:])
        p = np.arange(1, cfg.V + 1, dtype=np.float64) ** -s
        p /= p.sum()
        return rng.choice(cfg.V, size=cfg.N, p=p).astype(np.int32)
    return rng.integers(0, cfg.V, size=cfg.N, dtype=np.int32)


# ---------------------------------------------------------------------------------
@pytest.mark.parametrize("cfg", FULL, ids=IDS)
def test_norm_full_shape(ctx, cfg):
    rng = np.random.default_rng(cfg.seed)
    N, Cw = cfg.N, cfg.C
    R = min(BLOCK_ROWS, N)
    reps = N // R
    assert reps * R == N
    d = Dev(ctx, cfg)
    kind = capi.NORM_LAYER if cfg.norm == "layer" else capi.NORM_RMS
    try:
        xs, xv = d.host(rng.standard_normal((R, Cw)))
        rs, rv = d.host(rng.standard_normal((R, Cw))) if cfg.norm_residual else (None, None)
        dys, dyv = d.host(rng.standard_normal((R, Cw)))
        drs, drv = d.host(rng.standard_normal((R, Cw))) if cfg.norm_residual else (None, None)
        gamma = (1 + 0.02 * rng.standard_normal(Cw)).astype(np.float32)
        beta = (0.02 * rng.standard_normal(Cw)).astype(np.float32) if cfg.norm == "layer" else None

        x = d.tiled(xs, reps)
        res = d.tiled(rs, reps) if rs is not None else None
        g, b = d.upload(gamma), (d.upload(beta) if beta is not None else None)
        y = d.empty(N * Cw)
        h = d.empty(N * Cw) if res is not None else None
        ctx.call("agrad_norm_forward", kind, d.dt, vp(x), vp(res), vp(g), vp(b), vp(h), vp(y), N, Cw, cfg.norm_eps)

        # oracle on the block
        # h = x + r is stored in the I/O type, and that stored value is what gets normalised
        hv = K.add_forward(xv, rv) if rv is not None else xv
        if d.bf16 and rv is not None:
            hv = K.round_bf16(hv)
        h_seen = hv
        if cfg.norm == "layer":
            y_ref = K.layernorm_forward(hv, gamma, beta, cfg.norm_eps)
        else:
            y_ref = K.rmsnorm_forward(hv, gamma, cfg.norm_eps)
        for blk in sample_blocks(reps):
            d.close_enough(d.rows(y, blk * R, R, Cw), y_ref, f"{cfg.name} norm y block {blk}")
            if h is not None:
                got_h = d.rows(h, blk * R, R, Cw)
                np.testing.assert_array_equal(got_h, to_bf16_bits(hv) if d.bf16 else hv)

        # backward from the h the forward wrote (what a training step does)
        saved = h if h is not None else x
        dy = d.tiled(dys, reps)
        dres = d.tiled(drs, reps) if drs is not None else None
        dx = d.empty(N * Cw)
        dgamma, dbeta = d.upload(np.zeros(Cw, np.float32)), (d.upload(np.zeros(Cw, np.float32)) if beta is not None else None)
        ws_bytes = ctx.lib.agrad_norm_backward_workspace_bytes(N, Cw, d.dt)
        ws = d.empty(max(ws_bytes, 1), np.uint8)
        ctx.call("agrad_norm_backward", kind, d.dt, vp(saved), vp(dy), vp(g), vp(dres), vp(dx), None,
                 vp(dgamma), vp(dbeta), vp(ws), ws_bytes, N, Cw, cfg.norm_eps, 0)
        ctx.synchronize()

        dx_ref = np.zeros((R, Cw), np.float32)
        if cfg.norm == "layer":
            dg_blk, db_blk = np.zeros(Cw, np.float32), np.zeros(Cw, np.float32)
            K.layernorm_backward_into(h_seen, gamma, dyv, cfg.norm_eps, dx_ref, dg_blk, db_blk)
            _, dg64, db64 = cf.layernorm_grads(h_seen, gamma, dyv, cfg.norm_eps)
        else:
            dg_blk, db_blk, db64 = np.zeros(Cw, np.float32), None, None
            K.rmsnorm_backward_into(h_seen, gamma, dyv, cfg.norm_eps, dx_ref, dg_blk)
            _, dg64 = cf.rmsnorm_grads(h_seen, gamma, dyv, cfg.norm_eps)
        if drv is not None:
            dx_ref = dx_ref + drv
        for blk in sample_blocks(reps):
            d.close_enough(d.rows(dx, blk * R, R, Cw), dx_ref, f"{cfg.name} norm dx block {blk}")

        # linearity: the whole tensor's column sums are reps x the block's.  An fp32
        # sum of n terms is good to a few eps * sum|term| whatever the order, so the
        # budget is 1e-7 * sum|term| (the terms do not cancel like a random walk here:
        # the block repeats)
        h64 = h_seen.astype(np.float64)
        if cfg.norm == "layer":
            xhat = (h64 - h64.mean(-1, keepdims=True)) / np.sqrt(h64.var(-1, keepdims=True) + cfg.norm_eps)
        else:
            xhat = h64 / np.sqrt((h64 * h64).mean(-1, keepdims=True) + cfg.norm_eps)
        got_dg = dgamma.download()
        tol = 1e-7 * reps * np.abs(dyv * xhat).sum(0) + 2e-6 * np.abs(reps * dg64)
        assert (np.abs(got_dg - reps * dg64) <= tol).all(), np.abs(got_dg - reps * dg64).max()
        assert_fp32_close(got_dg, reps * dg_blk, "dgamma vs cpu", rtol=1e-5, atol=1e-4 * np.sqrt(N / 14))
        if dbeta is not None:
            got_db = dbeta.download()
            tol = 1e-7 * reps * np.abs(dyv).astype(np.float64).sum(0) + 2e-6 * np.abs(reps * db64)
            assert (np.abs(got_db - reps * db64) <= tol).all(), np.abs(got_db - reps * db64).max()
    finally:
        d.release()


# ---------------------------------------------------------------------------------
@pytest.mark.parametrize("cfg", FULL, ids=IDS)
def test_activation_full_shape(ctx, cfg):
    rng = np.random.default_rng(cfg.seed + 100)
    N, H = cfg.N, cfg.act_width
    R = min(256, N)
    reps = N // R
    d = Dev(ctx, cfg)
    try:
        if cfg.act == "swiglu":
            gus, guv = d.host(rng.standard_normal((R, 2 * H)))
            dhs, dhv = d.host(rng.standard_normal((R, H)))
            gu, dh = d.tiled(gus, reps), d.tiled(dhs, reps)
            hout = d.empty(N * H)
            ctx.call("agrad_swiglu_forward", d.dt, vp(gu), vp(hout), N, H)
            h_ref = K.swiglu_forward(guv)
            for blk in sample_blocks(reps):
                d.close_enough(d.rows(hout, blk * R, R, H), h_ref, f"{cfg.name} swiglu h block {blk}")
            # backward in place on gu, as the arena does it
            ctx.call("agrad_swiglu_backward", d.dt, vp(gu), vp(dh), vp(gu), N, H, 0)
            ctx.synchronize()
            dgu_ref = K.swiglu_backward(guv, dhv)
            for blk in sample_blocks(reps):
                d.close_enough(d.rows(gu, blk * R, R, 2 * H), dgu_ref, f"{cfg.name} swiglu dgu block {blk}")
        else:
            fwd, bwd = ("agrad_gelu_forward", "agrad_gelu_backward") if cfg.act == "gelu" else ("agrad_relu2_forward", "agrad_relu2_backward")
            xs, xv = d.host(rng.standard_normal((R, H)))
            dys, dyv = d.host(rng.standard_normal((R, H)))
            x, dy = d.tiled(xs, reps), d.tiled(dys, reps)
            y, dx = d.empty(N * H), d.empty(N * H)
            ctx.call(fwd, d.dt, vp(x), vp(y), N * H)
            ctx.call(bwd, d.dt, vp(x), vp(dy), vp(dx), N * H, 0)
            ctx.synchronize()
            if cfg.act == "gelu":
                y_ref = K.gelu_forward(xv)
                dx_ref = np.zeros_like(xv)
                K.gelu_backward_into(xv, dyv, dx_ref)
            else:
                y_ref = K.relu2_forward(xv)
                dx_ref = np.zeros_like(xv)
                K.relu2_backward_into(xv, dyv, dx_ref)
            for blk in sample_blocks(reps):
                d.close_enough(d.rows(y, blk * R, R, H), y_ref, f"{cfg.name} {cfg.act} y block {blk}")
                got = d.rows(dx, blk * R, R, H)
                if cfg.act == "gelu" and not d.bf16:
                    # the device derivative has no cancellation in 1 - tanh^2; in the
                    # far tails the CPU form loses bits, so hold both to float64 there
                    core = np.abs(xv) <= 4.5
                    assert_fp32_close(got[core], dx_ref[core], "gelu dx core")
                    ref64 = cf.gelu_grad(xv) * dyv.astype(np.float64)
                    assert_fp32_parity(got, dx_ref, ref64, "gelu dx")
                    assert (np.abs(got - ref64) <= 1e-6 + 1e-6 * np.abs(ref64)).all()
                else:
                    d.close_enough(got, dx_ref, f"{cfg.name} {cfg.act} dx block {blk}")
    finally:
        d.release()


# ---------------------------------------------------------------------------------
@pytest.mark.parametrize("cfg", [c for c in FULL if c.rope], ids=[f"cfg{c.index}" for c in FULL if c.rope])
def test_rope_full_shape(ctx, cfg):
    rng = np.random.default_rng(cfg.seed + 200)
    Hq, Hkv, D, theta, sign = cfg.rope
    B, T = cfg.B, cfg.T
    d = Dev(ctx, cfg)
    try:
        # one batch entry is the block (the rotation depends on t, not on b)
        qs, qv = d.host(rng.standard_normal((T, Hq, D)))
        ks, kv = d.host(rng.standard_normal((T, Hkv, D)))
        cos, sin = K.rope_tables(T, D, theta)
        q, k = d.tiled(qs.reshape(T, -1), B), d.tiled(ks.reshape(T, -1), B)
        dc, ds = d.upload(cos), d.upload(sin)
        ctx.call("agrad_rope_qk", d.dt, vp(q), vp(k), vp(dc), vp(ds), B, T, Hq, Hkv, D, sign, 0)
        ctx.synchronize()
        q_ref, k_ref = qv[None].copy(), kv[None].copy()
        K.rope_signed(q_ref, k_ref, cos, sin, sign, False)      # in place
        for b in sample_blocks(B):
            gq = d.rows(q, b * T, T, Hq * D)
            gk = d.rows(k, b * T, T, Hkv * D)
            if d.bf16:
                assert_bf16_close(d.values(gq), q_ref.reshape(T, -1), "rope q")
                assert_bf16_close(d.values(gk), k_ref.reshape(T, -1), "rope k")
            else:
                # same multiplies and adds in the same order: identical bits
                np.testing.assert_array_equal(gq, q_ref.reshape(T, -1))
                np.testing.assert_array_equal(gk, k_ref.reshape(T, -1))
        # the backward rotation undoes the forward one, over the whole tensor
        ctx.call("agrad_rope_qk", d.dt, vp(q), vp(k), vp(dc), vp(ds), B, T, Hq, Hkv, D, sign, 1)
        ctx.synchronize()
        for b in sample_blocks(B):
            back_q = d.values(d.rows(q, b * T, T, Hq * D))
            back_k = d.values(d.rows(k, b * T, T, Hkv * D))
            tol = 2.5e-2 if d.bf16 else 2e-6
            assert np.abs(back_q - qv.reshape(T, -1)).max() <= tol * max(1.0, np.abs(qv).max())
            assert np.abs(back_k - kv.reshape(T, -1)).max() <= tol * max(1.0, np.abs(kv).max())
    finally:
        d.release()


# ---------------------------------------------------------------------------------
@pytest.mark.parametrize("cfg", FULL, ids=IDS)
def test_embedding_full_shape(ctx, cfg):
    rng = np.random.default_rng(cfg.seed + 300)
    N, Cw, V, T = cfg.N, cfg.C, cfg.V, cfg.T
    d = Dev(ctx, cfg)
    try:
        ids = token_ids(cfg, rng)
        # the table is a block of P distinct rows repeated: row v holds block[v % P]
        P = 1024
        wblk_s, wblk_v = d.host(0.02 * rng.standard_normal((P, Cw)))
        reps_w = (V + P - 1) // P
        W = d.tiled(wblk_s, reps_w)            # at least V rows
        d_ids = d.upload(ids)
        wpe = wpe_s = None
        if cfg.embed == "gather_sum":
            wpe_s, wpe_v = d.host(0.02 * rng.standard_normal((T, Cw)))
            wpe = d.upload(wpe_s)
        out = d.empty(N * Cw)
        ctx.call("agrad_gather_forward", d.dt, vp(d_ids), vp(W), vp(wpe), vp(out), N, T, Cw, V)
        ctx.synchronize()
        got = d.rows(out, 0, N, Cw)
        if wpe is None:
            # a gather moves bits
            np.testing.assert_array_equal(got, wblk_s[ids % P])
        else:
            ref = K.embedding_sum_forward(ids.reshape(cfg.B, T), wblk_v[np.arange(V) % P], wpe_v).reshape(N, Cw)
            d.close_enough(got, ref, f"{cfg.name} gather-sum")
        del got

        # gradient: dY is a block of R rows repeated
        R = 2048
        dys, dyv = d.host(rng.standard_normal((R, Cw)))
        dY = d.tiled(dys, N // R)
        dW = d.empty(V * Cw)
        ws_bytes = ctx.lib.agrad_embedding_backward_workspace_bytes(N, Cw, V, d.dt)
        ws = d.empty(max(ws_bytes, 1), np.uint8)
        ctx.call("agrad_fill", dW.ptr, 0, 0, d.e, V * Cw)
        ctx.call("agrad_embedding_backward", d.dt, vp(d_ids), vp(dY), vp(dW), vp(ws), ws_bytes, N, Cw, V,
                 capi.ACC_PARAM_GRAD)
        ctx.synchronize()
        got = d.rows(dW, 0, V, Cw)
        # untouched rows are exactly zero
        counts = np.bincount(ids, minlength=V)
        assert not got[counts == 0].any()
        gotv = d.values(got) if d.bf16 else got
        # sampled columns against the row-order loop over all N ids
        cols = np.unique(np.concatenate([[0, 1, Cw // 2, Cw - 1], rng.integers(0, Cw, 28)]))
        ref = np.zeros((V, cols.size), np.float32)
        np.add.at(ref, ids, np.ascontiguousarray(dyv[:, cols])[np.arange(N) % R])
        longest = int(counts.max())
        if d.bf16:
            # an fp32 sum rounded to bf16 once (half an ulp = 2^-9 relative) plus the
            # fp32 re-association noise of a long run
            err = np.abs(gotv[:, cols] - ref)
            assert (err <= 6e-3 * np.abs(ref) + 1e-5 * np.sqrt(max(longest, 1))).all(), err.max()
        else:
            assert_fp32_close(gotv[:, cols], ref, f"{cfg.name} dW", rtol=1e-5, atol=max(2e-6, 2.5e-7 * longest))
        # column checksum: sum_v dW[v] = sum_n dY[n]
        total = dyv.sum(0, dtype=np.float64) * (N // R)
        budget = np.sqrt(N) * (2e-2 if d.bf16 else 1e-3)
        assert np.abs(gotv.sum(0, dtype=np.float64) - total).max() <= budget
        # a second run produces the same bits (no atomics anywhere)
        ctx.call("agrad_fill", dW.ptr, 0, 0, d.e, V * Cw)
        ctx.call("agrad_embedding_backward", d.dt, vp(d_ids), vp(dY), vp(dW), vp(ws), ws_bytes, N, Cw, V,
                 capi.ACC_PARAM_GRAD)
        ctx.synchronize()
        np.testing.assert_array_equal(got, d.rows(dW, 0, V, Cw))

        if wpe is not None:
            dwpe = d.empty(T * Cw)
            ctx.call("agrad_pos_embedding_backward", d.dt, vp(dY), vp(dwpe), cfg.B, T, Cw, 0)
            ctx.synchronize()
            ref = dyv[np.arange(N) % R].reshape(cfg.B, T, Cw).astype(np.float64).sum(0)
            gp = d.values(d.rows(dwpe, 0, T, Cw))
            assert np.abs(gp - ref).max() <= (1e-2 if d.bf16 else 1e-5) * max(1.0, np.abs(ref).max())
    finally:
        d.release()


# ---------------------------------------------------------------------------------
@pytest.mark.parametrize("cfg", FULL, ids=IDS)
def test_cross_entropy_full_shape(ctx, cfg):
    """logits [N, V] at the configuration's N and vocabulary: a block of R distinct
    rows repeated, labels drawn for all N rows.  The loss of every row follows from
    the block's log-sum-exp; the gradient is compared on sampled rows, including the
    first and last rows of the tensor (the backward kernel cuts very large tensors
    into slabs of rows)."""
    from scipy.special import logsumexp
    rng = np.random.default_rng(cfg.seed + 400)
    N, V = cfg.N, cfg.V
    R = 16
    d = Dev(ctx, cfg)
    try:
        xs, xv = d.host(3.0 * rng.standard_normal((R, V)))
        labels = rng.integers(0, V, N, dtype=np.int32)
        dloss = rng.standard_normal(N).astype(np.float32)
        x = d.tiled(xs, N // R)
        dl, dg = d.upload(labels), d.upload(dloss)
        loss, lse = d.empty(N, np.float32), d.empty(N, np.float32)
        dx = d.empty(N * V)
        ctx.call("agrad_cross_entropy_forward", d.dt, vp(x), vp(dl), vp(loss), vp(lse), N, V)
        ctx.call("agrad_cross_entropy_backward", d.dt, vp(x), vp(dl), vp(dg), vp(lse), vp(dx), N, V, 0)
        ctx.synchronize()
        lse64 = logsumexp(xv.astype(np.float64), axis=-1)
        blk = np.arange(N) % R
        want_loss = lse64[blk] - xv[blk, labels].astype(np.float64)
        tol = 1e-4 if d.bf16 else 1e-5            # bf16 logits go through the hardware exp2
        got_loss = loss.download()
        assert np.abs(got_loss - want_loss).max() <= tol * max(1.0, np.abs(want_loss).max())
        assert np.abs(lse.download() - lse64[blk]).max() <= tol * max(1.0, np.abs(lse64).max())
        for n in sorted({0, 1, R - 1, N // 2 + 3, N - R, N - 1} | set(rng.integers(0, N, 6).tolist())):
            got = d.rows(dx, n, 1, V)[0]
            ref = np.zeros((1, V), np.float32)
            K.cross_entropy_backward_into(xv[n % R][None], labels[n:n + 1], dloss[n:n + 1], ref)
            d.close_enough(got[None], ref, f"{cfg.name} dlogits row {n}")
    finally:
        d.release()
