"""Column sums of parameter gradients left pending and folded in one launch.

A backward call with AGRAD_DEFER_PARAM_GRAD runs its main kernel only; the partial rows
wait in its workspace and agrad_finalize_param_grads folds every pending job at once.
The batched fold runs, per job, the workgroups, loads and additions of the job's own second
launch, so every comparison here is for EQUAL BITS with the per-call path (whose values
the kernel tests hold to the CPU restatement): dgamma / dbeta of several norms of different
widths, types and accumulate modes in one fold; the explicit job-list form; a bias
gradient; whole graphs through Runtime with the deferral on and off; and a recorded graph.
"""
import ctypes as C

import numpy as np
import pytest

from autograd_amd import capi
from autograd_amd.op import AddLayerNormOp, AddOp, BiasGELUOp, LayerNormOp, RMSNormOp
from autograd_amd.runtime import Runtime
from autograd_amd.tensor import Tensor
from tests import gpu_ops as G
from tests.helpers import to_bf16_bits

pytestmark = pytest.mark.gpu
SEED = 1333


def _p(d):
    return C.c_void_p(d.ptr) if d is not None else None


class _NormCase:
    """operands of one norm backward on the device, with its own workspace"""

    def __init__(self, ctx, rng, kind, rows, Cw, bf16=False, accumulate=False, bf16_grads=False):
        self.ctx, self.kind, self.rows, self.C = ctx, kind, rows, Cw
        self.dt = capi.BF16 if bf16 else capi.F32
        x = rng.standard_normal((rows, Cw), dtype=np.float32)
        dy = rng.standard_normal((rows, Cw), dtype=np.float32)
        self.x = ctx.upload(to_bf16_bits(x) if bf16 else x)
        self.dy = ctx.upload(to_bf16_bits(dy) if bf16 else dy)
        self.gamma = ctx.upload((1 + 0.02 * rng.standard_normal(Cw)).astype(np.float32))
        self.dx = ctx.empty((rows, Cw), np.uint16 if bf16 else np.float32)
        self.flags = (capi.ACC_PARAM_GRAD if accumulate else 0) | (capi.PARAM_GRAD_BF16 if bf16_grads else 0)
        gtype = np.uint16 if bf16_grads else np.float32
        init = rng.standard_normal(Cw).astype(np.float32)
        self.init = to_bf16_bits(init) if bf16_grads else init
        self.dgamma = ctx.empty((Cw,), gtype)
        self.dbeta = ctx.empty((Cw,), gtype) if kind == capi.NORM_LAYER else None
        self.ws_bytes = ctx.lib.agrad_norm_backward_workspace_bytes(rows, Cw, self.dt)
        self.ws = ctx.empty((max(self.ws_bytes, 1),), np.uint8)

    def reset(self):
        for d in (self.dgamma, self.dbeta):
            if d is not None:
                self.ctx.call("agrad_copy_from_host", d.buffer_id, 0, self.init.ctypes.data_as(C.c_void_p), self.init.nbytes)
        self.ctx.call("agrad_fill", self.dx.buffer_id, 0, 0, 1, self.dx.nbytes)

    def args(self, extra_flags=0):
        return (self.kind, self.dt, _p(self.x), _p(self.dy), _p(self.gamma), None, _p(self.dx), None,
                _p(self.dgamma), _p(self.dbeta), _p(self.ws), self.ws_bytes, self.rows, self.C, 1e-5,
                self.flags | extra_flags)

    def results(self):
        return (self.dx.download(), self.dgamma.download(), None if self.dbeta is None else self.dbeta.download())

    def free(self):
        for d in (self.x, self.dy, self.gamma, self.dx, self.dgamma, self.dbeta, self.ws):
            if d is not None:
                d.free()


def _cases(ctx, rng):
    return [
        _NormCase(ctx, rng, capi.NORM_LAYER, 2048, 384),
        _NormCase(ctx, rng, capi.NORM_RMS, 4096, 1536, accumulate=True),
        _NormCase(ctx, rng, capi.NORM_LAYER, 1000, 768, accumulate=True),
        _NormCase(ctx, rng, capi.NORM_RMS, 777, 4096, bf16=True),
        _NormCase(ctx, rng, capi.NORM_LAYER, 300, 50),                       # scalar columns: a launch of its own
        _NormCase(ctx, rng, capi.NORM_RMS, 1024, 1536, bf16_grads=True, accumulate=True),
        _NormCase(ctx, rng, capi.NORM_LAYER, 5, 128),
    ]


def _pending(ctx):
    n = C.c_uint32(0)
    ctx.call("agrad_pending_param_grads", C.byref(n))
    return n.value


def test_deferred_norm_sums_equal_the_per_call_fold(ctx):
    rng = np.random.default_rng(SEED + 70)
    cases = _cases(ctx, rng)
    try:
        want = []
        for c in cases:
            c.reset()
            ctx.call("agrad_norm_backward", *c.args())
        ctx.synchronize()
        want = [c.results() for c in cases]
        for c in cases:
            c.reset()
            ctx.call("agrad_norm_backward", *c.args(capi.DEFER_PARAM_GRAD))
        assert _pending(ctx) == len(cases)
        ctx.call("agrad_finalize_param_grads")
        assert _pending(ctx) == 0
        ctx.synchronize()
        for i, c in enumerate(cases):
            for name, got, ref in zip(("dx", "dgamma", "dbeta"), c.results(), want[i]):
                if ref is not None:
                    np.testing.assert_array_equal(got, ref, err_msg=f"case {i} {name}")
        # a synchronise folds what is pending: nothing a caller waits for stays unfolded
        cases[0].reset()
        ctx.call("agrad_norm_backward", *cases[0].args(capi.DEFER_PARAM_GRAD))
        assert _pending(ctx) == 1
        ctx.synchronize()
        assert _pending(ctx) == 0
        np.testing.assert_array_equal(cases[0].results()[1], want[0][1])
    finally:
        ctx.synchronize()
        for c in cases:
            c.free()


def test_more_jobs_than_one_launch_takes(ctx):
    """40 pending sums: two batched launches"""
    rng = np.random.default_rng(SEED + 71)
    cases = [_NormCase(ctx, rng, capi.NORM_RMS if i % 2 else capi.NORM_LAYER, 257 + 13 * i, 128 + 64 * (i % 5))
             for i in range(40)]
    try:
        for c in cases:
            c.reset()
            ctx.call("agrad_norm_backward", *c.args())
        ctx.synchronize()
        want = [c.results() for c in cases]
        for c in cases:
            c.reset()
            ctx.call("agrad_norm_backward", *c.args(capi.DEFER_PARAM_GRAD))
        assert _pending(ctx) == 40
        ctx.call("agrad_finalize_param_grads")
        ctx.synchronize()
        for i, c in enumerate(cases):
            for name, got, ref in zip(("dx", "dgamma", "dbeta"), c.results(), want[i]):
                if ref is not None:
                    np.testing.assert_array_equal(got, ref, err_msg=f"case {i} {name}")
    finally:
        ctx.synchronize()
        for c in cases:
            c.free()


def test_explicit_job_list(ctx):
    """agrad_norm_backward_partial + agrad_colsum_finalize_many: the caller keeps the jobs"""
    rng = np.random.default_rng(SEED + 72)
    cases = _cases(ctx, rng)[:4]
    try:
        for c in cases:
            c.reset()
            ctx.call("agrad_norm_backward", *c.args())
        ctx.synchronize()
        want = [c.results() for c in cases]
        jobs = (capi.ColsumJob * len(cases))()
        for i, c in enumerate(cases):
            c.reset()
            ctx.call("agrad_norm_backward_partial", *c.args(), C.byref(jobs[i]))
            assert jobs[i].partial_rows > 0 and jobs[i].C == c.C
        assert _pending(ctx) == 0
        ctx.call("agrad_colsum_finalize_many", C.cast(jobs, C.c_void_p), len(cases))
        ctx.synchronize()
        for i, c in enumerate(cases):
            for name, got, ref in zip(("dx", "dgamma", "dbeta"), c.results(), want[i]):
                if ref is not None:
                    np.testing.assert_array_equal(got, ref, err_msg=f"case {i} {name}")
        # nothing to fold: dx only
        c = cases[0]
        job = capi.ColsumJob()
        ctx.call("agrad_norm_backward_partial", c.kind, c.dt, _p(c.x), _p(c.dy), _p(c.gamma), None, _p(c.dx), None,
                 None, None, None, 0, c.rows, c.C, 1e-5, 0, C.byref(job))
        assert job.partial_rows == 0
        # a job with partial rows and no destination is refused
        bad = (capi.ColsumJob * 1)()
        bad[0].partial_a, bad[0].partial_rows, bad[0].C = jobs[0].partial_a, 4, 4
        with pytest.raises(capi.AgradError):
            ctx.call("agrad_colsum_finalize_many", C.cast(bad, C.c_void_p), 1)
    finally:
        ctx.synchronize()
        for c in cases:
            c.free()


def test_jobs_that_share_a_destination_keep_their_order(ctx):
    """a gamma tied between two norms: the first call stores its gradient, the second adds to
    it; left pending, the two folds must still happen one after the other"""
    rng = np.random.default_rng(SEED + 77)
    a = _NormCase(ctx, rng, capi.NORM_LAYER, 3000, 384)
    b = _NormCase(ctx, rng, capi.NORM_LAYER, 2500, 384, accumulate=True)
    others = [_NormCase(ctx, rng, capi.NORM_RMS, 1000, 384) for _ in range(3)]
    try:
        def run(extra):
            a.reset()
            ctx.call("agrad_norm_backward", *a.args(extra))
            for o in others:
                o.reset()
                ctx.call("agrad_norm_backward", *o.args(extra))
            args = list(b.args(extra))
            args[8], args[9] = _p(a.dgamma), _p(a.dbeta)        # b adds into a's gradients
            ctx.call("agrad_norm_backward", *args)
            if extra:
                assert _pending(ctx) == 5
                ctx.call("agrad_finalize_param_grads")
            ctx.synchronize()
            return a.dgamma.download(), a.dbeta.download()
        want = run(0)
        got = run(capi.DEFER_PARAM_GRAD)
        np.testing.assert_array_equal(got[0], want[0])
        np.testing.assert_array_equal(got[1], want[1])
    finally:
        ctx.synchronize()
        for c in [a, b] + others:
            c.free()


def test_noalloc_entry_point_refuses_deferral(ctx):
    rng = np.random.default_rng(SEED + 73)
    c = _NormCase(ctx, rng, capi.NORM_LAYER, 64, 128)
    try:
        with pytest.raises(capi.AgradError):
            ctx.call("agrad_norm_backward_noalloc", c.kind, c.dt, _p(c.x), _p(c.dy), _p(c.gamma), None, _p(c.dx), None,
                     _p(c.dgamma), _p(c.dbeta), c.rows, c.C, 1e-5, capi.DEFER_PARAM_GRAD)
    finally:
        c.free()


def test_deferred_bias_gradient(ctx):
    rng = np.random.default_rng(SEED + 74)
    lead, inner = 3000, 768
    g = ctx.upload(rng.standard_normal((lead, inner), dtype=np.float32))
    ws_bytes = ctx.lib.agrad_broadcast_grad_workspace_bytes(lead, inner)
    ws = ctx.empty((max(ws_bytes, 1),), np.uint8)
    out = [ctx.zeros((inner,), np.float32) for _ in range(2)]
    try:
        ctx.call("agrad_broadcast_add_backward", capi.F32, _p(g), _p(out[0]), _p(ws), ws_bytes, lead, inner, 0)
        ctx.synchronize()
        ctx.call("agrad_broadcast_add_backward", capi.F32, _p(g), _p(out[1]), _p(ws), ws_bytes, lead, inner,
                 capi.DEFER_PARAM_GRAD)
        assert _pending(ctx) == 1
        ctx.call("agrad_finalize_param_grads")
        ctx.synchronize()
        np.testing.assert_array_equal(out[1].download(), out[0].download())
    finally:
        G._free(g, ws, *out)


# ---- through the runtime ---------------------------------------------------------------
def _leaf(shape, grad, val, dtype=np.float32):
    return Tensor(shape=tuple(shape), dtype=dtype, device="hip", requires_grad=grad, init_val=np.asarray(val))


def _norm_stack(rng, layers=6, rows=1500, Cw=384):
    """x -> (add+LN) x layers with a bias-GELU and a bias add between them: 2 sums per norm,
    one per bias"""
    x = _leaf((rows, Cw), True, rng.standard_normal((rows, Cw), dtype=np.float32))
    params = {"x": x}
    h = x
    res = _leaf((rows, Cw), True, rng.standard_normal((rows, Cw), dtype=np.float32))
    params["res"] = res
    for i in range(layers):
        g = _leaf((Cw,), True, (1 + 0.02 * rng.standard_normal(Cw)).astype(np.float32))
        b = _leaf((Cw,), True, (0.02 * rng.standard_normal(Cw)).astype(np.float32))
        bias = _leaf((Cw,), True, (0.02 * rng.standard_normal(Cw)).astype(np.float32))
        params.update({f"g{i}": g, f"b{i}": b, f"bias{i}": bias})
        if i % 2 == 0:
            hh, y = AddLayerNormOp(eps=1e-5)(h, res, g, b)
            h = BiasGELUOp()(y, bias)
        else:
            y = LayerNormOp(eps=1e-5)(h, g, b)
            h = AddOp()(y, bias)
    gl = _leaf((Cw,), True, np.ones(Cw, np.float32))
    params["g_last"] = gl
    return RMSNormOp(eps=1e-6)(h, gl), params


def _run_stack(defer, capture=False):
    rng = np.random.default_rng(SEED + 75)
    out, params = _norm_stack(rng)
    up_np = np.random.default_rng(SEED + 76).standard_normal(out.shape, dtype=np.float32)
    rt = Runtime(device="hip", defer_param_grad_sums=defer)
    rt.loss = out
    rt.build_topo(out)
    rt.bind_memory()
    deferred = sum(1 for n in rt.topo if n.defer_param_grads)
    up = _leaf(out.shape, False, up_np)
    up.storage = rt.allocator.alloc(up.shape, up.dtype)
    rt.backend.init(up)

    def step():
        rt.zero_grad()
        rt.forward()
        rt.backend._launch("copy_kernel", [up, out.grad], [up.numel * 4, 0])   # device-side upstream gradient
        rt.backward_graph()

    def read():
        rt.backend.synchronize()
        return {k: rt.backend.copy_to_host(t.grad).copy() for k, t in params.items()}

    step()
    grads = read()
    if capture:
        graph = rt.capture(step)
        for replay in range(3):
            for t in params.values():          # eager work between replays: scribble over the gradients
                rt.backend.fill(t.grad, float(replay + 1))
            rt.backend.synchronize()
            graph.launch()
            again = read()
            for k in grads:
                np.testing.assert_array_equal(again[k], grads[k], err_msg=f"replay {replay} {k}")
        graph.destroy()
    rt.release()
    return grads, deferred


def test_runtime_folds_a_pass_in_one_launch_same_bits():
    base, n0 = _run_stack(defer=False)
    got, n1 = _run_stack(defer=True)
    assert n0 == 0 and n1 == 13          # 7 norms + 3 bias-GELUs + 3 bias adds
    for k in base:
        np.testing.assert_array_equal(got[k], base[k], err_msg=k)


def test_runtime_deferred_sums_inside_a_recorded_graph():
    base, _ = _run_stack(defer=False)
    got, _ = _run_stack(defer=True, capture=True)
    for k in base:
        np.testing.assert_array_equal(got[k], base[k], err_msg=k)
