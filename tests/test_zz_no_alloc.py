"""agrad_norm_backward_noalloc: the norm backward for callers that cannot allocate.

It takes no workspace: the partial dgamma / dbeta rows go to a fixed array the
library keeps on the GPU.  Each case runs it and agrad_norm_backward (workspace from
the caller) on the same seeded operands through the C ABI and asks for the same
bits, since both run the same kernels over the same grid: first a larger problem,
then a smaller one straight after, so that whatever the first call left in the
array is there when the second runs.
"""
import ctypes as C

import numpy as np
import pytest

from autograd_amd import capi
from oracle import closed_form as cf
from oracle import cpu_ops as K
from tests.helpers import assert_fp32_parity, to_bf16_bits

pytestmark = pytest.mark.gpu


def _p(d):
    return C.c_void_p(d.ptr) if d is not None else None


def _run(ctx, entry, kind, x, dy, gamma, dres, eps, want_beta):
    rows, Cw = x.shape
    dt = capi.BF16 if x.dtype == np.uint16 else capi.F32
    d_x, d_dy, d_g = ctx.upload(x), ctx.upload(dy), ctx.upload(gamma)
    d_res = ctx.upload(dres) if dres is not None else None
    d_dx = ctx.upload(np.full(x.shape, 7, dtype=x.dtype))
    d_dg = ctx.upload(np.full((Cw,), 3, np.float32))
    d_db = ctx.upload(np.full((Cw,), 5, np.float32)) if want_beta else None
    ws = None
    if entry == "agrad_norm_backward":
        ws_bytes = ctx.lib.agrad_norm_backward_workspace_bytes(rows, Cw, dt)
        ws = ctx.empty((max(ws_bytes, 1),), np.uint8)
        ctx.call(entry, kind, dt, _p(d_x), _p(d_dy), _p(d_g), _p(d_res), _p(d_dx), None, _p(d_dg), _p(d_db),
                 _p(ws), ws_bytes, rows, Cw, eps, 0)
    else:
        ctx.call(entry, kind, dt, _p(d_x), _p(d_dy), _p(d_g), _p(d_res), _p(d_dx), None, _p(d_dg), _p(d_db),
                 rows, Cw, eps, 0)
    ctx.synchronize()
    out = dict(dx=d_dx.download(), dgamma=d_dg.download(), dbeta=d_db.download() if d_db else None)
    for d in (d_x, d_dy, d_g, d_res, d_dx, d_dg, d_db, ws):
        if d is not None:
            d.free()
    return out


def _operands(seed, rows, Cw, bf16):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, Cw), dtype=np.float32)
    dy = rng.standard_normal((rows, Cw), dtype=np.float32)
    dres = rng.standard_normal((rows, Cw), dtype=np.float32)
    gamma = (1 + 0.02 * rng.standard_normal(Cw)).astype(np.float32)
    if bf16:
        x, dy, dres = to_bf16_bits(x), to_bf16_bits(dy), to_bf16_bits(dres)
    return x, dy, gamma, dres


@pytest.mark.parametrize("kind,bf16,first,second", [
    (capi.NORM_LAYER, False, (4096, 768), (300, 384)),     # several rows per wave, then fewer and narrower
    (capi.NORM_RMS, False, (2048, 1536), (64, 1536)),      # a wave per row; second call leaves most partial rows stale
    (capi.NORM_RMS, True, (4096, 4096), (1000, 1536)),     # bf16 rows, a workgroup per row, the widest benchmark shape
    (capi.NORM_LAYER, False, (512, 1001), (77, 130)),      # odd widths: the scalar kernels
])
def test_noalloc_matches_workspace_entry_point_twice(ctx, kind, bf16, first, second):
    for call, (rows, Cw) in enumerate((first, second)):
        x, dy, gamma, dres = _operands(20 + call, rows, Cw, bf16)
        want_beta = kind == capi.NORM_LAYER
        got = _run(ctx, "agrad_norm_backward_noalloc", kind, x, dy, gamma, dres, 1e-5, want_beta)
        ref = _run(ctx, "agrad_norm_backward", kind, x, dy, gamma, dres, 1e-5, want_beta)
        for name in ("dx", "dgamma", "dbeta"):
            if ref[name] is not None:
                np.testing.assert_array_equal(got[name], ref[name], err_msg=f"call {call} {name} rows={rows} C={Cw}")


def test_noalloc_against_cpu_restatement(ctx):
    """and once against the checker itself, after a larger call has used the array"""
    x, dy, gamma, dres = _operands(31, 3000, 768, False)
    _run(ctx, "agrad_norm_backward_noalloc", capi.NORM_LAYER, x, dy, gamma, None, 1e-5, True)
    x, dy, gamma, _ = _operands(32, 96, 384, False)
    got = _run(ctx, "agrad_norm_backward_noalloc", capi.NORM_LAYER, x, dy, gamma, None, 1e-5, True)
    dx, dg, db = np.zeros_like(x), np.zeros_like(gamma), np.zeros_like(gamma)
    K.layernorm_backward_into(x, gamma, dy, 1e-5, dx, dg, db)
    dx64, dg64, db64 = cf.layernorm_grads(x, gamma, dy, 1e-5)
    assert_fp32_parity(got["dx"], dx, dx64, "dx")
    assert_fp32_parity(got["dgamma"], dg, dg64, "dgamma")
    assert_fp32_parity(got["dbeta"], db, db64, "dbeta")


def test_noalloc_refuses_what_the_array_cannot_hold(ctx):
    rows, Cw = 4096, 8192          # 768 partial rows x 2 x 8192 x 4 B = 48 MiB
    assert ctx.lib.agrad_norm_backward_workspace_bytes(rows, Cw, capi.F32) > capi.NOALLOC_SCRATCH_BYTES
    x = ctx.zeros((rows, Cw), np.float32)
    dy = ctx.zeros((rows, Cw), np.float32)
    dx = ctx.zeros((rows, Cw), np.float32)
    dg = ctx.zeros((Cw,), np.float32)
    with pytest.raises(capi.AgradError) as err:
        ctx.call("agrad_norm_backward_noalloc", capi.NORM_RMS, capi.F32, _p(x), _p(dy), None, None, _p(dx), None,
                 _p(dg), None, rows, Cw, 1e-5, 0)
    assert err.value.code == capi.EINVAL and "scratch" in str(err.value)
    # the same shape without parameter gradients needs no partial rows and runs
    ctx.call("agrad_norm_backward_noalloc", capi.NORM_RMS, capi.F32, _p(x), _p(dy), None, None, _p(dx), None,
             None, None, rows, Cw, 1e-5, 0)
    ctx.synchronize()
    for d in (x, dy, dx, dg):
        d.free()


def test_noalloc_call_recorded_into_a_graph(ctx):
    """the use it is for: the call is recorded into a HIP graph (a recording may not allocate) and
    replayed, with eager work between the replays; every replay gives the workspace entry point's bits"""
    x, dy, gamma, _ = _operands(33, 2048, 768, False)
    want = _run(ctx, "agrad_norm_backward", capi.NORM_LAYER, x, dy, gamma, None, 1e-5, True)
    d_x, d_dy, d_g = ctx.upload(x), ctx.upload(dy), ctx.upload(gamma)
    d_dx, d_dg, d_db = ctx.zeros(x.shape, np.float32), ctx.zeros((768,), np.float32), ctx.zeros((768,), np.float32)
    ctx.call("agrad_norm_backward_noalloc", capi.NORM_LAYER, capi.F32, _p(d_x), _p(d_dy), _p(d_g), None, _p(d_dx), None,
             _p(d_dg), _p(d_db), 2048, 768, 1e-5, 0)           # (kernels load on first use: once eagerly)
    ctx.synchronize()
    ctx.call("agrad_graph_begin")
    ctx.call("agrad_norm_backward_noalloc", capi.NORM_LAYER, capi.F32, _p(d_x), _p(d_dy), _p(d_g), None, _p(d_dx), None,
             _p(d_dg), _p(d_db), 2048, 768, 1e-5, 0)
    gid = C.c_uint64(0)
    ctx.call("agrad_graph_end", C.byref(gid))
    try:
        for replay in range(3):
            for d in (d_dx, d_dg, d_db):
                ctx.call("agrad_fill", d.buffer_id, 0, 0x7fc00000, 4, d.nbytes // 4)     # scribble: NaN
            # eager use of the same scratch between the replays (same stream: in order)
            _run(ctx, "agrad_norm_backward_noalloc", capi.NORM_RMS, *_operands(34 + replay, 500, 384, False)[:3], None, 1e-6, False)
            ctx.call("agrad_graph_launch", gid.value)
            ctx.synchronize()
            for name, d in (("dx", d_dx), ("dgamma", d_dg), ("dbeta", d_db)):
                np.testing.assert_array_equal(d.download(), want[name], err_msg=f"replay {replay} {name}")
    finally:
        ctx.call("agrad_graph_destroy", gid.value)
        for d in (d_x, d_dy, d_g, d_dx, d_dg, d_db):
            d.free()


def test_noalloc_refuses_a_second_stream_while_the_first_is_busy(ctx):
    """two contexts (two streams) on one GPU share the array: the second is told so instead of racing"""
    other = capi.Context(0)
    try:
        x, dy, gamma, _ = _operands(40, 16384, 1536, False)
        d = [ctx.upload(a) for a in (x, dy, gamma)]
        dx, dg = ctx.zeros(x.shape, np.float32), ctx.zeros((1536,), np.float32)
        args = (capi.NORM_RMS, capi.F32, _p(d[0]), _p(d[1]), _p(d[2]), None, _p(dx), None, _p(dg), None, 16384, 1536, 1e-6, 0)
        ctx.synchronize()
        for _ in range(20):                                     # a millisecond of work in flight on the first stream
            ctx.call("agrad_norm_backward_noalloc", *args)
        with pytest.raises(capi.AgradError):
            other.call("agrad_norm_backward_noalloc", *args)
        ctx.synchronize()
        other.call("agrad_norm_backward_noalloc", *args)        # the first stream has drained: fine now
        other.synchronize()
        for a in d + [dx, dg]:
            a.free()
    finally:
        other.close()
