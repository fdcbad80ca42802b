"""Edge cases of the C ABI on the GPU: empty inputs are no-ops that touch nothing,
bad arguments come back as error codes (never as a launch), and a one-row /
one-column problem works.  The reference's CPU kernels accept empty arrays the
same way (numpy no-ops, backend.py:74-105, 376-487, 525-538).
"""
import ctypes as C

import numpy as np
import pytest

from autograd_amd import capi
from oracle import cpu_ops as K
from tests.helpers import assert_fp32_close

pytestmark = pytest.mark.gpu

SENTINEL = np.float32(123.25)


def vp(d):
    return C.c_void_p(d.ptr) if d is not None else None


@pytest.fixture()
def bufs(ctx):
    """a few small device buffers pre-filled with a sentinel; freed afterwards"""
    held = []

    def make(n=256, dtype=np.float32, value=SENTINEL):
        d = ctx.upload(np.full(n, value, dtype=dtype))
        held.append(d)
        return d

    yield make
    ctx.synchronize()
    for d in held:
        d.free()


def untouched(d):
    return bool((d.download() == SENTINEL).all())


def test_empty_inputs_are_noops(ctx, bufs):
    a, b, c, g = bufs(), bufs(), bufs(), bufs()
    ids = bufs(dtype=np.int32, value=0)
    ws = bufs(n=4096)
    f32 = capi.F32
    ctx.call("agrad_add_forward", f32, vp(a), vp(b), vp(c), 0)
    ctx.call("agrad_grad_accumulate", f32, vp(a), vp(b), 0, capi.ACC_INPUT_GRAD)
    ctx.call("agrad_copy", vp(a), vp(b), 0)
    ctx.call("agrad_cast_f32_to_bf16", vp(a), vp(b), 0, 0)
    ctx.call("agrad_cast_bf16_to_f32", vp(a), vp(b), 0)
    ctx.call("agrad_fill", a.ptr, 0, 0, 4, 0)
    for kind in (capi.NORM_LAYER, capi.NORM_RMS):
        ctx.call("agrad_norm_forward", kind, f32, vp(a), None, vp(g), None, None, vp(c), 0, 64, 1e-5)
        ctx.call("agrad_norm_forward", kind, f32, vp(a), None, vp(g), None, None, vp(c), 4, 0, 1e-5)
        ctx.call("agrad_norm_backward", kind, f32, vp(a), vp(b), vp(g), None, vp(c), None, None, None,
                 None, 0, 0, 64, 1e-5, 0)
    for name in ("agrad_gelu_forward", "agrad_relu2_forward"):
        ctx.call(name, f32, vp(a), vp(c), 0)
    for name in ("agrad_gelu_backward", "agrad_relu2_backward"):
        ctx.call(name, f32, vp(a), vp(b), vp(c), 0, 0)
    ctx.call("agrad_swiglu_forward", f32, vp(a), vp(c), 0, 16)
    ctx.call("agrad_swiglu_forward", f32, vp(a), vp(c), 4, 0)
    ctx.call("agrad_swiglu_backward", f32, vp(a), vp(b), vp(c), 0, 16, 0)
    ctx.call("agrad_rope_qk", f32, vp(a), vp(b), vp(g), vp(g), 0, 4, 2, 2, 8, 1, 0)
    ctx.call("agrad_rope_qk", f32, vp(a), vp(b), vp(g), vp(g), 2, 0, 2, 2, 8, 1, 0)
    ctx.call("agrad_gather_forward", f32, vp(ids), vp(a), None, vp(c), 0, 1, 16, 8)
    ctx.call("agrad_embedding_backward", f32, vp(ids), vp(a), vp(c), vp(ws), 4096 * 4, 0, 16, 8, 0)
    ctx.call("agrad_pos_embedding_backward", f32, vp(a), vp(c), 0, 4, 16, 0)
    ctx.synchronize()
    for d in (a, b, c, g, ws):
        assert untouched(d)


def test_zero_rows_norm_backward_defines_param_grads(ctx, bufs):
    """no rows: a stored dgamma / dbeta is zero (an empty sum), an accumulated one keeps its value"""
    x, dy, gamma = bufs(), bufs(), bufs()
    dgamma, dbeta = bufs(n=64), bufs(n=64)
    ws = bufs(n=1 << 16)
    for flags, expect in ((0, 0.0), (capi.ACC_PARAM_GRAD, float(SENTINEL))):
        for d in (dgamma, dbeta):
            ctx.call("agrad_fill", d.ptr, 0, int(np.float32(SENTINEL).view(np.uint32)), 4, 64)
        ctx.call("agrad_norm_backward", capi.NORM_LAYER, capi.F32, vp(x), vp(dy), vp(gamma), None, None, None,
                 vp(dgamma), vp(dbeta), vp(ws), (1 << 16) * 4, 0, 64, 1e-5, flags)
        ctx.synchronize()
        assert (dgamma.download() == expect).all() and (dbeta.download() == expect).all()


def test_bad_arguments_are_reported_not_launched(ctx, bufs):
    a, b, c = bufs(), bufs(), bufs()
    ids = bufs(dtype=np.int32, value=0)
    with pytest.raises(capi.AgradError) as e:
        ctx.call("agrad_norm_forward", 7, capi.F32, vp(a), None, None, None, None, vp(c), 1, 64, 1e-5)
    assert e.value.code == capi.EINVAL
    with pytest.raises(capi.AgradError):
        ctx.call("agrad_norm_forward", capi.NORM_RMS, 9, vp(a), None, None, None, None, vp(c), 1, 64, 1e-5)
    with pytest.raises(capi.AgradError):
        ctx.call("agrad_norm_forward", capi.NORM_RMS, capi.F32, None, None, None, None, None, vp(c), 1, 64, 1e-5)
    with pytest.raises(capi.AgradError):      # odd head dimension
        ctx.call("agrad_rope_qk", capi.F32, vp(a), vp(b), vp(c), vp(c), 1, 1, 1, 1, 7, 1, 0)
    with pytest.raises(capi.AgradError):      # sign must be +-1
        ctx.call("agrad_rope_qk", capi.F32, vp(a), vp(b), vp(c), vp(c), 1, 1, 1, 1, 8, 0, 0)
    with pytest.raises(capi.AgradError) as e: # workspace too small
        ctx.call("agrad_embedding_backward", capi.F32, vp(ids), vp(a), vp(c), vp(b), 16, 8, 16, 8, 0)
    assert e.value.code == capi.EWORKSPACE
    with pytest.raises(capi.AgradError) as e: # parameter grads wanted but no workspace
        ctx.call("agrad_norm_backward", capi.NORM_RMS, capi.F32, vp(a), vp(b), None, None, vp(c), None,
                 vp(b), None, None, 0, 2, 64, 1e-5, 0)
    assert e.value.code == capi.EWORKSPACE
    with pytest.raises(capi.AgradError):      # fill item size
        ctx.call("agrad_fill", a.ptr, 0, 0, 3, 4)
    with pytest.raises((capi.AgradError, ValueError)):   # offset beyond the allocation
        ctx.call("agrad_fill", a.ptr, 1 << 20, 0, 4, 4)
    ctx.synchronize()
    for d in (a, b, c):
        assert untouched(d)


def test_out_of_range_token_is_an_index_error_and_skips_the_row(ctx, bufs):
    V, Cw = 8, 16
    W = ctx.upload(np.arange(V * Cw, dtype=np.float32).reshape(V, Cw))
    ids = ctx.upload(np.array([1, 8, -1, 3], np.int32))
    out = bufs(n=4 * Cw)
    ctx.call("agrad_gather_forward", capi.F32, vp(ids), vp(W), None, vp(out), 4, 4, Cw, V)
    with pytest.raises(IndexError):
        ctx.synchronize()
    got = out.download().reshape(4, Cw)
    np.testing.assert_array_equal(got[0], np.arange(Cw, 2 * Cw, dtype=np.float32))
    np.testing.assert_array_equal(got[3], np.arange(3 * Cw, 4 * Cw, dtype=np.float32))
    assert (got[1:3] == SENTINEL).all()
    ctx.synchronize()          # the error was consumed
    W.free()
    ids.free()


def test_single_row_single_column(ctx):
    """the smallest non-empty problems: [1, 1] norm, one-element activations, one token"""
    x = np.array([[2.5]], np.float32)
    g = np.array([1.5], np.float32)
    b = np.array([0.25], np.float32)
    dx, dg, db, dy = ctx.upload(x), ctx.upload(g), ctx.upload(b), ctx.empty((1, 1), np.float32)
    ctx.call("agrad_norm_forward", capi.NORM_LAYER, capi.F32, vp(dx), None, vp(dg), vp(db), None, vp(dy), 1, 1, 1e-5)
    ctx.synchronize()
    assert_fp32_close(dy.download(), K.layernorm_forward(x, g, b, 1e-5), "1x1 layernorm")
    ctx.call("agrad_norm_forward", capi.NORM_RMS, capi.F32, vp(dx), None, vp(dg), None, None, vp(dy), 1, 1, 1e-6)
    ctx.synchronize()
    assert_fp32_close(dy.download(), K.rmsnorm_forward(x, g, 1e-6), "1x1 rmsnorm")
    ctx.call("agrad_gelu_forward", capi.F32, vp(dx), vp(dy), 1)
    ctx.synchronize()
    assert_fp32_close(dy.download(), K.gelu_forward(x), "1-element gelu")
    for d in (dx, dg, db, dy):
        d.free()
    # one token, one column: the gradient of a [V, 1] table
    ids = np.array([2], np.int32)
    dY = np.array([[0.75]], np.float32)
    d_ids, d_dY, d_dW = ctx.upload(ids), ctx.upload(dY), ctx.upload(np.zeros((4, 1), np.float32))
    ws_bytes = ctx.lib.agrad_embedding_backward_workspace_bytes(1, 1, 4, capi.F32)
    ws = ctx.empty((max(ws_bytes, 1),), np.uint8)
    ctx.call("agrad_embedding_backward", capi.F32, vp(d_ids), vp(d_dY), vp(d_dW), vp(ws), ws_bytes, 1, 1, 4,
             capi.ACC_PARAM_GRAD)
    ctx.synchronize()
    np.testing.assert_array_equal(d_dW.download().ravel(), np.array([0, 0, 0.75, 0], np.float32))
    for d in (d_ids, d_dY, d_dW, ws):
        d.free()


def test_plain_c_program_drives_the_library():
    """tests/c_abi/layer_check (gcc, C99, no Python in the process) runs LayerNorm
    forward / backward and GELU through the C ABI and checks them against the
    textbook formulas in double precision"""
    import subprocess
    from pathlib import Path
    exe = Path(__file__).parent / "c_abi" / "layer_check"
    assert exe.exists(), f"{exe} is missing: build it with `python -m autograd_amd.build`"
    proc = subprocess.run([str(exe)], capture_output=True, text=True, timeout=100)
    assert proc.returncode == 0 and proc.stdout.strip() == "ok", proc.stdout + proc.stderr
