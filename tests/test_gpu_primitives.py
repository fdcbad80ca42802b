"""Mul (all four broadcast kinds), Exp, Log, Rsqrt and Softmax through the C ABI
against the CPU restatement (cpu_mul_*, cpu_exp_*, cpu_log_*, cpu_rsqrt_*,
cpu_softmax_*, backend.py:107-146, 320-374).

fp32: Mul forward / its dx and Rsqrt are bit-exact (one or two correctly rounded
operations per element); Exp, Log and Softmax are within rtol 1e-5 / atol 1e-6;
the summed Mul gradients are compared to float64 with a bound that grows with the
number of terms.  bf16 storage: 1e-2 relative to the fp32 restatement on the same
bf16-rounded inputs.
"""
import ctypes as C

import numpy as np
import pytest

from autograd_amd import capi
from oracle import cpu_ops as ref
from tests.helpers import assert_bf16_close, assert_fp32_close, from_bf16_bits, to_bf16_bits

pytestmark = pytest.mark.gpu
SEED = 1333


def vp(d):
    return C.c_void_p(d.ptr) if d is not None else None


def _io(a, dtype):
    """(storage array, fp32 value actually stored)"""
    if dtype == "bf16":
        bits = to_bf16_bits(a)
        return bits, from_bf16_bits(bits)
    return a, a


UNARY = [("exp", capi.UNARY_EXP, ref.exp_forward, ref.exp_backward_into, True, (-3.0, 3.0)),
         ("log", capi.UNARY_LOG, ref.log_forward, ref.log_backward_into, False, (0.05, 8.0)),
         ("rsqrt", capi.UNARY_RSQRT, ref.rsqrt_forward, ref.rsqrt_backward_into, True, (0.05, 8.0))]


@pytest.mark.parametrize("name,op,fwd,bwd,saves_y,rng_", UNARY, ids=[u[0] for u in UNARY])
@pytest.mark.parametrize("n", [1, 7, 64, 1000, 4099, 1 << 18])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_unary_primitives(ctx, name, op, fwd, bwd, saves_y, rng_, n, dtype):
    rng = np.random.default_rng(SEED + n)
    dt = capi.BF16 if dtype == "bf16" else capi.F32
    xs, x = _io(rng.uniform(*rng_, n).astype(np.float32), dtype)
    dys, dy = _io(rng.standard_normal(n).astype(np.float32), dtype)
    base_s, base = _io(rng.standard_normal(n).astype(np.float32), dtype)
    d_x, d_dy = ctx.upload(xs), ctx.upload(dys)
    d_y = ctx.empty((n,), xs.dtype)
    ctx.call("agrad_unary_forward", op, dt, vp(d_x), vp(d_y), n)
    ctx.synchronize()
    ys = d_y.download()
    y = from_bf16_bits(ys) if dtype == "bf16" else ys
    want_y = fwd(x)
    saved = d_y if saves_y else d_x
    results = []
    for flags, init in ((0, np.full(n, 7, xs.dtype)), (capi.ACC_INPUT_GRAD, base_s)):
        d_dx = ctx.upload(init)
        ctx.call("agrad_unary_backward", op, dt, vp(d_dy), vp(saved), vp(d_dx), n, flags)
        ctx.synchronize()
        results.append(d_dx.download())
        d_dx.free()
    want_dx = np.zeros(n, np.float32)
    bwd(dy, y if saves_y else x, want_dx)        # from the value the device saved
    if dtype == "bf16":
        assert_bf16_close(y, want_y, f"{name} y")
        assert_bf16_close(from_bf16_bits(results[0]), want_dx, f"{name} dx")
        assert_bf16_close(from_bf16_bits(results[1]), base + want_dx, f"{name} dx accumulate")
    else:
        if name == "rsqrt":
            np.testing.assert_array_equal(y, want_y)
            np.testing.assert_array_equal(results[0], want_dx)
        else:
            assert_fp32_close(y, want_y, f"{name} y")
            assert_fp32_close(results[0], want_dx, f"{name} dx")
        assert_fp32_close(results[1], base + want_dx, f"{name} dx accumulate")
    for d in (d_x, d_dy, d_y):
        d.free()


MUL_SHAPES = [(1, 1), (3, 5), (5, 64), (64, 96), (65, 96), (33, 100), (700, 768), (16, 4096), (4096, 50), (2000, 384),
              (7, 10000)]


@pytest.mark.parametrize("lead,inner", MUL_SHAPES)
@pytest.mark.parametrize("kind", ["same", "row", "col", "scalar"])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_mul_and_its_gradients(ctx, lead, inner, kind, dtype):
    rng = np.random.default_rng(SEED + lead + 3 * inner)
    dt = capi.BF16 if dtype == "bf16" else capi.F32
    K = {"same": capi.MUL_SAME, "row": capi.MUL_ROW, "col": capi.MUL_COL, "scalar": capi.MUL_SCALAR}[kind]
    yshape = {"same": (lead, inner), "row": (inner,), "col": (lead, 1), "scalar": (1,)}[kind]
    xs, x = _io(rng.standard_normal((lead, inner)).astype(np.float32), dtype)
    ys, y = _io(rng.standard_normal(yshape).astype(np.float32), dtype)
    gs, g = _io(rng.standard_normal((lead, inner)).astype(np.float32), dtype)
    bx_s, bx = _io(rng.standard_normal((lead, inner)).astype(np.float32), dtype)
    by_s, by = _io(rng.standard_normal(yshape).astype(np.float32), dtype)
    d_x, d_y, d_g = ctx.upload(xs), ctx.upload(ys), ctx.upload(gs)
    d_out = ctx.empty(xs.shape, xs.dtype)
    ctx.call("agrad_mul_forward", dt, K, vp(d_x), vp(d_y), vp(d_out), lead, inner)
    ws_b = ctx.lib.agrad_mul_backward_workspace_bytes(K, lead, inner)
    ws = ctx.empty((max(ws_b, 16),), np.uint8)
    runs = []
    for flags, ix, iy in ((0, np.full(xs.shape, 7, xs.dtype), np.full(yshape, 5, xs.dtype)),
                          (capi.ACC_INPUT_GRAD | capi.ACC_INPUT_GRAD2, bx_s, by_s)):
        d_dx, d_dy = ctx.upload(ix), ctx.upload(iy)
        ctx.call("agrad_mul_backward", dt, K, vp(d_g), vp(d_x), vp(d_y), vp(d_dx), vp(d_dy), vp(ws), ws_b, lead, inner,
                 flags)
        ctx.synchronize()
        runs.append((d_dx.download(), d_dy.download()))
        d_dx.free()
        d_dy.free()
    # dx alone and dy alone (the other pointer NULL) give the same bits
    d_dx, d_dy = ctx.upload(np.full(xs.shape, 7, xs.dtype)), ctx.upload(np.full(yshape, 5, xs.dtype))
    ctx.call("agrad_mul_backward", dt, K, vp(d_g), None, vp(d_y), vp(d_dx), None, None, 0, lead, inner, 0)
    ctx.call("agrad_mul_backward", dt, K, vp(d_g), vp(d_x), None, None, vp(d_dy), vp(ws), ws_b, lead, inner, 0)
    ctx.synchronize()
    np.testing.assert_array_equal(d_dx.download(), runs[0][0])
    np.testing.assert_array_equal(d_dy.download(), runs[0][1])
    out = d_out.download()
    for d in (d_x, d_y, d_g, d_out, ws, d_dx, d_dy):
        d.free()

    want_out = ref.mul_forward(x, y)
    want_dx = np.zeros_like(x)
    ref.mul_backward_into(g, x, y, dx=want_dx)
    prod64 = g.astype(np.float64) * x.astype(np.float64)
    mag = np.abs(prod64)
    red = {"same": lambda a: a, "row": lambda a: a.sum(0), "col": lambda a: a.sum(1, keepdims=True),
           "scalar": lambda a: a.sum().reshape(1)}[kind]
    want_dy, dy_mag = red(prod64), red(mag)
    if dtype == "bf16":
        np.testing.assert_array_equal(out, to_bf16_bits(want_out))            # one product, one rounding
        np.testing.assert_array_equal(runs[0][0], to_bf16_bits(want_dx))
        np.testing.assert_array_equal(runs[1][0], to_bf16_bits(bx + want_dx))
        tol = 1e-2 * dy_mag + 1e-6                       # bf16 rounding of a sum whose terms may cancel
        assert (np.abs(from_bf16_bits(runs[0][1]) - want_dy) <= tol).all()
        assert (np.abs(from_bf16_bits(runs[1][1]) - (by + want_dy)) <= tol + 1e-2 * np.abs(by)).all()
    else:
        np.testing.assert_array_equal(out, want_out)
        np.testing.assert_array_equal(runs[0][0], want_dx)
        np.testing.assert_array_equal(runs[1][0], bx + want_dx)
        # an fp32 sum of many terms in any fixed order: a few eps * sum |term|
        tol = 2e-7 * dy_mag + 1e-6
        assert (np.abs(runs[0][1] - want_dy) <= tol).all()
        assert (np.abs(runs[1][1] - (by + want_dy)) <= tol + 2e-7 * np.abs(by)).all()
        cpu = np.zeros(yshape, np.float32)
        ref.mul_backward_into(g, x, y, dy=cpu)
        assert (np.abs(runs[0][1] - cpu) <= 2 * tol).all()


# rows of a whole number of vectors up to 512 vectors stay in one wave's registers (1, 2, 4 or 8
# vectors per lane); the others take the two-pass kernels (one wave or 256 threads per row)
SOFTMAX_SHAPES = [(1, 1), (3, 5), (2 * 4 * 64, 64), (12 * 128, 128), (37, 257), (5, 520), (9, 1024), (5, 1025),
                  (7, 2048), (3, 4096), (4, 4104), (6, 4099), (3, 32768), (2, 50257)]


@pytest.mark.parametrize("rows,V", SOFTMAX_SHAPES)
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_softmax_forward_and_backward(ctx, rows, V, dtype):
    rng = np.random.default_rng(SEED + V)
    dt = capi.BF16 if dtype == "bf16" else capi.F32
    x_raw = (3.0 * rng.standard_normal((rows, V))).astype(np.float32)
    if V > 8:
        x_raw[0, 3:6] = -np.inf                  # masked positions
    xs, x = _io(x_raw, dtype)
    gs, g = _io(rng.standard_normal((rows, V)).astype(np.float32), dtype)
    base_s, base = _io(rng.standard_normal((rows, V)).astype(np.float32), dtype)
    d_x, d_g = ctx.upload(xs), ctx.upload(gs)
    d_y = ctx.empty(xs.shape, xs.dtype)
    ctx.call("agrad_softmax_forward", dt, vp(d_x), vp(d_y), rows, V)
    ctx.synchronize()
    ys = d_y.download()
    y = from_bf16_bits(ys) if dtype == "bf16" else ys
    runs = []
    for flags, init in ((0, np.full(xs.shape, 7, xs.dtype)), (capi.ACC_INPUT_GRAD, base_s)):
        d_dx = ctx.upload(init)
        ctx.call("agrad_softmax_backward", dt, vp(d_y), vp(d_g), vp(d_dx), rows, V, flags)
        ctx.synchronize()
        runs.append(d_dx.download())
        d_dx.free()
    # in place: y written over x
    ctx.call("agrad_softmax_forward", dt, vp(d_x), vp(d_x), rows, V)
    ctx.synchronize()
    np.testing.assert_array_equal(d_x.download(), ys)
    for d in (d_x, d_g, d_y):
        d.free()
    want_y = ref.softmax_forward(x)
    want_dx = np.zeros_like(x)
    ref.softmax_backward_into(y, g, want_dx)       # from the y the device stored
    assert np.isfinite(y).all()
    if dtype == "bf16":
        assert_bf16_close(y, want_y, "softmax y")
        # dx = y * (g - dot): bf16 rounding of y and g enters the row dot product
        scale = np.abs(want_dx).max() + 1e-6
        assert np.abs(from_bf16_bits(runs[0]) - want_dx).max() <= 2e-2 * scale
        assert np.abs(from_bf16_bits(runs[1]) - (base + want_dx)).max() <= 2e-2 * (scale + np.abs(base).max())
    else:
        assert_fp32_close(y, want_y, "softmax y", atol=1e-7)
        np.testing.assert_allclose(y.sum(-1), 1.0, atol=3e-6)
        assert_fp32_close(runs[0], want_dx, "softmax dx", atol=1e-6)
        assert_fp32_close(runs[1], base + want_dx, "softmax dx accumulate", atol=2e-6)
        if V > 8:
            assert not y[0, 3:6].any() and not runs[0][0, 3:6].any()


def test_argument_errors(ctx):
    buf = ctx.upload(np.ones(64, np.float32))
    with pytest.raises(capi.AgradError):
        ctx.call("agrad_unary_forward", 9, capi.F32, vp(buf), vp(buf), 64)
    with pytest.raises(capi.AgradError):
        ctx.call("agrad_mul_forward", capi.F32, 7, vp(buf), vp(buf), vp(buf), 8, 8)
    with pytest.raises(capi.AgradError):      # scalar dy without its workspace
        ctx.call("agrad_mul_backward", capi.F32, capi.MUL_SCALAR, vp(buf), vp(buf), vp(buf), None, vp(buf), None, 0, 8, 8, 0)
    with pytest.raises(capi.AgradError):
        ctx.call("agrad_softmax_forward", capi.F32, None, vp(buf), 8, 8)
    # empty problems are fine
    ctx.call("agrad_softmax_forward", capi.F32, vp(buf), vp(buf), 0, 8)
    ctx.call("agrad_mul_forward", capi.F32, capi.MUL_ROW, vp(buf), vp(buf), vp(buf), 0, 8)
    ctx.call("agrad_unary_forward", capi.UNARY_EXP, capi.F32, vp(buf), vp(buf), 0)
    ctx.synchronize()
    buf.free()


# -- GELU(h + b) and its backward with the bias gradient ---------------------------------
BIAS_GELU_SHAPES = [(1, 1), (3, 5), (64, 384), (65, 384), (1000, 96), (300, 1536), (2048, 1000), (5000, 130),
                    (16384, 64)]


@pytest.mark.parametrize("rows,Cw", BIAS_GELU_SHAPES)
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_bias_gelu_forward_and_backward(ctx, rows, Cw, dtype):
    """agrad_gelu_bias_forward / _backward against the CPU composition Add -> GELU
    (cpu_add_forward, cpu_gelu_forward / backward, cpu_add_backward's reduction):
    dh stored and accumulated, db stored and accumulated, each alone and together.
    fp32: rtol 1e-5 / atol 1e-6 for y and dh; the bias gradient is a sum of `rows`
    terms, compared to float64 with the bound of the other column sums.  bf16
    storage: 1e-2 relative to the fp32 restatement on the bf16-rounded inputs."""
    rng = np.random.default_rng(SEED + rows * 7 + Cw)
    dt = capi.BF16 if dtype == "bf16" else capi.F32
    hs, h = _io(rng.standard_normal((rows, Cw)).astype(np.float32), dtype)
    bs, b = _io((0.5 * rng.standard_normal(Cw)).astype(np.float32), dtype)
    dys, dy = _io(rng.standard_normal((rows, Cw)).astype(np.float32), dtype)
    dh0s, dh0 = _io(rng.standard_normal((rows, Cw)).astype(np.float32), dtype)
    db0s, db0 = _io(rng.standard_normal(Cw).astype(np.float32), dtype)
    d_h, d_b, d_dy = ctx.upload(hs), ctx.upload(bs), ctx.upload(dys)
    d_y = ctx.empty((rows, Cw), hs.dtype)
    ctx.call("agrad_gelu_bias_forward", dt, vp(d_h), vp(d_b), vp(d_y), rows, Cw)
    ctx.synchronize()
    got_y = d_y.download()
    want_y = ref.bias_gelu_forward(h, b)
    if dtype == "bf16":
        assert_bf16_close(from_bf16_bits(got_y), want_y, "bias gelu forward")
    else:
        assert_fp32_close(got_y, want_y, "bias gelu forward")

    term = np.zeros((rows, Cw), np.float32)
    ref.bias_gelu_backward_into(h, b, dy, dh=term)
    col = term.astype(np.float64).sum(axis=0)
    ws_b = ctx.lib.agrad_gelu_bias_backward_workspace_bytes(rows, Cw)
    assert ws_b >= 4 * Cw
    ws = ctx.empty((ws_b,), np.uint8)
    cases = [(0, True, True), (capi.ACC_INPUT_GRAD | capi.ACC_PARAM_GRAD, True, True),
             (capi.ACC_INPUT_GRAD, True, False), (capi.ACC_PARAM_GRAD, False, True), (0, False, True)]
    for flags, want_dh, want_db in cases:
        d_dh = ctx.upload(dh0s) if want_dh else None
        d_db = ctx.upload(db0s) if want_db else None
        ctx.call("agrad_gelu_bias_backward", dt, vp(d_dy), vp(d_h), vp(d_b), vp(d_dh), vp(d_db),
                 vp(ws) if want_db else None, ws_b if want_db else 0, rows, Cw, flags)
        ctx.synchronize()
        what = f"bias gelu backward flags={flags} dh={want_dh} db={want_db}"
        if want_dh:
            got = d_dh.download()
            want = term + dh0 if flags & capi.ACC_INPUT_GRAD else term
            if dtype == "bf16":
                assert_bf16_close(from_bf16_bits(got), want, what + " dh")
            else:
                # beyond |h + b| = 4.5 the CPU's 1 - tanh^2 has lost its bits to cancellation
                # and the device value is the accurate one: 3e-6 absolute, as for plain GELU
                assert_fp32_close(got, want, what + " dh", rtol=1e-5, atol=3e-6)
            d_dh.free()
        if want_db:
            got = d_db.download()
            want = col + db0 if flags & capi.ACC_PARAM_GRAD else col
            if dtype == "bf16":
                scale = np.abs(term).astype(np.float64).sum(axis=0) + np.abs(db0)
                err = np.abs(from_bf16_bits(got).astype(np.float64) - want)
                assert (err <= 1e-2 * np.maximum(np.abs(want), 1e-2 * scale) + 1e-3).all(), what + " db"
            else:
                assert_fp32_close(got, want.astype(np.float32), what + " db", rtol=1e-5,
                                  atol=max(2e-6, 1e-4 * np.sqrt(rows / 14)))
            d_db.free()
    if dtype == "f32":
        # the bias gradient stored as bf16: the fp32 call's sum (plus the stored value) rounded once
        wide_db = ctx.zeros((Cw,), np.float32)
        d_dh = ctx.upload(dh0s)
        ctx.call("agrad_gelu_bias_backward", dt, vp(d_dy), vp(d_h), vp(d_b), vp(d_dh), vp(wide_db), vp(ws), ws_b, rows, Cw, 0)
        ctx.synchronize()
        sums = wide_db.download()
        old_bits = to_bf16_bits(db0)
        for accumulate in (False, True):
            narrow = ctx.upload(old_bits)
            ctx.call("agrad_gelu_bias_backward", dt, vp(d_dy), vp(d_h), vp(d_b), vp(d_dh), vp(narrow), vp(ws), ws_b, rows, Cw,
                     capi.PARAM_GRAD_BF16 | (capi.ACC_PARAM_GRAD if accumulate else 0))
            ctx.synchronize()
            base = from_bf16_bits(old_bits) if accumulate else np.zeros(Cw, np.float32)
            np.testing.assert_array_equal(narrow.download(), to_bf16_bits(base + sums))
            narrow.free()
        wide_db.free()
        d_dh.free()
    for d in (d_h, d_b, d_dy, d_y, ws):
        d.free()


def test_bias_gelu_argument_errors(ctx):
    h = ctx.zeros((128, 64), np.float32)
    b = ctx.zeros((64,), np.float32)
    with pytest.raises(capi.AgradError):         # the bias gradient needs its workspace
        ctx.call("agrad_gelu_bias_backward", capi.F32, vp(h), vp(h), vp(b), vp(h), vp(b), None, 0, 128, 64, 0)
    with pytest.raises(capi.AgradError):         # nothing to compute
        ctx.call("agrad_gelu_bias_backward", capi.F32, vp(h), vp(h), vp(b), None, None, None, 0, 128, 64, 0)
    with pytest.raises(capi.AgradError):
        ctx.call("agrad_gelu_bias_forward", 7, vp(h), vp(b), vp(h), 128, 64)
    ctx.call("agrad_gelu_bias_forward", capi.F32, vp(h), vp(b), vp(h), 0, 64)      # empty: no launch
    ctx.synchronize()
    h.free()
    b.free()
