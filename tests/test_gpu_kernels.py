"""Parity of every HIP kernel against the CPU restatement, through the C ABI.

Tolerances: fp32 outputs rtol 1e-5 / atol 1e-6 (helpers.FP32_*); gather and
fill / cast are bit-exact; bf16-I/O outputs 1e-2 relative to the fp32 path fed
the same bf16-rounded inputs (helpers.BF16_REL).  Row-summed parameter
gradients (dgamma, dbeta) are compared to the fp32 CPU result at probe sizes and
to the float64 closed form at large row counts, where the CPU's own sequential
fp32 row sum is the noisier of the two.

Seeds follow the reference's probes (SEED = 1333, check_tiny_gpt2_kernel.py:47).
"""
import zlib

import numpy as np
import pytest

from autograd_amd import capi
from oracle import closed_form as cf
from oracle import cpu_ops as ref
from tests import gpu_ops as G
from tests.helpers import (assert_bf16_close, assert_fp32_close, assert_fp32_parity, from_bf16_bits, to_bf16_bits)

pytestmark = pytest.mark.gpu
SEED = 1333
KINDS = {"layer": capi.NORM_LAYER, "rms": capi.NORM_RMS}


def _rng(k):
    return np.random.default_rng(SEED + k)


def _norm_ref_forward(kind, x, gamma, beta, eps):
    if kind == "layer":
        return ref.layernorm_forward(x, gamma, beta, eps)
    return ref.rmsnorm_forward(x, gamma, eps)


def _norm_ref_backward(kind, x, gamma, dy, eps, want_params=True):
    dx = np.zeros_like(x)
    dgamma = np.zeros_like(gamma) if want_params else None
    if kind == "layer":
        dbeta = np.zeros_like(gamma) if want_params else None
        ref.layernorm_backward_into(x, gamma, dy, eps, dx, dgamma, dbeta)
        return dx, dgamma, dbeta
    ref.rmsnorm_backward_into(x, gamma, dy, eps, dx, dgamma)
    return dx, dgamma, None


# shapes cover every launch geometry: wave-per-row (C <= 1024) with 1..4 vectors
# per lane, workgroup-per-row (256 and 1024 threads), and the scalar fallback
NORM_SHAPES = [
    ((2, 16, 64), 1e-5),     # the reference's probe_layernorm shape (check_tiny_gpt2_kernel.py:758-782)
    ((512, 128), 1e-5),      # config 1
    ((67, 384), 1e-5),       # config 2 width, ragged row count
    ((45, 768), 1e-5),       # config 3 width
    ((33, 1024), 1e-6),
    ((21, 1536), 1e-6),      # config 4 width
    ((9, 4096), 1e-5),       # config 5 width
    ((5, 8192), 1e-5),       # 1024-thread rows
    ((7, 50), 1e-5),         # C % 4 != 0 -> scalar kernel
    ((3, 20000), 1e-5),      # wider than any register-resident geometry
    ((1, 4), 1e-5),
]


@pytest.mark.parametrize("kind", ["layer", "rms"])
@pytest.mark.parametrize("shape,eps", NORM_SHAPES)
def test_norm_forward_fp32(ctx, kind, shape, eps):
    rng = _rng(4)
    C = shape[-1]
    x = rng.standard_normal(shape, dtype=np.float32)
    gamma = (1 + 0.02 * rng.standard_normal(C)).astype(np.float32)
    beta = (0.02 * rng.standard_normal(C)).astype(np.float32) if kind == "layer" else None
    got, _ = G.norm_forward(ctx, KINDS[kind], x, gamma, beta, eps)
    assert_fp32_close(got, _norm_ref_forward(kind, x, gamma, beta, eps), f"{kind} forward {shape}")


def test_norm_forward_probe_recipe(ctx):
    """probe_layernorm: seed+4, (2,16,64), gamma/beta ~ N(0,1), eps 1e-5."""
    rng = _rng(4)
    x = rng.standard_normal((2, 16, 64), dtype=np.float32)
    g = rng.standard_normal((64,), dtype=np.float32)
    b = rng.standard_normal((64,), dtype=np.float32)
    up = rng.standard_normal((2, 16, 64), dtype=np.float32)
    got, _ = G.norm_forward(ctx, capi.NORM_LAYER, x, g, b, 1e-5)
    assert_fp32_close(got, ref.layernorm_forward(x, g, b, 1e-5), "probe forward", rtol=1e-6, atol=1e-6)
    out = G.norm_backward(ctx, capi.NORM_LAYER, x, g, up, 1e-5)
    dx, dg, db = _norm_ref_backward("layer", x, g, up, 1e-5)
    assert_fp32_close(out["dx"], dx, "probe x.grad")
    assert_fp32_close(out["dgamma"], dg, "probe gamma.grad")
    assert_fp32_close(out["dbeta"], db, "probe beta.grad")


def test_rmsnorm_weightless_and_layernorm_without_affine(ctx):
    rng = _rng(6)
    x = rng.standard_normal((19, 384), dtype=np.float32)
    got, _ = G.norm_forward(ctx, capi.NORM_RMS, x, None, None, 1e-6)
    assert_fp32_close(got, ref.rmsnorm_forward(x, None, 1e-6), "weightless rms")
    got, _ = G.norm_forward(ctx, capi.NORM_LAYER, x, None, None, 1e-5)
    one, zero = np.ones(384, np.float32), np.zeros(384, np.float32)
    assert_fp32_close(got, ref.layernorm_forward(x, one, zero, 1e-5), "plain layernorm")
    # gamma = 1, beta = 0 (config 1): rows have mean 0 and variance 1
    assert np.abs(got.mean(-1)).max() < 1e-6
    assert np.abs(got.var(-1) - 1).max() < 1e-4
    dy = rng.standard_normal(x.shape, dtype=np.float32)
    out = G.norm_backward(ctx, capi.NORM_RMS, x, None, dy, 1e-6, want_dgamma=False, want_dbeta=False)
    dx = np.zeros_like(x)
    ref.rmsnorm_backward_into(x, None, dy, 1e-6, dx, None)
    assert_fp32_close(out["dx"], dx, "weightless rms dx")


@pytest.mark.parametrize("kind", ["layer", "rms"])
@pytest.mark.parametrize("shape,eps", NORM_SHAPES)
def test_norm_backward_fp32(ctx, kind, shape, eps):
    rng = _rng(4)
    C = shape[-1]
    x = rng.standard_normal(shape, dtype=np.float32)
    gamma = (1 + 0.02 * rng.standard_normal(C)).astype(np.float32)
    dy = rng.standard_normal(shape, dtype=np.float32)
    out = G.norm_backward(ctx, KINDS[kind], x, gamma, dy, eps, want_dbeta=(kind == "layer"))
    dx, dgamma, dbeta = _norm_ref_backward(kind, x, gamma, dy, eps)
    assert_fp32_close(out["dx"], dx, f"{kind} dx {shape}")
    # row sums: both sides round differently (the CPU adds rows one by one), so
    # the absolute budget grows with sqrt(rows); at probe sizes it is 2e-6
    rows = int(np.prod(shape[:-1]))
    atol = max(2e-6, 1e-6 * np.sqrt(rows))
    assert_fp32_close(out["dgamma"], dgamma, f"{kind} dgamma {shape}", rtol=1e-5, atol=atol)
    if kind == "layer":
        assert_fp32_close(out["dbeta"], dbeta, f"{kind} dbeta {shape}", rtol=1e-5, atol=atol)
        _, dg64, db64 = cf.layernorm_grads(x, gamma, dy, eps)
        assert np.abs(out["dbeta"] - db64).max() <= atol
    else:
        _, dg64 = cf.rmsnorm_grads(x, gamma, dy, eps)
    assert np.abs(out["dgamma"] - dg64).max() <= atol


@pytest.mark.parametrize("kind", ["layer", "rms"])
def test_norm_backward_accumulate_and_residual_grad(ctx, kind):
    """CPU semantics: grads accumulate (backend.py:477-487); the fused residual
    gradient is added in the same pass (metal_ops.metal:8164); dx2 mirrors dx."""
    rng = _rng(7)
    shape = (37, 384)
    x = rng.standard_normal(shape, dtype=np.float32)
    gamma = (1 + 0.02 * rng.standard_normal(384)).astype(np.float32)
    dy = rng.standard_normal(shape, dtype=np.float32)
    dx0 = rng.standard_normal(shape, dtype=np.float32)
    dres = rng.standard_normal(shape, dtype=np.float32)
    dg0 = rng.standard_normal(384).astype(np.float32)
    db0 = rng.standard_normal(384).astype(np.float32)
    eps = 1e-5
    flags = capi.ACC_INPUT_GRAD | capi.ACC_PARAM_GRAD
    out = G.norm_backward(ctx, KINDS[kind], x, gamma, dy, eps, dres=dres, dx_init=dx0, want_dx2=True,
                          dgamma_init=dg0, dbeta_init=db0, want_dbeta=(kind == "layer"), flags=flags)
    dx, dgamma, dbeta = _norm_ref_backward(kind, x, gamma, dy, eps)
    if kind == "layer":
        dx64, dg64, db64 = cf.layernorm_grads(x, gamma, dy, eps)
    else:
        (dx64, dg64), db64 = cf.rmsnorm_grads(x, gamma, dy, eps), None
    r64, x0_64 = dres.astype(np.float64), dx0.astype(np.float64)
    # (sums of three or four terms: where the fp32 adds associate differently from numpy's the
    # result may miss atol 1e-6 by an ulp of the largest term; then it must be as close to
    # the float64 sum as the CPU restatement's)
    assert_fp32_parity(out["dx"], dx0 + (dres + dx), x0_64 + r64 + dx64, "accumulated dx")
    assert_fp32_parity(out["dx2"], dres + dx, r64 + dx64, "stored dx2")   # dx2 has its own flag
    out2 = G.norm_backward(ctx, KINDS[kind], x, gamma, dy, eps, dres=dres, want_dx2=True,
                           want_dgamma=False, want_dbeta=False, flags=capi.ACC_INPUT_GRAD2)
    assert_fp32_parity(out2["dx"], dres + dx, r64 + dx64, "stored dx")
    assert_fp32_parity(out2["dx2"], 9 + (dres + dx), 9 + r64 + dx64, "accumulated dx2")
    assert_fp32_parity(out["dgamma"], dg0 + dgamma, dg0.astype(np.float64) + dg64, "accumulated dgamma")
    if kind == "layer":
        assert_fp32_parity(out["dbeta"], db0 + dbeta, db0.astype(np.float64) + db64, "accumulated dbeta")
    # overwrite mode with a residual gradient and no accumulate
    out = G.norm_backward(ctx, KINDS[kind], x, gamma, dy, eps, dres=dres, want_dgamma=False, want_dbeta=False)
    assert_fp32_parity(out["dx"], dres + dx, r64 + dx64, "dres + dx")
    # parameter grads only
    out = G.norm_backward(ctx, KINDS[kind], x, gamma, dy, eps, want_dx=False, want_dbeta=(kind == "layer"))
    assert out["dx"] is None
    assert_fp32_parity(out["dgamma"], dgamma, dg64, "dgamma only")


@pytest.mark.parametrize("kind,C,eps", [("layer", 384, 1e-5), ("layer", 768, 1e-5), ("rms", 1536, 1e-6)])
def test_norm_backward_param_grads_many_rows(ctx, kind, C, eps):
    """N = 16384 rows (configs 2-4).  The fp32 CPU result sums rows sequentially
    and carries ~1e-4 of rounding noise, so the GPU is held to the float64 value
    and must be at least as close to it as the CPU result is."""
    rng = _rng(8)
    N = 16384
    x = rng.standard_normal((N, C), dtype=np.float32)
    gamma = (1 + 0.02 * rng.standard_normal(C)).astype(np.float32)
    dy = rng.standard_normal((N, C), dtype=np.float32)
    out = G.norm_backward(ctx, KINDS[kind], x, gamma, dy, eps, want_dbeta=(kind == "layer"))
    dx_cpu, dg_cpu, db_cpu = _norm_ref_backward(kind, x, gamma, dy, eps)
    assert_fp32_close(out["dx"], dx_cpu, f"{kind} dx at N={N}")
    if kind == "layer":
        _, dg64, db64 = cf.layernorm_grads(x, gamma, dy, eps)
    else:
        _, dg64 = cf.rmsnorm_grads(x, gamma, dy, eps)
        db64 = None
    tol = 1e-6 * np.sqrt(N) + 2e-6 * np.abs(dg64)
    err_gpu = np.abs(out["dgamma"] - dg64)
    err_cpu = np.abs(dg_cpu - dg64).max()
    assert (err_gpu <= tol).all(), (err_gpu.max(), tol.max())
    assert err_gpu.max() <= err_cpu + 1e-6, (err_gpu.max(), err_cpu)
    # and against the CPU restatement at the tolerance the reference's own
    # checker uses for these sums (debug/check_qwen_kernel.py:128-130, atol 1e-4 scaled by sqrt(N/14))
    assert_fp32_close(out["dgamma"], dg_cpu, "dgamma vs cpu", rtol=1e-5, atol=1e-4 * np.sqrt(N / 14))
    if db64 is not None:
        assert (np.abs(out["dbeta"] - db64) <= 1e-6 * np.sqrt(N) + 2e-6 * np.abs(db64)).all()
        assert_fp32_close(out["dbeta"], db_cpu, "dbeta vs cpu", rtol=1e-5, atol=1e-4 * np.sqrt(N / 14))


@pytest.mark.parametrize("kind", ["layer", "rms"])
@pytest.mark.parametrize("C", [384, 1536, 4096, 50])
def test_fused_residual_norm_forward(ctx, kind, C):
    rng = _rng(9)
    shape = (29, C)
    x = rng.standard_normal(shape, dtype=np.float32)
    r = rng.standard_normal(shape, dtype=np.float32)
    gamma = (1 + 0.02 * rng.standard_normal(C)).astype(np.float32)
    beta = (0.02 * rng.standard_normal(C)).astype(np.float32) if kind == "layer" else None
    y, h = G.norm_forward(ctx, KINDS[kind], x, gamma, beta, 1e-5, residual=r, want_h=True)
    h_ref, y_ref = ref.add_norm_forward(kind, x, r, gamma, beta, 1e-5)
    np.testing.assert_array_equal(h, h_ref)   # a single fp32 add: bit-exact
    assert_fp32_close(y, y_ref, f"add+{kind} forward")


@pytest.mark.parametrize("kind", ["layer", "rms"])
@pytest.mark.parametrize("C", [384, 1536, 4096, 8192, 72])
def test_norm_bf16_io(ctx, kind, C):
    rng = _rng(10)
    shape = (23, C)
    xb = to_bf16_bits(rng.standard_normal(shape, dtype=np.float32))
    rb = to_bf16_bits(rng.standard_normal(shape, dtype=np.float32))
    dyb = to_bf16_bits(rng.standard_normal(shape, dtype=np.float32))
    gamma = (1 + 0.02 * rng.standard_normal(C)).astype(np.float32)
    beta = (0.02 * rng.standard_normal(C)).astype(np.float32) if kind == "layer" else None
    eps = 1e-5
    x, r, dy = from_bf16_bits(xb), from_bf16_bits(rb), from_bf16_bits(dyb)
    # forward, plain and with the residual fused
    y, _ = G.norm_forward(ctx, KINDS[kind], xb, gamma, beta, eps)
    assert_bf16_close(from_bf16_bits(y), _norm_ref_forward(kind, x, gamma, beta, eps), f"bf16 {kind} forward")
    y, h = G.norm_forward(ctx, KINDS[kind], xb, gamma, beta, eps, residual=rb, want_h=True)
    h_ref = ref.round_bf16(x + r)
    np.testing.assert_array_equal(h, to_bf16_bits(x + r))
    assert_bf16_close(from_bf16_bits(y), _norm_ref_forward(kind, h_ref, gamma, beta, eps), f"bf16 add+{kind}")
    # backward
    out = G.norm_backward(ctx, KINDS[kind], xb, gamma, dyb, eps, want_dbeta=(kind == "layer"))
    dx, dgamma, dbeta = _norm_ref_backward(kind, x, gamma, dy, eps)
    assert_bf16_close(from_bf16_bits(out["dx"]), dx, f"bf16 {kind} dx")
    assert_fp32_close(out["dgamma"], dgamma, "bf16-io dgamma (fp32 accumulate)", rtol=1e-5, atol=2e-6)
    if kind == "layer":
        assert_fp32_close(out["dbeta"], dbeta, "bf16-io dbeta", rtol=1e-5, atol=2e-6)


# ---------------------------------------------------------------------------
# activations
# ---------------------------------------------------------------------------
ACT_SHAPES = [(2, 16, 64), (512, 512), (257, 1536), (3, 5, 7), (1,), (4099,)]


@pytest.mark.parametrize("shape", ACT_SHAPES)
def test_gelu_fp32(ctx, shape):
    rng = _rng(5)
    x = rng.standard_normal(shape, dtype=np.float32)
    dy = rng.standard_normal(shape, dtype=np.float32)
    assert_fp32_close(G.unary(ctx, "agrad_gelu_forward", x), ref.gelu_forward(x), f"gelu {shape}")
    dx = np.zeros_like(x)
    ref.gelu_backward_into(x, dy, dx)
    assert_fp32_close(G.unary_backward(ctx, "agrad_gelu_backward", x, dy), dx, f"gelu bwd {shape}")
    dx0 = rng.standard_normal(shape, dtype=np.float32)
    acc = dx0.copy()
    ref.gelu_backward_into(x, dy, acc)
    got = G.unary_backward(ctx, "agrad_gelu_backward", x, dy, dx_init=dx0, flags=capi.ACC_INPUT_GRAD)
    assert_fp32_close(got, acc, f"gelu bwd accumulate {shape}")


def test_gelu_dense_sweep_and_special_values(ctx):
    """tanhf on the device against np.tanh over [-10, 10], plus the limits."""
    x = np.linspace(-10, 10, 2_000_001, dtype=np.float32)
    got = G.unary(ctx, "agrad_gelu_forward", x)
    assert_fp32_close(got, ref.gelu_forward(x), "gelu sweep")
    assert np.abs(got - cf.gelu(x)).max() < 2e-6
    one = np.ones_like(x)
    dgot = G.unary_backward(ctx, "agrad_gelu_backward", x, one)
    dref = np.zeros_like(x)
    ref.gelu_backward_into(x, one, dref)
    # The CPU forms 1 - t*t from the rounded tanh; one ulp of t moves its result
    # by 6e-8 * |x| C (1 + A3 x^2), which passes 1e-6 at |x| ~ 4.9.  Inside that
    # range the stated tolerance holds; over the whole sweep the device value is
    # the one nearer the float64 derivative.
    core = np.abs(x) <= 4.5
    assert_fp32_close(dgot[core], dref[core], "gelu' sweep, |x| <= 4.5")
    d64 = cf.gelu_grad(x)
    assert_fp32_parity(dgot, dref, d64, "gelu' sweep")
    assert np.abs(dgot - d64).max() <= 4e-7   # values reach 1.13: two ulp
    assert np.abs(dgot - d64).max() <= np.abs(dref - d64).max()
    sp = np.array([0.0, -0.0, 30.0, -30.0, 1e-20, 80.0, -80.0], dtype=np.float32)
    y = G.unary(ctx, "agrad_gelu_forward", sp)
    assert y[0] == 0 and y[2] == 30.0 and y[3] == 0 and y[5] == 80.0 and y[6] == 0
    d = G.unary_backward(ctx, "agrad_gelu_backward", sp, np.ones_like(sp))
    assert d[0] == 0.5 and d[2] == 1.0 and d[3] == 0.0


@pytest.mark.parametrize("shape", ACT_SHAPES)
def test_relu2_fp32_bit_exact(ctx, shape):
    rng = _rng(11)
    x = rng.standard_normal(shape, dtype=np.float32)
    dy = rng.standard_normal(shape, dtype=np.float32)
    np.testing.assert_array_equal(G.unary(ctx, "agrad_relu2_forward", x), ref.relu2_forward(x))
    dx = np.zeros_like(x)
    ref.relu2_backward_into(x, dy, dx)
    np.testing.assert_array_equal(G.unary_backward(ctx, "agrad_relu2_backward", x, dy) + 0.0, dx + 0.0)
    # closed form: y = max(x,0)^2 and dx = 2 max(x,0) dy
    assert np.abs(G.unary(ctx, "agrad_relu2_forward", x) - cf.relu2(x)).max() < 1e-6


@pytest.mark.parametrize("rows,H", [(32, 64), (17, 8960), (5, 14336), (9, 50), (3, 1)])
def test_swiglu_fp32(ctx, rows, H):
    rng = _rng(12)
    gu = rng.standard_normal((rows, 2 * H), dtype=np.float32) * 2
    dh = rng.standard_normal((rows, H), dtype=np.float32)
    assert_fp32_close(G.swiglu_forward(ctx, gu), ref.swiglu_forward(gu), f"swiglu {rows}x{H}")
    want = ref.swiglu_backward(gu, dh)
    assert_fp32_close(G.swiglu_backward(ctx, gu, dh, inplace=True), want, "swiglu bwd in place")
    assert_fp32_close(G.swiglu_backward(ctx, gu, dh, inplace=False), want, "swiglu bwd out of place")
    d0 = rng.standard_normal(gu.shape, dtype=np.float32)
    got = G.swiglu_backward(ctx, gu, dh, inplace=False, dgu_init=d0, flags=capi.ACC_INPUT_GRAD)
    assert_fp32_parity(got, d0 + want, d0.astype(np.float64) + cf.swiglu_grads(gu, dh), "swiglu bwd accumulate")


def test_swiglu_extremes(ctx):
    g = np.array([[-100.0, -20.0, 0.0, 20.0, 100.0, -0.0]], dtype=np.float32)
    u = np.full_like(g, 3.0)
    gu = np.concatenate([g, u], axis=1)
    got = G.swiglu_forward(ctx, gu)
    assert_fp32_close(got, ref.swiglu_forward(gu), "swiglu extremes")
    assert got[0, 2] == 0 and got[0, 4] == 300.0


@pytest.mark.parametrize("name,fwd,bwd", [
    ("gelu", ref.gelu_forward, ref.gelu_backward_into),
    ("relu2", ref.relu2_forward, ref.relu2_backward_into)])
def test_unary_bf16_io(ctx, name, fwd, bwd):
    rng = _rng(13)
    shape = (33, 1544)
    xb = to_bf16_bits(rng.standard_normal(shape, dtype=np.float32))
    dyb = to_bf16_bits(rng.standard_normal(shape, dtype=np.float32))
    x, dy = from_bf16_bits(xb), from_bf16_bits(dyb)
    y = G.unary(ctx, f"agrad_{name}_forward", xb)
    if name == "relu2":   # exact fp32 arithmetic, one RNE on store
        np.testing.assert_array_equal(y, to_bf16_bits(fwd(x)))
    else:
        assert_bf16_close(from_bf16_bits(y), fwd(x), f"bf16 {name}")
    dx = np.zeros_like(x)
    bwd(x, dy, dx)
    got = G.unary_backward(ctx, f"agrad_{name}_backward", xb, dyb)
    assert_bf16_close(from_bf16_bits(got), dx, f"bf16 {name} bwd")


def test_swiglu_bf16_io(ctx):
    rng = _rng(14)
    rows, H = 19, 8960
    gub = to_bf16_bits(rng.standard_normal((rows, 2 * H), dtype=np.float32))
    dhb = to_bf16_bits(rng.standard_normal((rows, H), dtype=np.float32))
    gu, dh = from_bf16_bits(gub), from_bf16_bits(dhb)
    assert_bf16_close(from_bf16_bits(G.swiglu_forward(ctx, gub)), ref.swiglu_forward(gu), "bf16 swiglu")
    assert_bf16_close(from_bf16_bits(G.swiglu_backward(ctx, gub, dhb)), ref.swiglu_backward(gu, dh), "bf16 swiglu bwd")


@pytest.mark.parametrize("rows,H,h0,h", [(7, 64, 0, 64), (7, 64, 16, 32), (33, 200, 8, 100), (5, 96, 3, 50),
                                        (2, 8960, 2048, 2048), (3, 10, 9, 1), (4, 40, 40, 0)])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_swiglu_forward_column_tile(ctx, rows, H, h0, h, dtype):
    """agrad_swiglu_forward_tile (swiglu_forward_tile_kernel, metal_ops.metal:12043-12088):
    columns h0 .. h0 + h of the hidden activations, dense [rows, h] -- the very bits of
    those columns of the full forward call (aligned tiles take the 16-byte path, odd
    offsets and widths the element-wise one), and within tolerance of the CPU kernel"""
    import ctypes as Ct
    rng = _rng(15 + h0)
    gu = (2 * rng.standard_normal((rows, 2 * H))).astype(np.float32)
    if dtype == "bf16":
        store = to_bf16_bits(gu)
        seen = from_bf16_bits(store)
        dt = capi.BF16
    else:
        store, seen, dt = gu, gu, capi.F32
    full = G.swiglu_forward(ctx, store)
    d_gu = ctx.upload(store)
    tile = ctx.upload(np.full((rows, max(h, 1)), 0x7F7F if dtype == "bf16" else 7.0, store.dtype))
    ctx.call("agrad_swiglu_forward_tile", dt, Ct.c_void_p(d_gu.ptr), Ct.c_void_p(tile.ptr), rows, H, h0, h)
    ctx.synchronize()
    got = tile.download()
    if h:
        got = got.reshape(-1)[:rows * h].reshape(rows, h)
        np.testing.assert_array_equal(got, full[:, h0:h0 + h])
        want = ref.swiglu_forward(seen)[:, h0:h0 + h]
        if dtype == "bf16":
            assert_bf16_close(from_bf16_bits(got), want, "swiglu tile")
        else:
            assert_fp32_close(got, want, "swiglu tile")
    with pytest.raises(capi.AgradError):       # the tile must lie inside the row
        ctx.call("agrad_swiglu_forward_tile", dt, Ct.c_void_p(d_gu.ptr), Ct.c_void_p(tile.ptr), rows, H, H - 1, 2)
    d_gu.free()
    tile.free()


# ---------------------------------------------------------------------------
# RoPE
# ---------------------------------------------------------------------------
ROPE_CASES = [
    # B, T, H, HKV, D, theta
    (2, 16, 6, 6, 64, 1e4),      # config 2 heads
    (2, 33, 12, 2, 128, 1e6),    # config 4 heads (GQA)
    (1, 9, 32, 8, 128, 5e5),     # config 5 heads
    (2, 5, 3, 1, 6, 1e4),        # D/2 = 3: scalar kernel
]


@pytest.mark.parametrize("B,T,H,HKV,D,theta", ROPE_CASES)
@pytest.mark.parametrize("sign", [1, -1])
@pytest.mark.parametrize("backward", [False, True])
def test_rope_fp32_bit_exact(ctx, B, T, H, HKV, D, theta, sign, backward):
    rng = _rng(15)
    q = rng.standard_normal((B, T, H, D), dtype=np.float32)
    k = rng.standard_normal((B, T, HKV, D), dtype=np.float32)
    cos, sin = ref.rope_tables(T, D, theta)
    gq, gk = G.rope(ctx, q, k, cos, sin, sign, backward)
    rq, rk = q.copy(), k.copy()
    ref.rope_signed(rq, rk, cos, sin, sign, backward)
    # separate fp32 multiplies and adds in the reference's order: identical bits
    np.testing.assert_array_equal(gq, rq)
    np.testing.assert_array_equal(gk, rk)
    if sign == -1:
        nq, nk = q.copy(), k.copy()
        ref.rope_nanochat(nq, nk, cos, sin, backward)
        np.testing.assert_array_equal(gq, nq)
        np.testing.assert_array_equal(gk, nk)


@pytest.mark.parametrize("B,T,H,HKV,D,theta", ROPE_CASES)
@pytest.mark.parametrize("sign", [1, -1])
@pytest.mark.parametrize("backward", [False, True])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_rope_bhtd_layout(ctx, B, T, H, HKV, D, theta, sign, backward, dtype):
    """agrad_rope_qk_bhtd on q[B,H,T,D], k[B,HKV,T,D] gives the very bits of agrad_rope_qk
    on the transposed tensors, which is bit-exact against the CPU loops in fp32
    (test_rope_fp32_bit_exact); also k alone and q alone"""
    import ctypes as Ct
    rng = _rng(17)
    q = rng.standard_normal((B, T, H, D), dtype=np.float32)
    k = rng.standard_normal((B, T, HKV, D), dtype=np.float32)
    cos, sin = ref.rope_tables(T, D, theta)
    if dtype == "bf16":
        q, k, dt = to_bf16_bits(q), to_bf16_bits(k), capi.BF16
    else:
        dt = capi.F32
    want_q, want_k = G.rope(ctx, q, k, cos, sin, sign, backward)
    if dtype == "f32":
        rq, rk = q.copy(), k.copy()
        ref.rope_signed(rq, rk, cos, sin, sign, backward)
        np.testing.assert_array_equal(want_q, rq)
    d_c, d_s = ctx.upload(cos), ctx.upload(sin)
    for with_q, with_k in ((True, True), (True, False)):
        d_q = ctx.upload(np.ascontiguousarray(q.transpose(0, 2, 1, 3)))
        d_k = ctx.upload(np.ascontiguousarray(k.transpose(0, 2, 1, 3))) if with_k else None
        ctx.call("agrad_rope_qk_bhtd", dt, Ct.c_void_p(d_q.ptr), Ct.c_void_p(d_k.ptr) if d_k is not None else None,
                 Ct.c_void_p(d_c.ptr), Ct.c_void_p(d_s.ptr), B, T, H, HKV if with_k else 0, D, sign, int(backward))
        ctx.synchronize()
        np.testing.assert_array_equal(d_q.download().transpose(0, 2, 1, 3), want_q)
        d_q.free()
        if d_k is not None:
            np.testing.assert_array_equal(d_k.download().transpose(0, 2, 1, 3), want_k)
            d_k.free()
    d_c.free()
    d_s.free()


def test_rope_invariants(ctx):
    rng = _rng(16)
    B, T, H, HKV, D = 2, 64, 12, 2, 128
    q = rng.standard_normal((B, T, H, D), dtype=np.float32)
    k = rng.standard_normal((B, T, HKV, D), dtype=np.float32)
    cos, sin = ref.rope_tables(T, D, 1e6)
    fq, fk = G.rope(ctx, q, k, cos, sin, 1, False)
    # position 0 is the identity; the rotation preserves each (lo, hi) pair's norm
    np.testing.assert_array_equal(fq[:, 0], q[:, 0])
    half = D // 2
    n0 = q[..., :half] ** 2 + q[..., half:] ** 2
    n1 = fq[..., :half] ** 2 + fq[..., half:] ** 2
    assert np.abs(n1 - n0).max() < 1e-5
    # backward undoes forward; the two sign conventions are mutual inverses
    bq, bk = G.rope(ctx, fq, fk, cos, sin, 1, True)
    assert np.abs(bq - q).max() < 1e-6 and np.abs(bk - k).max() < 1e-6
    iq, _ = G.rope(ctx, fq, fk, cos, sin, -1, False)
    np.testing.assert_array_equal(iq, bq)
    # q only
    oq, ok = G.rope(ctx, q, None, cos, sin, 1, False)
    np.testing.assert_array_equal(oq, fq)
    assert ok is None
    # float64 closed form
    assert np.abs(fq - cf.rope(q, cos, sin, 1)).max() < 1e-6


def test_rope_bf16_io(ctx):
    rng = _rng(17)
    B, T, H, HKV, D = 2, 31, 12, 2, 128
    qb = to_bf16_bits(rng.standard_normal((B, T, H, D), dtype=np.float32))
    kb = to_bf16_bits(rng.standard_normal((B, T, HKV, D), dtype=np.float32))
    cos, sin = ref.rope_tables(T, D, 1e6)
    gq, gk = G.rope(ctx, qb, kb, cos, sin, 1, False)
    rq, rk = from_bf16_bits(qb), from_bf16_bits(kb)
    ref.rope_signed(rq, rk, cos, sin, 1, False)
    np.testing.assert_array_equal(gq, to_bf16_bits(rq))  # fp32 math is exact; one RNE on store
    np.testing.assert_array_equal(gk, to_bf16_bits(rk))


# ---------------------------------------------------------------------------
# embedding
# ---------------------------------------------------------------------------
def test_gather_reference_case(ctx):
    """verify_model.py:298-318: B,T,V,C = 2,3,11,4, seed 1234, w = 0.1 N(0,1)."""
    rng = np.random.default_rng(1234)
    B, T, V, C = 2, 3, 11, 4
    idx = rng.integers(0, V, size=(B, T), dtype=np.int32)
    w = (rng.standard_normal((V, C)) * 0.1).astype(np.float32)
    got = G.gather_forward(ctx, idx, w)
    np.testing.assert_array_equal(got.view(np.uint32), w[idx].view(np.uint32))
    up = rng.standard_normal((B, T, C)).astype(np.float32)
    dW = np.zeros_like(w)
    ref.gather_backward_into(idx, up, dW)
    np.testing.assert_array_equal(G.embedding_backward(ctx, idx, up, V), dW)


@pytest.mark.parametrize("B,T,V,C", [(4, 128, 50257, 128), (3, 37, 1000, 384), (2, 50, 300, 768),
                                     (2, 9, 97, 1536), (2, 7, 53, 50), (1, 1, 1, 4)])
def test_gather_forward_bit_exact(ctx, B, T, V, C):
    rng = _rng(18)
    ids = rng.integers(0, V, size=(B, T), dtype=np.int32)
    W = (0.02 * rng.standard_normal((V, C))).astype(np.float32)
    W.reshape(-1)[:3] = [np.nan, -0.0, np.inf]          # payloads must survive the copy
    ids.reshape(-1)[0] = 0
    got = G.gather_forward(ctx, ids, W)
    np.testing.assert_array_equal(got.view(np.uint32), ref.gather_forward(ids, W).view(np.uint32))
    Wb = to_bf16_bits(W)
    np.testing.assert_array_equal(G.gather_forward(ctx, ids, Wb), Wb[ids])


@pytest.mark.parametrize("B,T,V,C", [(4, 128, 50257, 128), (3, 37, 1000, 768), (2, 7, 53, 50)])
def test_embedding_sum_forward(ctx, B, T, V, C):
    rng = _rng(19)
    ids = rng.integers(0, V, size=(B, T), dtype=np.int32)
    wte = (0.02 * rng.standard_normal((V, C))).astype(np.float32)
    wpe = (0.02 * rng.standard_normal((T, C))).astype(np.float32)
    got = G.gather_forward(ctx, ids, wte, wpe)
    np.testing.assert_array_equal(got, ref.embedding_sum_forward(ids, wte, wpe))  # one fp32 add


def test_gather_out_of_range_id_raises(ctx):
    ids = np.array([[0, 5, 11]], dtype=np.int32)
    W = np.ones((11, 8), np.float32)
    with pytest.raises(IndexError):
        G.gather_forward(ctx, ids, W)
    with pytest.raises(IndexError):
        G.embedding_backward(ctx, np.array([[0, -1]], np.int32), np.ones((1, 2, 8), np.float32), 11)
    # the context stays usable
    np.testing.assert_array_equal(G.gather_forward(ctx, np.array([[1, 2]], np.int32), W), W[[[1, 2]]])


def _zipf_ids(rng, n, V, s=1.1):
    p = np.arange(1, V + 1, dtype=np.float64) ** (-s)
    p /= p.sum()
    return rng.choice(V, size=n, p=p).astype(np.int32)


@pytest.mark.parametrize("B,T,V,C,dist", [
    (2, 16, 64, 64, "uniform"),
    (4, 128, 50257, 128, "uniform"),      # config 1
    (8, 512, 32768, 384, "uniform"),      # config 2 at a quarter of its rows
    (3, 700, 97, 50, "uniform"),          # heavy duplication, scalar columns
    (4, 1024, 1000, 768, "zipf"),         # long runs crossing chunk edges
    (1, 3000, 1, 16, "uniform"),          # a single token: one run over every chunk
    (1, 12000, 1, 8, "uniform"),          # one token group larger than the sort's LDS list
    (2, 8000, 5, 24, "uniform"),          # several such groups
    (4, 8192, 4000, 64, "zipf"),          # N = 32768: 256 hash groups
    (2, 24000, 4000, 64, "zipf"),         # N = 48000: 512 hash groups
    (3, 23000, 4000, 32, "zipf"),         # N = 69000: the radix-sort path
])
def test_embedding_backward_fp32(ctx, B, T, V, C, dist):
    rng = _rng(20)
    ids = (_zipf_ids(rng, B * T, V) if dist == "zipf" else rng.integers(0, V, size=B * T, dtype=np.int32)).reshape(B, T)
    dY = rng.standard_normal((B, T, C), dtype=np.float32)
    got = G.embedding_backward(ctx, ids, dY, V)
    dW = np.zeros((V, C), np.float32)
    ref.gather_backward_into(ids, dY, dW)
    # the CPU adds a token's rows one by one in fp32: its own rounding noise grows
    # with the longest run (about 6e-8 * run length for N(0,1) rows), so the
    # absolute budget follows it; for runs of a few rows it is 2e-6
    longest = int(np.bincount(ids.ravel(), minlength=V).max())
    atol = max(2e-6, 2.5e-7 * longest)
    assert_fp32_close(got, dW, f"embedding backward {dist}", rtol=1e-5, atol=atol)
    # rows of tokens that never occur stay exactly zero; column sums are preserved
    unseen = np.setdiff1d(np.arange(V), ids.ravel())
    assert not got[unseen].any()
    assert np.abs(got.sum(0, dtype=np.float64) - dY.reshape(-1, C).sum(0, dtype=np.float64)).max() < 1e-3 * np.sqrt(B * T)
    # against the float64 row loop, on the scale of the sum
    d64 = cf.gather_backward(ids, dY, V)
    assert np.abs(got - d64).max() <= 1e-6 * max(1.0, np.abs(d64).max()) * 8
    # deterministic: a second run gives the same bits
    np.testing.assert_array_equal(got, G.embedding_backward(ctx, ids, dY, V))
    # accumulate onto an existing table
    base = rng.standard_normal((V, C), dtype=np.float32)
    acc = G.embedding_backward(ctx, ids, dY, V, dW_init=base, flags=capi.ACC_PARAM_GRAD)
    assert_fp32_close(acc, base + dW, "embedding backward accumulate", rtol=1e-5, atol=max(1e-4, atol))
    np.testing.assert_array_equal(acc[unseen], base[unseen])


@pytest.mark.parametrize("dist", ["uniform", "zipf"])
def test_embedding_backward_beyond_the_one_launch_ordering(ctx, dist):
    """Above 65536 rows the ids are ordered by the library radix sort (several launches)
    instead of the one-launch hash-group ordering: same contract -- np.add.at's sums, rows
    without a token untouched, the same bits on every run, an id outside the table
    reported -- and the call is refused while a graph is being recorded."""
    import ctypes as Ct
    rng = _rng(31)
    N, V, C = 131072, 30000, 32
    ids = (_zipf_ids(rng, N, V) if dist == "zipf" else rng.integers(0, V, size=N, dtype=np.int32)).reshape(1, N)
    dY = rng.standard_normal((1, N, C), dtype=np.float32)
    got = G.embedding_backward(ctx, ids, dY, V)
    dW = np.zeros((V, C), np.float32)
    ref.gather_backward_into(ids, dY, dW)
    longest = int(np.bincount(ids.ravel(), minlength=V).max())
    assert_fp32_close(got, dW, f"embedding backward, {N} rows, {dist}", rtol=1e-5, atol=max(2e-6, 2.5e-7 * longest))
    if longest <= 127:
        np.testing.assert_array_equal(got, dW)          # every run short enough for np.add.at's own order
    unseen = np.setdiff1d(np.arange(V), ids.ravel())
    assert not got[unseen].any()
    np.testing.assert_array_equal(got, G.embedding_backward(ctx, ids, dY, V))
    # the pre-sorted pair takes the same path at this size
    d_ids, d_dY = ctx.upload(ids.reshape(-1)), ctx.upload(dY.reshape(N, C))
    d_W, out = ctx.zeros((V, C), np.float32), ctx.empty((N, C), np.float32)
    order = ctx.empty((6 * N + 128,), np.uint32)
    sws_b = ctx.lib.agrad_embedding_sort_workspace_bytes(N, V)
    bws_b = ctx.lib.agrad_embedding_backward_sorted_workspace_bytes(N, C)
    sws, bws = ctx.empty((sws_b,), np.uint8), ctx.empty((max(bws_b, 1),), np.uint8)
    dW2 = ctx.zeros((V, C), np.float32)

    def vp(d):
        return Ct.c_void_p(d.ptr)
    ctx.call("agrad_gather_forward_sorted", capi.F32, vp(d_ids), vp(d_W), None, vp(out), N, 1, C, V, vp(order), vp(sws), sws_b)
    ctx.call("agrad_embedding_backward_sorted", capi.F32, vp(order), vp(d_dY), vp(dW2), None, vp(bws), bws_b, N, 1, C, V, 0)
    ctx.synchronize()
    np.testing.assert_array_equal(dW2.download(), got)
    _check_order(order.download(), N, ids.reshape(-1), V)
    # refused under graph capture (the library sort is not recordable), and the capture survives
    ctx.call("agrad_graph_begin")
    with pytest.raises((RuntimeError, ValueError)):
        ctx.call("agrad_gather_forward_sorted", capi.F32, vp(d_ids), vp(d_W), None, vp(out), N, 1, C, V, vp(order), vp(sws), sws_b)
    ctx.call("agrad_fill", sws.ptr, 0, 0, 4, 16)         # something recordable, so the graph is not empty
    gid = Ct.c_uint64(0)
    ctx.call("agrad_graph_end", Ct.byref(gid))
    ctx.call("agrad_graph_launch", gid.value)
    ctx.synchronize()
    ctx.call("agrad_graph_destroy", gid.value)
    # an id outside the table is reported when the work has run
    bad = ids.reshape(-1).copy()
    bad[N // 2] = V + 5
    d_bad = ctx.upload(bad)
    ctx.call("agrad_gather_forward_sorted", capi.F32, vp(d_bad), vp(d_W), None, vp(out), N, 1, C, V, vp(order), vp(sws), sws_b)
    with pytest.raises(IndexError):
        ctx.synchronize()
    ctx.synchronize()
    for d in (d_ids, d_dY, d_W, out, order, sws, bws, dW2, d_bad):
        d.free()


@pytest.mark.parametrize("N,C,tokens", [(4096, 10240, 1), (2000, 8196, 3), (65536, 8, 1), (40000, 72, 2)])
def test_embedding_backward_long_runs_wide_rows_and_deep_trees(ctx, N, C, tokens):
    """Long runs at the corners of their hand-off scheme: rows of more than 32 column blocks
    (several blocks then share one arrival counter), a scalar-column width, a run long
    enough for the second level of adding-up (more than 2048 rows), and two such runs side
    by side.  Against the float64 row loop and the sequential fp32 loop, twice (the
    counters must be back at zero), and through the accumulate flag."""
    rng = _rng(33)
    V = 50
    ids = rng.integers(0, tokens, size=N, dtype=np.int32).reshape(1, N) * 7 + 3
    dY = rng.standard_normal((1, N, C), dtype=np.float32)
    got = G.embedding_backward(ctx, ids, dY, V)
    rows = np.flatnonzero(np.bincount(ids.ravel(), minlength=V))
    d64 = np.zeros((V, C))
    seq = np.zeros((V, C), np.float32)
    for t in rows:
        sel = dY[0][ids[0] == t]
        d64[t] = sel.astype(np.float64).sum(0)
        seq[t] = np.add.accumulate(sel, axis=0, dtype=np.float32)[-1]          # np.add.at's order
    assert_fp32_parity(got, seq, d64, f"dW {N}x{C}, {tokens} tokens")
    assert not np.delete(got, rows, axis=0).any()
    np.testing.assert_array_equal(got, G.embedding_backward(ctx, ids, dY, V))
    base = rng.standard_normal((V, C), dtype=np.float32)
    acc = G.embedding_backward(ctx, ids, dY, V, dW_init=base, flags=capi.ACC_PARAM_GRAD)
    np.testing.assert_array_equal(acc, base + got)


def _sums_in_row_order(ids, dY, V):
    """dW[t] = ((dY[r0] + dY[r1]) + dY[r2]) + ... over the rows of token t in ascending order, in
    fp32: what np.add.at does to a zero table, written with one vector add per position in
    the run instead of one numpy call per row (cpu_ops.gather_backward_into takes 20 s
    where this takes a fraction of one; the test below checks the two against each other on
    a slice)"""
    N, C = dY.shape
    rows = np.argsort(ids, kind="stable")
    toks = ids[rows]
    starts = np.flatnonzero(np.concatenate([[True], toks[1:] != toks[:-1]]))
    lens = np.diff(np.concatenate([starts, [N]]))
    dW = np.zeros((V, C), np.float32)
    for L in np.unique(lens):
        first = starts[lens == L]
        acc = dY[rows[first]].copy()
        for j in range(1, L):
            acc += dY[rows[first + j]]
        dW[toks[first]] = acc
    return dW


def _ids_with_runs(rng, lengths, V):
    """a shuffled id list in which token k occurs lengths[k] times"""
    toks = rng.choice(V, size=len(lengths), replace=False).astype(np.int32)
    return rng.permutation(np.repeat(toks, lengths))


@pytest.mark.parametrize("C,io", [(96, "f32"), (1024, "f32"), (2048, "bf16")])
def test_embedding_backward_every_run_length(ctx, C, io):
    """Runs of every length around the places where the gradient kernel changes its way of
    adding a run up: a token's only row (moved by the row's own wave); 2 to 10 rows (added by
    the first row's wave when a wave takes one column block -- narrow rows -- and by a task
    wave when it takes several: the wide shapes here start more than 131072 waves); 11 to
    127 rows (a task wave, ascending row order: np.add.at's own bits); 128 rows and more
    (64-row chunks, the last taking the rest, in groups of 16).  Twice (the arrival counters
    must be back at zero) and through the accumulate flag."""
    rng = _rng(C + 5)
    lengths = np.array(list(range(1, 14)) * 40 + [1] * 20000 + [2] * 3000 + [3] * 500
                       + [62, 63, 64, 65, 66, 126, 127, 128, 129, 130, 191, 192, 193, 255, 256, 257, 1023, 1024, 1025, 1100, 2049, 2500])
    V = 26000
    ids = _ids_with_runs(rng, lengths, V)
    N = ids.size
    if io == "bf16":
        dY = to_bf16_bits(rng.random((1, N, C), dtype=np.float32) - 0.5)
        dY32 = from_bf16_bits(dY)
    else:
        dY = dY32 = rng.random((1, N, C), dtype=np.float32) - 0.5
    ids2 = ids.reshape(1, N)
    got = G.embedding_backward(ctx, ids2, dY, V)
    seq = _sums_in_row_order(ids, dY32[0], V)                          # np.add.at: ascending rows
    part = np.zeros((V, 16), np.float32)
    ref.gather_backward_into(ids2, np.ascontiguousarray(dY32[:, :, :16]), part)
    np.testing.assert_array_equal(seq[:, :16], part)
    run = np.bincount(ids, minlength=V)
    if io == "bf16":
        got32 = from_bf16_bits(got)
        short = (run >= 1) & (run <= 127)
        np.testing.assert_array_equal(got[short], to_bf16_bits(seq[short]))       # the same fp32 sum, rounded once
        assert_bf16_close(got32, seq, "bf16 embedding backward, every run length")
        assert not got32[run == 0].any()
    else:
        short = run <= 127
        np.testing.assert_array_equal(got[short], seq[short])
        d64 = np.zeros((V, C))
        for t in np.flatnonzero(run > 127):
            d64[t] = dY32[0][ids == t].astype(np.float64).sum(0)
        long_rows = run > 127
        assert_fp32_parity(got[long_rows], seq[long_rows], d64[long_rows], f"dW of the long runs, C = {C}")
        base = rng.standard_normal((V, C), dtype=np.float32)
        acc = G.embedding_backward(ctx, ids2, dY, V, dW_init=base, flags=capi.ACC_PARAM_GRAD)
        np.testing.assert_array_equal(acc, base + got)
    np.testing.assert_array_equal(got, G.embedding_backward(ctx, ids2, dY, V))


def test_embedding_backward_short_runs_bit_exact(ctx):
    """Runs of up to 127 rows are summed by their first row in ascending row order: the
    same sequence of fp32 adds as np.add.at."""
    rng = _rng(21)
    V, C, N = 4096, 128, 512
    # every token occurs exactly four times
    toks = rng.choice(V, size=N // 4, replace=False).astype(np.int32)
    ids = rng.permutation(np.repeat(toks, 4)).reshape(1, N)
    dY = rng.standard_normal((1, N, C), dtype=np.float32)
    got = G.embedding_backward(ctx, ids, dY, V)
    dW = np.zeros((V, C), np.float32)
    ref.gather_backward_into(ids, dY, dW)
    np.testing.assert_array_equal(got, dW)


def test_embedding_backward_bf16_io(ctx):
    rng = _rng(22)
    B, T, V, C = 4, 256, 5000, 1536
    ids = rng.integers(0, V, size=(B, T), dtype=np.int32)
    dYb = to_bf16_bits(rng.standard_normal((B, T, C), dtype=np.float32))
    got = G.embedding_backward(ctx, ids, dYb, V)
    dW = np.zeros((V, C), np.float32)
    ref.gather_backward_into(ids, from_bf16_bits(dYb), dW)
    assert_bf16_close(from_bf16_bits(got), dW, "bf16 embedding backward")


@pytest.mark.parametrize("B,T,C", [(4, 128, 128), (16, 64, 768), (3, 5, 7)])
def test_pos_embedding_backward(ctx, B, T, C):
    rng = _rng(23)
    dY = rng.standard_normal((B, T, C), dtype=np.float32)
    ids = rng.integers(0, 10, size=(B, T), dtype=np.int32)
    dwpe = np.zeros((T, C), np.float32)
    ref.embedding_sum_backward_into(ids, dY, None, dwpe)
    np.testing.assert_array_equal(G.pos_embedding_backward(ctx, dY), dwpe)  # b ascending: same adds
    base = rng.standard_normal((T, C), dtype=np.float32)
    got = G.pos_embedding_backward(ctx, dY, dwpe_init=base, flags=capi.ACC_PARAM_GRAD)
    assert_fp32_close(got, base + dwpe, "pos grad accumulate")


# ---------------------------------------------------------------------------
# fills and casts
# ---------------------------------------------------------------------------
def test_cast_f32_bf16_bit_exact(ctx):
    """fp32 -> bf16 on the device equals the reference's integer rule (utils.py:20-27)
    on random bit patterns, ties, infinities and NaN payloads; accumulate adds the
    widened old value first (metal_ops.metal:12010-12041)."""
    import ctypes as C
    rng = _rng(30)
    bits = rng.integers(0, 2 ** 32, size=1_000_003, dtype=np.uint64).astype(np.uint32)
    special = np.array([0x3F808000, 0x3F818000, 0x3F808001, 0x7F800000, 0xFF800000, 0x7F800001, 0x7FC00000,
                        0xFFFFFFFF, 0x7FA12345, 0x7F7FFFFF, 0x80000000, 0x00000001, 0x00008000, 0x00018000],
                       dtype=np.uint32)
    bits[:special.size] = special
    src = bits.view(np.float32)
    d_src = ctx.upload(src)
    d_dst = ctx.upload(np.zeros(src.size, np.uint16))
    ctx.call("agrad_cast_f32_to_bf16", C.c_void_p(d_src.ptr), C.c_void_p(d_dst.ptr), src.size, 0)
    ctx.synchronize()
    got = d_dst.download()
    np.testing.assert_array_equal(got, ref.f32_to_bf16_bits(src))
    # widen back: exact
    d_up = ctx.empty((src.size,), np.float32)
    ctx.call("agrad_cast_bf16_to_f32", C.c_void_p(d_dst.ptr), C.c_void_p(d_up.ptr), src.size)
    ctx.synchronize()
    np.testing.assert_array_equal(d_up.download().view(np.uint32), got.astype(np.uint32) << 16)
    # accumulate: dst = rne(src + widen(dst)) on finite values
    a = rng.standard_normal(4099).astype(np.float32)
    b = to_bf16_bits(rng.standard_normal(4099).astype(np.float32))
    d_a, d_b = ctx.upload(a), ctx.upload(b)
    ctx.call("agrad_cast_f32_to_bf16", C.c_void_p(d_a.ptr), C.c_void_p(d_b.ptr), a.size, 1)
    ctx.synchronize()
    np.testing.assert_array_equal(d_b.download(), ref.f32_to_bf16_bits(a + from_bf16_bits(b)))
    for d in (d_src, d_dst, d_up, d_a, d_b):
        d.free()


@pytest.mark.parametrize("itemsize,n,offset", [(4, 1000, 0), (4, 77, 12), (2, 1001, 2), (1, 4099, 3), (4, 1, 4), (2, 0, 0)])
def test_fill_patterns(ctx, itemsize, n, offset):
    dt = {1: np.uint8, 2: np.uint16, 4: np.uint32}[itemsize]
    total = 8192
    base = ctx.upload(np.full(total, 0xAB, np.uint8))
    bits = 0x3DCCCCCD if itemsize == 4 else (0x3DCD if itemsize == 2 else 0x5A)
    ctx.call("agrad_fill", base.buffer_id, offset, bits, itemsize, n)
    ctx.synchronize()
    want = np.full(total, 0xAB, np.uint8)
    want[offset:offset + n * itemsize] = np.full(n, bits, dtype=dt).view(np.uint8)
    np.testing.assert_array_equal(base.download(), want)
    base.free()


def test_add_and_accumulate(ctx):
    import ctypes as C
    rng = _rng(31)
    for n in (1, 5, 4096, 100_003):
        x = rng.standard_normal(n).astype(np.float32)
        y = rng.standard_normal(n).astype(np.float32)
        dx, dy_ = ctx.upload(x), ctx.upload(y)
        out = ctx.empty((n,), np.float32)
        ctx.call("agrad_add_forward", capi.F32, C.c_void_p(dx.ptr), C.c_void_p(dy_.ptr), C.c_void_p(out.ptr), n)
        ctx.call("agrad_grad_accumulate", capi.F32, C.c_void_p(dx.ptr), C.c_void_p(dy_.ptr), n, capi.ACC_INPUT_GRAD)
        ctx.synchronize()
        np.testing.assert_array_equal(out.download(), x + y)
        np.testing.assert_array_equal(dy_.download(), y + x)
        ctx.call("agrad_grad_accumulate", capi.F32, C.c_void_p(dx.ptr), C.c_void_p(dy_.ptr), n, 0)
        ctx.synchronize()
        np.testing.assert_array_equal(dy_.download(), x)
        for d in (dx, dy_, out):
            d.free()


# ---------------------------------------------------------------------------
# broadcast add and its column-sum gradient (cpu_add_forward / backward, backend.py:74-105)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("lead,inner", [(1, 8), (5, 7), (16, 1024), (64, 96), (65, 96), (700, 768), (4096, 50), (20000, 384)])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_broadcast_add_and_gradient(ctx, lead, inner, dtype):
    import ctypes as C
    rng = _rng(40 + inner)
    x = rng.standard_normal((lead, inner)).astype(np.float32)
    y = rng.standard_normal(inner).astype(np.float32)
    g = rng.standard_normal((lead, inner)).astype(np.float32)
    base = rng.standard_normal(inner).astype(np.float32)
    if dtype == "bf16":
        xs, ys, gs, bs = (to_bf16_bits(a) for a in (x, y, g, base))
        x, y, g, base = (from_bf16_bits(a) for a in (xs, ys, gs, bs))
        dt = capi.BF16
    else:
        xs, ys, gs, bs, dt = x, y, g, base, capi.F32
    dxs, dys, dgs = ctx.upload(xs), ctx.upload(ys), ctx.upload(gs)
    out = ctx.empty(xs.shape, xs.dtype)
    ctx.call("agrad_broadcast_add_forward", dt, C.c_void_p(dxs.ptr), C.c_void_p(dys.ptr), C.c_void_p(out.ptr), lead, inner)
    ws_bytes = ctx.lib.agrad_broadcast_grad_workspace_bytes(lead, inner)
    assert (ws_bytes > 0) == (lead > 64)
    ws = ctx.empty((max(ws_bytes, 16),), np.uint8)
    results = []
    for flags, init in ((0, np.full(inner, 7, bs.dtype)), (capi.ACC_PARAM_GRAD, bs)):
        ddy = ctx.upload(init)
        ctx.call("agrad_broadcast_add_backward", dt, C.c_void_p(dgs.ptr), C.c_void_p(ddy.ptr), C.c_void_p(ws.ptr),
                 ws_bytes, lead, inner, flags)
        ctx.synchronize()
        results.append(ddy.download())
        ddy.free()
    got_out = out.download()
    want = ref.add_forward(x, y)
    col = g.astype(np.float64).sum(0)
    mag = np.abs(g).astype(np.float64).sum(0)
    if dtype == "bf16":
        np.testing.assert_array_equal(got_out, to_bf16_bits(want))       # one add, one rounding
        assert_bf16_close(from_bf16_bits(results[0]), col, "bf16 column sum")
        assert_bf16_close(from_bf16_bits(results[1]), base + col, "bf16 column sum accumulate")
    else:
        np.testing.assert_array_equal(got_out, want)
        # an fp32 sum of `lead` terms in any fixed order: a few eps * sum|term|
        assert (np.abs(results[0] - col) <= 1e-7 * mag + 1e-6).all()
        assert (np.abs(results[1] - (base + col)) <= 1e-7 * (mag + np.abs(base)) + 1e-6).all()
        cpu = np.zeros(inner, np.float32)
        ref.add_backward_into(g, cpu)
        # the CPU adds the rows one by one in fp32; the tolerance is the one the
        # reference's own checker uses for such sums (debug/check_qwen_kernel.py:128-130)
        assert_fp32_close(results[0], cpu, "column sum vs cpu", rtol=1e-5, atol=max(2e-6, 1e-4 * np.sqrt(lead / 14)))
    for d in (dxs, dys, dgs, out, ws):
        d.free()


@pytest.mark.parametrize("B,T,V,C,dist", [(4, 128, 50257, 128, "uniform"), (2, 700, 300, 48, "zipf"),
                                          (32, 512, 32768, 384, "uniform"), (5, 4000, 1000, 64, "zipf"),
                                          (5, 14000, 3000, 32, "zipf"), (3, 50, 77, 10, "uniform")])
@pytest.mark.parametrize("with_wpe", [False, True])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_presorted_embedding_pair_matches_the_plain_pair(ctx, B, T, V, C, dist, with_wpe, dtype):
    """agrad_gather_forward_sorted (gather and id ordering in one launch) +
    agrad_embedding_backward_sorted give the very bits of agrad_gather_forward +
    agrad_embedding_backward (+ agrad_pos_embedding_backward for the position
    table, whose sum rides in the sorted call's launch), call after call, both
    overwriting and accumulating; (5, 14000) takes the radix path and C = 10 the
    element-wise one."""
    import ctypes as Ct
    rng = _rng(60 + C)
    N = B * T
    if dist == "zipf":
        p = np.arange(1, V + 1, dtype=np.float64) ** -1.1
        ids = rng.choice(V, size=(B, T), p=p / p.sum()).astype(np.int32)
    else:
        ids = rng.integers(0, V, (B, T), dtype=np.int32)
    W = (0.02 * rng.standard_normal((V, C))).astype(np.float32)
    wpe = (0.02 * rng.standard_normal((T, C))).astype(np.float32) if with_wpe else None
    dY = rng.standard_normal((B, T, C)).astype(np.float32)
    if dtype == "bf16":
        W, dY = to_bf16_bits(W), to_bf16_bits(dY)
        wpe = to_bf16_bits(wpe) if wpe is not None else None
        dt = capi.BF16
    else:
        dt = capi.F32
    want_out = G.gather_forward(ctx, ids, W, wpe)
    want_dW = G.embedding_backward(ctx, ids, dY, V)
    d_dwpe = want_dwpe = None
    if with_wpe:
        d_dwpe = ctx.zeros((T, C), W.dtype)
        plain = ctx.zeros((T, C), W.dtype)
        d_plain_dY = ctx.upload(dY)
        # expected: one overwriting call, then two accumulating ones, as below
        for flag in (0, capi.ACC_PARAM_GRAD, capi.ACC_PARAM_GRAD):
            ctx.call("agrad_pos_embedding_backward", dt, Ct.c_void_p(d_plain_dY.ptr), Ct.c_void_p(plain.ptr), B, T, C,
                     flag)
        ctx.synchronize()
        want_dwpe = plain.download()
        plain.free()
        d_plain_dY.free()

    def vp(d):
        return Ct.c_void_p(d.ptr) if d is not None else None
    d_ids, d_W, d_dY = ctx.upload(ids), ctx.upload(W), ctx.upload(dY)
    d_wpe = ctx.upload(wpe) if wpe is not None else None
    out = ctx.empty((N, C), W.dtype)
    order = ctx.empty((6 * N + 128,), np.uint32)
    sws_b = ctx.lib.agrad_embedding_sort_workspace_bytes(N, V)
    bws_b = ctx.lib.agrad_embedding_backward_sorted_workspace_bytes(N, C)
    sws, bws = ctx.empty((sws_b,), np.uint8), ctx.empty((bws_b,), np.uint8)
    for rep in range(3):
        dW = ctx.zeros((V, C), W.dtype)
        ctx.call("agrad_gather_forward_sorted", dt, vp(d_ids), vp(d_W), vp(d_wpe), vp(out), N, T, C, V,
                 vp(order), vp(sws), sws_b)
        # the sort scratch is free once the forward call's work is queued: scribble over it
        ctx.call("agrad_fill", sws.ptr, 0, 0xFFFFFFFF, 4, sws_b // 4)
        ctx.call("agrad_embedding_backward_sorted", dt, vp(order), vp(d_dY), vp(dW), vp(d_dwpe), vp(bws), bws_b, N, T,
                 C, V, capi.ACC_PARAM_GRAD | (capi.ACC_PARAM_GRAD2 if rep else 0))
        ctx.synchronize()
        np.testing.assert_array_equal(out.download().reshape(B, T, C), want_out)
        np.testing.assert_array_equal(dW.download(), want_dW)
        got = order.download()
        rows, toks = _check_order(got, N, ids.reshape(-1), V)
        # each token's rows are adjacent and ascending
        d_tok = np.diff(toks.astype(np.int64))
        assert len(np.unique(toks)) == int((d_tok != 0).sum()) + 1
        assert (np.diff(rows.astype(np.int64))[d_tok == 0] > 0).all()
        dW.free()
    if with_wpe:
        np.testing.assert_array_equal(d_dwpe.download(), want_dwpe)
    for d in (d_ids, d_W, d_dY, d_wpe, d_dwpe, out, order, sws, bws):
        if d is not None:
            d.free()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("B,T,V,C,dist", [(32, 512, 32768, 384, "uniform"), (2, 700, 300, 48, "zipf"),
                                          (5, 14000, 3000, 32, "zipf"), (3, 50, 77, 10, "uniform")])
def test_table_gradient_cleared_by_rows(ctx, dtype, B, T, V, C, dist):
    """agrad_gather_forward_sorted_kept is the sorted forward call and leaves a copy of its ids;
    after the backward call of that order agrad_embedding_grad_reset with the copy brings the
    gradient table back to all zero, touching nothing outside the listed rows (the rows of other
    ids and the guard rows around the table keep their values).  (5, 14000) takes the forward
    call's two-launch path, C = 10 the reset's scalar kernel; ids outside the table are skipped."""
    import ctypes as Ct
    rng = _rng(170 + C)
    N = B * T
    dt = capi.BF16 if dtype == "bf16" else capi.F32
    if dist == "zipf":
        p = np.arange(1, V + 1, dtype=np.float64) ** -1.1
        ids = rng.choice(V, size=(B, T), p=p / p.sum()).astype(np.int32)
    else:
        ids = rng.integers(0, V, (B, T), dtype=np.int32)
    up = (lambda a: ctx.upload(to_bf16_bits(a))) if dtype == "bf16" else ctx.upload
    np_t = np.uint16 if dtype == "bf16" else np.float32
    W = (0.02 * rng.standard_normal((V, C))).astype(np.float32)
    dY = rng.standard_normal((B, T, C)).astype(np.float32)

    def vp(d, off=0):
        return Ct.c_void_p(d.ptr + off) if d is not None else None
    d_ids, d_W, d_dY = ctx.upload(ids), up(W), up(dY)
    out_a, out_b = ctx.empty((N, C), np_t), ctx.empty((N, C), np_t)
    order_a, order_b = ctx.empty((6 * N + 128,), np.uint32), ctx.empty((6 * N + 128,), np.uint32)
    kept = ctx.upload(np.full(N + 2, -5, np.int32))          # one guard word either side
    sws_b = ctx.lib.agrad_embedding_sort_workspace_bytes(N, V)
    bws_b = ctx.lib.agrad_embedding_backward_sorted_workspace_bytes(N, C)
    sws, bws = ctx.empty((sws_b,), np.uint8), ctx.empty((bws_b,), np.uint8)
    ctx.call("agrad_gather_forward_sorted", dt, vp(d_ids), vp(d_W), None, vp(out_a), N, T, C, V, vp(order_a), vp(sws), sws_b)
    ctx.call("agrad_gather_forward_sorted_kept", dt, vp(d_ids), vp(d_W), None, vp(out_b), N, T, C, V, vp(order_b), vp(sws),
             sws_b, vp(kept, 4))
    ctx.synchronize()
    np.testing.assert_array_equal(out_b.download(), out_a.download())
    info_at = (N + 3) & ~3
    used = info_at + 4 * N + (N // 128 + 1) * 32 + (N // 2048 + 1) * 32
    wa, wb = order_a.download(), order_b.download()
    np.testing.assert_array_equal(np.concatenate([wb[:N], wb[info_at:used]]), np.concatenate([wa[:N], wa[info_at:used]]))
    got_kept = kept.download()
    np.testing.assert_array_equal(got_kept[1:-1], ids.reshape(-1))
    assert got_kept[0] == -5 and got_kept[-1] == -5
    # a table of sevens between two guard rows: the backward call stores the rows of the ids
    e = 2 if dtype == "bf16" else 4
    seven = np.full((V + 2, C), 7.0, np.float32)
    dW = up(seven)
    seven_bits = dW.download().copy()
    ctx.call("agrad_embedding_backward_sorted", dt, vp(order_b), vp(d_dY), vp(dW, C * e), None, vp(bws), bws_b, N, T, C, V, 0)
    ctx.call("agrad_embedding_grad_reset", dt, vp(kept, 4), N, vp(dW, C * e), C, V)
    ctx.synchronize()
    table = dW.download().reshape(V + 2, C)
    present = np.zeros(V + 2, bool)
    present[ids.reshape(-1) + 1] = True
    assert not table[present].any()
    np.testing.assert_array_equal(table[~present], seven_bits.reshape(V + 2, C)[~present])
    # ids outside the table name no row
    bad = ids.reshape(-1).copy()
    bad[::3] = V + 5
    bad[1::7] = -1
    d_bad = ctx.upload(bad)
    dW2 = up(seven)
    ctx.call("agrad_embedding_grad_reset", dt, vp(d_bad), N, vp(dW2, C * e), C, V)
    ctx.synchronize()
    table = dW2.download().reshape(V + 2, C)
    ok = bad[(bad >= 0) & (bad < V)]
    present = np.zeros(V + 2, bool)
    present[ok + 1] = True
    assert not table[present].any()
    np.testing.assert_array_equal(table[~present], seven_bits.reshape(V + 2, C)[~present])
    # the copy may not be the ids' own buffer
    with pytest.raises(capi.AgradError):
        ctx.call("agrad_gather_forward_sorted_kept", dt, vp(d_ids), vp(d_W), None, vp(out_b), N, T, C, V, vp(order_b),
                 vp(sws), sws_b, vp(d_ids))
    for d in (d_ids, d_W, d_dY, out_a, out_b, order_a, order_b, kept, sws, bws, dW, dW2, d_bad):
        d.free()


@pytest.mark.parametrize("B,T,V,C,dist", [(32, 512, 32768, 384, "uniform"), (2, 700, 300, 48, "zipf"),
                                          (5, 14000, 3000, 32, "zipf"), (3, 50, 77, 10, "uniform")])
def test_ordering_with_the_zero_fill_matches_the_forward_call(ctx, B, T, V, C, dist):
    """agrad_embedding_order writes the order buffer agrad_gather_forward_sorted writes, word for
    word, and clears the gradient table in the same launch; the plain gather plus the sorted
    backward call then give the bits of the plain pair.  (5, 14000) takes the radix path with a
    fill of its own, C = 10 a fill whose size is no multiple of 16."""
    import ctypes as Ct
    rng = _rng(160 + C)
    N = B * T
    if dist == "zipf":
        p = np.arange(1, V + 1, dtype=np.float64) ** -1.1
        ids = rng.choice(V, size=(B, T), p=p / p.sum()).astype(np.int32)
    else:
        ids = rng.integers(0, V, (B, T), dtype=np.int32)
    W = (0.02 * rng.standard_normal((V, C))).astype(np.float32)
    dY = rng.standard_normal((B, T, C)).astype(np.float32)
    want_out = G.gather_forward(ctx, ids, W, None)
    want_dW = G.embedding_backward(ctx, ids, dY, V)

    def vp(d, off=0):
        return Ct.c_void_p(d.ptr + off) if d is not None else None
    d_ids, d_W, d_dY = ctx.upload(ids), ctx.upload(W), ctx.upload(dY)
    out = ctx.empty((N, C), np.float32)
    order_a, order_b = ctx.empty((6 * N + 128,), np.uint32), ctx.empty((6 * N + 128,), np.uint32)
    sws_b = ctx.lib.agrad_embedding_sort_workspace_bytes(N, V)
    bws_b = ctx.lib.agrad_embedding_backward_sorted_workspace_bytes(N, C)
    sws, bws = ctx.empty((sws_b,), np.uint8), ctx.empty((bws_b,), np.uint8)
    ctx.call("agrad_gather_forward_sorted", capi.F32, vp(d_ids), vp(d_W), None, vp(out), N, T, C, V, vp(order_a), vp(sws), sws_b)
    ctx.synchronize()
    # words of the buffer that an ordering writes: rows, four words of run info per row, arrival counters
    info_at = (N + 3) & ~3                  # (words N .. info_at are padding nobody writes)
    used = info_at + 4 * N + (N // 128 + 1) * 32 + (N // 2048 + 1) * 32

    def written(order):
        words = order.download()
        return np.concatenate([words[:N], words[info_at:used]])
    # the gradient table sits between two guard rows that must survive the fill
    dW = ctx.upload(np.full((V + 2, C), 7.0, np.float32))
    ctx.call("agrad_embedding_order", vp(d_ids), N, V, vp(order_b), vp(sws), sws_b, vp(dW, C * 4), V * C * 4)
    ctx.call("agrad_gather_forward", capi.F32, vp(d_ids), vp(d_W), None, vp(out), N, T, C, V)
    ctx.synchronize()
    np.testing.assert_array_equal(written(order_b), written(order_a))
    table = dW.download()
    assert not table[1:-1].any() and (table[0] == 7.0).all() and (table[-1] == 7.0).all()
    ctx.call("agrad_embedding_backward_sorted", capi.F32, vp(order_b), vp(d_dY), vp(dW, C * 4), None, vp(bws), bws_b, N, T,
             C, V, capi.ACC_PARAM_GRAD)
    ctx.synchronize()
    np.testing.assert_array_equal(out.download().reshape(B, T, C), want_out)
    np.testing.assert_array_equal(dW.download()[1:-1], want_dW)
    # without a table to clear it is the ordering alone
    ctx.call("agrad_fill", order_b.ptr, 0, 0xFFFFFFFF, 4, 6 * N + 128)
    ctx.call("agrad_embedding_order", vp(d_ids), N, V, vp(order_b), vp(sws), sws_b, None, 0)
    ctx.synchronize()
    np.testing.assert_array_equal(written(order_b), written(order_a))
    for d in (d_ids, d_W, d_dY, out, order_a, order_b, sws, bws, dW):
        d.free()


def _check_order(order, N, tokens, V):
    """The order buffer of the pre-sorted embedding pair: rows[N] (each token's rows adjacent
    and ascending; the top bit of a word marks a task of the gradient kernel: the first row
    of a run of 2 to 127 rows, or the first row of a 64-row chunk of a longer run, whose last
    chunk takes the rest; the bit below marks the tasks of more than 10 rows), then, from the next multiple of four words, four words for every
    row: its token, where its token's run starts, and (R, x): R = 0 for a later row of a run
    of up to 127 rows and for an id outside the table; the run's length for the first row of
    such a run, with x = the run's second row (or 0xFFFFFFFF: not given); for a longer run
    its length and x = the row's index in it.  Then the gradient kernel's arrival counters,
    all zero.  Returns the rows and their tokens."""
    rows = (order[:N] & 0x3FFFFFFF).astype(np.int64)
    marked = (order[:N] >> 31).astype(bool)
    marked_big = ((order[:N] >> 30) & 1).astype(bool)
    at = (N + 3) // 4 * 4
    info = order[at:at + 4 * N].reshape(N, 4).astype(np.int64)
    tickets = order[at + 4 * N:at + 4 * N + (N // 128 + 1) * 32 + (N // 2048 + 1) * 32]
    assert not tickets.any()
    np.testing.assert_array_equal(np.sort(rows), np.arange(N))
    toks = tokens[rows].astype(np.int64)
    run = np.bincount(tokens, minlength=int(tokens.max()) + 1)[toks]
    change = np.flatnonzero(np.diff(toks) != 0) + 1
    starts = np.concatenate([[0], change])
    start = np.repeat(starts, np.diff(np.concatenate([starts, [N]])))
    j = np.arange(N) - start
    tok, got_start, R, x = (info[rows, k] for k in range(4))
    np.testing.assert_array_equal(tok, toks)
    np.testing.assert_array_equal(got_start, start)
    valid = toks < V
    short = valid & (run <= 127)
    np.testing.assert_array_equal(R[~valid], 0)
    np.testing.assert_array_equal(R[short], np.where(j == 0, run, 0)[short])
    second = short & (j == 0) & (run >= 2)
    given = second & (x != 0xFFFFFFFF)
    np.testing.assert_array_equal(x[given], rows[np.flatnonzero(given) + 1])
    np.testing.assert_array_equal(x[short & (j == 0) & (run == 1)], 0xFFFFFFFF)
    np.testing.assert_array_equal(R[valid & ~short], run[valid & ~short])
    np.testing.assert_array_equal(x[valid & ~short], j[valid & ~short])
    chunk_head = valid & ~short & (j % 64 == 0) & (j // 64 < run // 64)
    np.testing.assert_array_equal(marked, second | chunk_head)
    np.testing.assert_array_equal(marked_big, (second & (run > 10)) | chunk_head)
    return rows, toks


def _same_group_tokens(V, how_many, N):
    """tokens below V that the grouping sort hands to one workgroup (its hash: the log2g
    bits below bit 24 of (token mod 2^24) * 0x9E3779; 128, 256 or 512 groups by the number
    of rows)"""
    log2g = 9 if N > 32768 else 8 if N > 16384 else 7 if N > 1024 else 4
    toks = np.arange(V, dtype=np.uint64)
    prod = ((toks & np.uint64(0xFFFFFF)) * np.uint64(0x9E3779)) & np.uint64(0xFFFFFFFF)
    group = (prod >> np.uint64(24 - log2g)) & np.uint64((1 << log2g) - 1)
    best = np.bincount(group.astype(np.int64)).argmax()
    found = toks[group == best][:how_many].astype(np.int32)
    assert len(found) == how_many
    return found


_SKEWED = {
    # name: (N, [(rows of a token, how many such tokens)...] all within one hash group, rest of N uniform:
    # about 125 more pairs in the group at 16384 rows, 64 at 8192)
    "all_rows_one_token": (16384, [(16384, 1)]),
    "padding_third": (16384, [(5500, 1)]),                    # ids read again; dense map: two words a wave and step
    "two_tokens_split": (16384, [(8192, 2)]),                 # what is left after the frequent one exceeds LDS
    "frequent_plus_few": (16384, [(5000, 1), (2, 50)]),       # ids read again, the rest (under 257 pairs) placed by rank
    "frequent_plus_some": (16384, [(5000, 1), (3, 100)]),     # ids read again, the rest (257 .. 3072) through the network
    "frequent_plus_many": (16384, [(5000, 1), (20, 100)]),    # ids read again, the rest through the network
    "listed_frequent_plus_few": (8192, [(1500, 1), (2, 60)]),    # list fits LDS, the rest moves over and is placed by rank
    "listed_frequent_plus_some": (8192, [(1500, 1), (2, 150)]),  # list fits LDS, the rest (257 .. 512) through the network
    "listed_no_frequent": (8192, [(400, 3)]),                 # list fits LDS, no single frequent token
    "list_of_300_pairs": (16384, [(200, 1)]),                 # 257 .. 512 pairs: the frequent-token way, a sparse map
    "medium_token": (16384, [(900, 1)]),                      # a sparse map: each lane walks the marks of its own word
    "frequent_in_one_stretch": (16384, [(2048, 1)]),          # its rows are rows 0 .. 2047: one wave's words dense, the others' empty
    "short_input": (1500, [(1400, 1)]),                       # fewer rows than the row map has bits
    "most_rows_one_token_64k": (65536, [(60000, 1)]),         # 512 groups, every word of the row map
    "padding_40k": (40001, [(15000, 1), (3, 40)]),            # 512 groups, a ragged last word
    "padding_20k": (20001, [(7000, 1), (3, 80)]),             # 256 groups
    "two_frequent_one_group_64k": (65536, [(9000, 1), (1500, 1), (2, 50)]),     # a sparse map of 2048 words
    "bad_ids_frequent": (4096, [(0, 1)]),                     # out-of-range ids (one sentinel token) dominate
}


@pytest.mark.parametrize("case", sorted(_SKEWED))
def test_id_ordering_with_frequent_tokens(ctx, case):
    """The one-launch ordering on skewed ids: one token holding most rows (its rows
    go through a bit map instead of the sorting network), several such tokens in
    one hash group, and the fall-backs behind them.  Checked on the order itself
    (each token's rows adjacent and ascending, every row once) and on the
    gradient built from it, bit for bit against the atomic-free plain call."""
    import ctypes as Ct
    N, spec = _SKEWED[case]
    V, C = 30000, 64
    rng = _rng(zlib.crc32(case.encode()) % 1000)
    ids = rng.integers(0, V, N, dtype=np.int32)
    if case == "bad_ids_frequent":
        ids[rng.permutation(N)[:3000]] = -5
    else:
        same = _same_group_tokens(V, sum(k for _, k in spec), N)
        slots = np.arange(N) if case == "frequent_in_one_stretch" else rng.permutation(N)
        at = t = 0
        for rows, k in spec:
            for _ in range(k):
                ids[slots[at:at + rows]] = same[t]
                at += rows
                t += 1
    dY = rng.standard_normal((N, C)).astype(np.float32)
    W = np.zeros((V, C), np.float32)

    def vp(d):
        return Ct.c_void_p(d.ptr)
    d_ids, d_W, d_dY = ctx.upload(ids), ctx.upload(W), ctx.upload(dY)
    out = ctx.empty((N, C), np.float32)
    order = ctx.empty((6 * N + 128,), np.uint32)
    sws_b = ctx.lib.agrad_embedding_sort_workspace_bytes(N, V)
    bws_b = ctx.lib.agrad_embedding_backward_sorted_workspace_bytes(N, C)
    sws, bws = ctx.empty((sws_b,), np.uint8), ctx.empty((bws_b,), np.uint8)
    valid = (ids >= 0) & (ids < V)
    want_dW = np.zeros((V, C), np.float32)
    if case != "bad_ids_frequent":
        want_dW = G.embedding_backward(ctx, ids.reshape(1, N), dY.reshape(1, N, C), V)
    for rep in range(2):
        dW = ctx.zeros((V, C), np.float32)
        ctx.call("agrad_gather_forward_sorted", capi.F32, vp(d_ids), vp(d_W), None, vp(out), N, 1, C, V,
                 vp(order), vp(sws), sws_b)
        if case == "bad_ids_frequent":
            with pytest.raises(IndexError):
                ctx.synchronize()
        ctx.synchronize()
        got = order.download()
        rows, toks = _check_order(got, N, np.where(valid, ids, V), V)
        d_tok = np.diff(toks.astype(np.int64))
        assert len(np.unique(toks)) == int((d_tok != 0).sum()) + 1
        assert (np.diff(rows.astype(np.int64))[d_tok == 0] > 0).all()
        if case != "bad_ids_frequent":
            ctx.call("agrad_embedding_backward_sorted", capi.F32, vp(order), vp(d_dY), vp(dW), None, vp(bws), bws_b,
                     N, 1, C, V, 0)
            ctx.synchronize()
            np.testing.assert_array_equal(dW.download(), want_dW)
        dW.free()
    for d in (d_ids, d_W, d_dY, out, order, sws, bws):
        d.free()


@pytest.mark.parametrize("B,T,V,C,dist", [(4, 128, 500, 64, "uniform"), (2, 700, 90, 50, "zipf"), (8, 512, 4000, 384, "zipf"),
                                          (3, 23000, 3000, 32, "zipf"), (2, 21000, 3000, 1024, "zipf")])
def test_embedding_gradient_stored_as_bf16_under_an_fp32_upstream(ctx, B, T, V, C, dist):
    """AGRAD_PARAM_GRAD_BF16 (gather_backward_bf16_kernel, metal_ops.metal:12395-12446): dY is
    fp32, dW and dwpe are bf16.  A row's sum is finished in fp32, added to the stored bf16
    value (when accumulating) and rounded once: compared with that computation on the CPU
    row sums to one bf16 ulp (the fp32 sums may associate differently across chunk edges);
    rows without a token keep their bits.  Through the plain and the pre-sorted call."""
    import ctypes as Ct
    rng = _rng(70 + C)
    N = B * T
    ids = (_zipf_ids(rng, N, V) if dist == "zipf" else rng.integers(0, V, size=N, dtype=np.int32)).reshape(B, T)
    dY = rng.standard_normal((B, T, C)).astype(np.float32)
    old_w = to_bf16_bits((0.5 * rng.standard_normal((V, C))).astype(np.float32))
    old_p = to_bf16_bits((0.5 * rng.standard_normal((T, C))).astype(np.float32))
    rows = _sums_in_row_order(ids.reshape(-1), dY.reshape(N, C), V)      # np.add.at's sums (the last case: row waves of
    pos = dY.astype(np.float64).sum(0)                                   # several column blocks, every run a task)
    touched = np.zeros(V, bool)
    touched[ids.reshape(-1)] = True

    def vp(d):
        return Ct.c_void_p(d.ptr) if d is not None else None

    def check(got_bits, sums, old_bits, accumulate, what, only=None):
        want = (from_bf16_bits(old_bits).astype(np.float64) if accumulate else 0.0) + sums.astype(np.float64)
        got = from_bf16_bits(got_bits).astype(np.float64)
        ulp = np.maximum(np.abs(want), 1e-30) * 2.0 ** -7            # one bf16 ulp is at most 2^-7 of the value
        bound = ulp + 1e-5 * np.sqrt(N / V + 1)                       # plus the fp32 sums' own re-association noise
        bad = np.abs(got - want) > bound
        if only is not None:
            bad &= only[:, None]
        assert not bad.any(), (what, int(bad.sum()), float(np.abs(got - want).max()))

    d_ids, d_dY = ctx.upload(ids), ctx.upload(dY)
    ws_b = ctx.lib.agrad_embedding_backward_workspace_bytes(N, C, V, capi.F32)
    ws = ctx.empty((ws_b,), np.uint8)
    for accumulate in (False, True):
        dW = ctx.upload(old_w)
        ctx.call("agrad_embedding_backward", capi.F32, vp(d_ids), vp(d_dY), vp(dW), vp(ws), ws_b, N, C, V,
                 capi.PARAM_GRAD_BF16 | (capi.ACC_PARAM_GRAD if accumulate else 0))
        ctx.synchronize()
        got = dW.download()
        check(got, rows, old_w, accumulate, f"plain call, accumulate={accumulate}", touched)
        np.testing.assert_array_equal(got[~touched], old_w[~touched])
        dW.free()
    # pre-sorted pair with the position table in the same launch
    d_W = ctx.upload(np.zeros((V, C), np.float32))
    out = ctx.empty((N, C), np.float32)
    order = ctx.empty((6 * N + 128,), np.uint32)
    sws_b = ctx.lib.agrad_embedding_sort_workspace_bytes(N, V)
    bws_b = ctx.lib.agrad_embedding_backward_sorted_workspace_bytes(N, C)
    sws, bws = ctx.empty((sws_b,), np.uint8), ctx.empty((bws_b,), np.uint8)
    ctx.call("agrad_gather_forward_sorted", capi.F32, vp(d_ids), vp(d_W), None, vp(out), N, T, C, V, vp(order), vp(sws), sws_b)
    for accumulate in (False, True):
        dW, dP = ctx.upload(old_w), ctx.upload(old_p)
        flags = capi.PARAM_GRAD_BF16 | ((capi.ACC_PARAM_GRAD | capi.ACC_PARAM_GRAD2) if accumulate else 0)
        ctx.call("agrad_embedding_backward_sorted", capi.F32, vp(order), vp(d_dY), vp(dW), vp(dP), vp(bws), bws_b, N, T, C, V, flags)
        ctx.synchronize()
        got = dW.download()
        check(got, rows, old_w, accumulate, f"sorted call, accumulate={accumulate}", touched)
        np.testing.assert_array_equal(got[~touched], old_w[~touched])
        check(dP.download(), pos, old_p, accumulate, f"position table, accumulate={accumulate}")
        dW.free()
        dP.free()
    with pytest.raises(capi.AgradError):      # the narrow store goes with an fp32 upstream only
        dW = ctx.upload(old_w)
        ctx.call("agrad_embedding_backward", capi.BF16, vp(d_ids), vp(d_dY), vp(dW), vp(ws), ws_b, N, C, V, capi.PARAM_GRAD_BF16)
    for d in (d_ids, d_dY, ws, d_W, out, order, sws, bws):
        d.free()


@pytest.mark.parametrize("kind", [capi.NORM_LAYER, capi.NORM_RMS])
@pytest.mark.parametrize("rows,Cw", [(37, 96), (2048, 384), (500, 1536)])
@pytest.mark.parametrize("io", ["f32", "bf16"])
def test_norm_parameter_gradients_stored_as_bf16(ctx, kind, rows, Cw, io):
    """AGRAD_PARAM_GRAD_BF16 on the norm backward: dgamma / dbeta point at bf16 (the bf16
    option of rmsnorm_weighted_dgamma, gqa_rms_dgamma_bf16).  The stored value is the fp32
    call's sum (plus the stored bf16 value when accumulating) rounded once: the two calls
    share the partial sums, so the comparison is exact."""
    rng = _rng(90 + Cw)
    x = rng.standard_normal((rows, Cw)).astype(np.float32)
    dy = rng.standard_normal((rows, Cw)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(Cw)).astype(np.float32)
    if io == "bf16":
        x, dy = to_bf16_bits(x), to_bf16_bits(dy)
    want_beta = kind == capi.NORM_LAYER
    wide = G.norm_backward(ctx, kind, x, gamma, dy, 1e-5, want_dbeta=want_beta)
    old_g = to_bf16_bits(rng.standard_normal(Cw).astype(np.float32))
    old_b = to_bf16_bits(rng.standard_normal(Cw).astype(np.float32))
    for accumulate in (False, True):
        flags = capi.PARAM_GRAD_BF16 | (capi.ACC_PARAM_GRAD if accumulate else 0)
        got = G.norm_backward(ctx, kind, x, gamma, dy, 1e-5, want_dbeta=want_beta, dgamma_init=old_g,
                              dbeta_init=old_b if want_beta else None, flags=flags)
        np.testing.assert_array_equal(got["dx"], wide["dx"])
        for name, old in (("dgamma", old_g), ("dbeta", old_b)):
            if wide[name] is None:
                continue
            base = from_bf16_bits(old) if accumulate else np.zeros(Cw, np.float32)
            np.testing.assert_array_equal(got[name], to_bf16_bits(base + wide[name]), err_msg=f"{name} accumulate={accumulate}")


@pytest.mark.parametrize("lead,inner", [(16, 384), (64, 130), (65, 384), (3000, 96), (16384, 768), (5, 7)])
def test_bias_gradient_stored_as_bf16_under_an_fp32_upstream(ctx, lead, inner):
    """AGRAD_PARAM_GRAD_BF16 on the broadcast-add gradient (bias_grad_reduce_bf16): the column
    sum of fp32 rows lands in a bf16 vector -- the fp32 call's sum (plus the stored bf16
    value when accumulating) rounded once; few rows take the direct kernel, many the two
    stages.  Also through agrad_pos_embedding_backward."""
    import ctypes as Ct
    rng = _rng(95 + inner)
    g = rng.standard_normal((lead, inner)).astype(np.float32)
    old = to_bf16_bits(rng.standard_normal(inner).astype(np.float32))

    def vp(d):
        return Ct.c_void_p(d.ptr) if d is not None else None
    d_g = ctx.upload(g)
    ws_b = ctx.lib.agrad_broadcast_grad_workspace_bytes(lead, inner)
    ws = ctx.empty((max(ws_b, 1),), np.uint8)
    wide = ctx.zeros((inner,), np.float32)
    ctx.call("agrad_broadcast_add_backward", capi.F32, vp(d_g), vp(wide), vp(ws) if ws_b else None, ws_b, lead, inner, 0)
    ctx.synchronize()
    sums = wide.download()
    assert_fp32_close(sums, g.astype(np.float64).sum(0).astype(np.float32), "fp32 column sum", rtol=1e-5,
                      atol=max(2e-6, 1e-4 * np.sqrt(lead / 14)))
    for accumulate in (False, True):
        for entry in ("agrad_broadcast_add_backward", "agrad_pos_embedding_backward"):
            if entry == "agrad_pos_embedding_backward" and lead > 64:
                continue                      # one thread per column walks the rows: the small-batch kernel
            narrow = ctx.upload(old)
            flags = capi.PARAM_GRAD_BF16 | (capi.ACC_PARAM_GRAD if accumulate else 0)
            if entry == "agrad_broadcast_add_backward":
                ctx.call(entry, capi.F32, vp(d_g), vp(narrow), vp(ws) if ws_b else None, ws_b, lead, inner, flags)
            else:
                ctx.call(entry, capi.F32, vp(d_g), vp(narrow), lead, 1, inner, flags)
            ctx.synchronize()
            base = from_bf16_bits(old) if accumulate else np.zeros(inner, np.float32)
            np.testing.assert_array_equal(narrow.download(), to_bf16_bits(base + sums), err_msg=f"{entry} accumulate={accumulate}")
            narrow.free()
    with pytest.raises(capi.AgradError):
        narrow = ctx.upload(old)
        ctx.call("agrad_broadcast_add_backward", capi.BF16, vp(d_g), vp(narrow), vp(ws) if ws_b else None, ws_b, lead, inner,
                 capi.PARAM_GRAD_BF16)
    for d in (d_g, ws, wide):
        d.free()
