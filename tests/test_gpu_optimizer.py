"""AdamW and the gradient-norm partial sums on the GPU against the CPU
restatement of cpu_adamw_step (backend.py:2013-2038), through the C ABI and
through Runtime + AdamW on the "hip" device.

Every operation of the update is a single IEEE fp32 operation on both sides
(no FMA contraction, correctly rounded divide and square root), so for the same
gradients the parameters and moments are compared bit for bit.
"""
import ctypes as C
import math

import numpy as np
import pytest

from autograd_amd import capi
from autograd_amd.op import GatherOp, GELUOp, LayerNormOp
from autograd_amd.optimizer import AdamW, get_lr_cosine_schedule
from autograd_amd.runtime import Runtime
from autograd_amd.tensor import Tensor
from oracle import cpu_ops as K
from tests.helpers import from_bf16_bits, to_bf16_bits

pytestmark = pytest.mark.gpu


def vp(d, off=0):
    return C.c_void_p(d.ptr + off)


def f32r(x):
    """the fp32 value numpy makes of a Python float"""
    return float(np.float32(x))


@pytest.mark.parametrize("n", [1, 3, 4, 1023, 4096, 100_003])
@pytest.mark.parametrize("wd", [0.0, 0.1])
def test_adamw_matches_cpu_bit_for_bit(ctx, n, wd):
    rng = np.random.default_rng(50 + n)
    lr, b1, b2, eps = 1e-3, 0.9, 0.999, 1e-8
    p = rng.standard_normal(n).astype(np.float32)
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    dp, dm, dv = ctx.upload(p), ctx.upload(m), ctx.upload(v)
    dg = ctx.empty((n,), np.float32)
    for t in range(1, 5):
        g = (rng.standard_normal(n) * 10.0 ** rng.integers(-6, 2, n)).astype(np.float32)
        lr_t = lr * math.sqrt(1.0 - b2 ** t) / (1.0 - b1 ** t)
        K.adamw_step(p, g, m, v, lr, lr_t, b1, b2, eps, wd)
        ctx.call("agrad_copy_from_host", dg.ptr, 0, g.ctypes.data_as(C.c_void_p), g.nbytes)
        ctx.call("agrad_adamw_step", capi.F32, vp(dp), vp(dg), vp(dm), vp(dv), n, n if wd else 0,
                 lr * wd, b1, 1.0 - b1, b2, 1.0 - b2, eps, lr_t, 1.0, 1.0)
        ctx.synchronize()
        np.testing.assert_array_equal(dm.download(), m, err_msg=f"m at step {t}")
        np.testing.assert_array_equal(dv.download(), v, err_msg=f"v at step {t}")
        np.testing.assert_array_equal(dp.download(), p, err_msg=f"p at step {t}")
    for d in (dp, dm, dv, dg):
        d.free()


@pytest.mark.parametrize("grad_dtype", ["f32", "bf16"])
def test_adamw_split_form_scale_and_decay_prefix(ctx, grad_dtype):
    """the Metal calling convention: lr / (1 - b1^t), 1 / sqrt(1 - b2^t), a clip
    coefficient, decay on a prefix of the slab; from an offset that is only
    4-byte aligned so that the element-wise kernel runs too"""
    rng = np.random.default_rng(61)
    n, dn, off = 10_007, 6_000, 3
    lr, b1, b2, eps, wd, scale = 3e-4, 0.9, 0.95, 1e-8, 0.05, 0.37
    p_all = rng.standard_normal(n + off).astype(np.float32)
    m_all = (0.1 * rng.standard_normal(n + off)).astype(np.float32)
    v_all = (0.01 * rng.standard_normal(n + off) ** 2).astype(np.float32)
    g = rng.standard_normal(n + off).astype(np.float32)
    if grad_dtype == "bf16":
        g_store = to_bf16_bits(g)
        g_seen = from_bf16_bits(g_store)
        dt, gsz = capi.BF16, 2
    else:
        g_store, g_seen, dt, gsz = g, g, capi.F32, 4
    for first in (0, off):
        p, m, v = p_all.copy(), m_all.copy(), v_all.copy()
        dp, dm, dv, dg = ctx.upload(p), ctx.upload(m), ctx.upload(v), ctx.upload(g_store)
        t = 3
        step_lr, inv = lr / (1.0 - b1 ** t), 1.0 / math.sqrt(1.0 - b2 ** t)
        K.adamw_step_split(p[first:first + n], g_seen[first:first + n], m[first:first + n], v[first:first + n],
                           lr * wd, b1, b2, eps, step_lr, inv, scale, dn)
        ctx.call("agrad_adamw_step", dt, vp(dp, 4 * first), vp(dg, gsz * first), vp(dm, 4 * first), vp(dv, 4 * first),
                 n, dn, lr * wd, b1, 1.0 - b1, b2, 1.0 - b2, eps, step_lr, inv, scale)
        ctx.synchronize()
        np.testing.assert_array_equal(dp.download(), p)     # includes the untouched elements around the slice
        np.testing.assert_array_equal(dm.download(), m)
        np.testing.assert_array_equal(dv.download(), v)
        for d in (dp, dm, dv, dg):
            d.free()


def test_adamw_argument_errors(ctx):
    d = ctx.upload(np.zeros(16, np.float32))
    with pytest.raises(capi.AgradError):
        ctx.call("agrad_adamw_step", capi.F32, vp(d), vp(d), vp(d), vp(d), 8, 9, 0.0, 0.9, 0.1, 0.99, 0.01, 1e-8, 1e-3, 1.0, 1.0)
    with pytest.raises(capi.AgradError):
        ctx.call("agrad_adamw_step", 5, vp(d), vp(d), vp(d), vp(d), 8, 0, 0.0, 0.9, 0.1, 0.99, 0.01, 1e-8, 1e-3, 1.0, 1.0)
    ctx.call("agrad_adamw_step", capi.F32, vp(d), vp(d), vp(d), vp(d), 0, 0, 0.0, 0.9, 0.1, 0.99, 0.01, 1e-8, 1e-3, 1.0, 1.0)
    ctx.synchronize()
    assert not d.download().any()
    d.free()


@pytest.mark.parametrize("n", [1, 255, 256, 257, 100_003])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_grad_norm_partials(ctx, n, dtype):
    rng = np.random.default_rng(70 + n)
    g = rng.standard_normal(n).astype(np.float32)
    if dtype == "bf16":
        store = to_bf16_bits(g)
        g = from_bf16_bits(store)
        dt = capi.BF16
    else:
        store, dt = g, capi.F32
    groups = ctx.lib.agrad_grad_norm_groups(n)
    assert groups == (n + 255) // 256
    dg = ctx.upload(store)
    part = ctx.upload(np.full(groups + 3, -1.0, np.float32))
    ctx.call("agrad_grad_norm_sq", dt, vp(dg), vp(part), n)
    ctx.synchronize()
    got = part.download()
    assert (got[groups:] == -1.0).all()
    want = K.grad_norm_partials(g)
    # 256 fp32 squares added in a fixed tree: a few ulp of the sum
    assert np.abs(got[:groups] - want).max() <= 2e-6 * max(1.0, want.max())
    total = math.sqrt(float(np.sum(got[:groups], dtype=np.float64)))
    assert abs(total - float(np.linalg.norm(g.astype(np.float64)))) <= 1e-6 * max(1.0, total)
    dg.free()
    part.free()


def test_cosine_schedule():
    assert get_lr_cosine_schedule(0, 100, 10, 1.0, 0.1) == pytest.approx(0.1)
    assert get_lr_cosine_schedule(9, 100, 10, 1.0, 0.1) == pytest.approx(1.0)
    assert get_lr_cosine_schedule(10, 100, 10, 1.0, 0.1) == pytest.approx(1.0)
    assert get_lr_cosine_schedule(55, 100, 10, 1.0, 0.1) == pytest.approx(0.55)
    assert get_lr_cosine_schedule(101, 100, 10, 1.0, 0.1) == 0.1


def test_adamw_over_the_runtime_slab():
    """Embedding -> LayerNorm -> GELU on the hip device, three optimizer steps.
    The runtime packs wte, gamma, beta into one slab (matrices first), so the
    optimizer issues ONE launch per step with decay on the matrix prefix; the
    expectation is the CPU kernel applied per parameter to the gradients the
    device produced."""
    rng = np.random.default_rng(80)
    B, T, C_, V = 2, 16, 64, 50
    ids_np = rng.integers(0, V, (B, T), dtype=np.int32)
    rt = Runtime(device="hip")
    ids = Tensor(shape=(B, T), dtype=np.int32, device="hip", requires_grad=False, init_val=ids_np, name="ids")
    wte = Tensor(shape=(V, C_), dtype=np.float32, device="hip", requires_grad=True,
                 init_val=(0.5 * rng.standard_normal((V, C_))).astype(np.float32), name="wte")
    gamma = Tensor(shape=(C_,), dtype=np.float32, device="hip", requires_grad=True,
                   init_val=(1 + 0.1 * rng.standard_normal(C_)).astype(np.float32), name="gamma")
    beta = Tensor(shape=(C_,), dtype=np.float32, device="hip", requires_grad=True,
                  init_val=(0.1 * rng.standard_normal(C_)).astype(np.float32), name="beta")
    out = GELUOp()(LayerNormOp(eps=1e-5)(GatherOp()(ids, wte), gamma, beta))
    rt.loss = out
    rt.build_topo(out)
    rt.bind_memory()
    lr, betas, eps, wd = 1e-2, (0.9, 0.95), 1e-8, 0.1
    opt = AdamW([wte, gamma, beta], lr=lr, betas=betas, eps=eps, weight_decay=wd, runtime=rt)
    assert len(opt.dispatches) == 1, "parameters of one slab take one launch"
    assert opt.dispatches[0][5] == V * C_, "weight decay covers exactly the matrix prefix"
    clip = opt.build_grad_clip()
    params = {"wte": wte, "gamma": gamma, "beta": beta}
    host = {k: rt.backend.copy_to_host(t).copy() for k, t in params.items()}
    mom = {k: (np.zeros_like(a), np.zeros_like(a)) for k, a in host.items()}
    upstream = rng.standard_normal((B, T, C_)).astype(np.float32)
    for t in range(1, 4):
        rt.forward()
        rt.zero_grad()
        rt.backend.copy_from_host(out.grad, upstream)
        rt.backward_graph()
        rt.backend.synchronize()
        grads = {k: rt.backend.copy_to_host(p.grad).copy() for k, p in params.items()}
        norm, coef = clip(1.0)
        want_norm = math.sqrt(sum(float(np.sum(g.astype(np.float64) ** 2)) for g in grads.values()))
        assert norm == pytest.approx(want_norm, rel=1e-6)
        assert coef == pytest.approx(min(1.0, 1.0 / (want_norm + 1e-6)), rel=1e-6)
        opt.step(grad_scale=coef)
        lr_t = lr * math.sqrt(1.0 - betas[1] ** t) / (1.0 - betas[0] ** t)
        for k in params:
            m, v = mom[k]
            K.adamw_step_split(host[k].reshape(-1), grads[k].reshape(-1), m.reshape(-1), v.reshape(-1),
                               lr * wd if params[k].ndim > 1 else 0.0, betas[0], betas[1], eps, lr_t, 1.0, coef)
            np.testing.assert_array_equal(rt.backend.copy_to_host(params[k]), host[k], err_msg=f"{k} at step {t}")
    opt.release()
    rt.release()


# -- AdamW with 8-bit moments ---------------------------------------------------------
@pytest.mark.parametrize("n,decay_n", [(1, 0), (3, 3), (255, 100), (256, 256), (257, 0), (4096, 4096), (5000, 2500),
                                       (100_003, 70_001), (1 << 20, 1 << 19)])
@pytest.mark.parametrize("grad_dtype", ["f32", "bf16"])
def test_adamw8bit_matches_the_restatement_bit_for_bit(ctx, n, decay_n, grad_dtype):
    """agrad_adamw8bit_step against oracle.cpu_ops.adamw8bit_step (the restatement of
    adamw8bit_step, metal_ops.metal:10229-10361) over four steps: parameters, both code
    arrays and both scale arrays must be identical -- every operation is one IEEE fp32
    operation on both sides and the code search is integer work.  Sizes straddle the
    4-element vectors and the 256-element blocks; weight decay stops inside a block."""
    rng = np.random.default_rng(77 + n)
    lr, b1, b2, eps, wd = 2e-3, 0.9, 0.95, 1e-8, 0.1
    qm_map, qv_map = K.dynamic_map(True), K.dynamic_map(False)
    p = rng.standard_normal(n).astype(np.float32)
    blocks = (n + 255) // 256
    qm, qv = np.zeros(n, np.uint8), np.zeros(n, np.uint8)
    am, av = np.zeros(blocks, np.float32), np.zeros(blocks, np.float32)
    dt = capi.BF16 if grad_dtype == "bf16" else capi.F32
    d_p = ctx.upload(p)
    d_qm, d_qv = ctx.upload(np.full(n, 0xAB, np.uint8)), ctx.upload(np.full(n, 0xCD, np.uint8))   # garbage: step 1 must not read it
    d_am, d_av = ctx.upload(np.full(blocks, np.nan, np.float32)), ctx.upload(np.full(blocks, np.nan, np.float32))
    d_mapm, d_mapv = ctx.upload(qm_map), ctx.upload(qv_map)
    for t in range(1, 5):
        g = (rng.standard_normal(n) * (10.0 ** rng.uniform(-3, 0, n))).astype(np.float32)   # magnitudes over three decades
        if t == 3:
            g[::7] = 0.0
        if grad_dtype == "bf16":
            bits = to_bf16_bits(g)
            g_seen, d_g = from_bf16_bits(bits), ctx.upload(bits)
        else:
            g_seen, d_g = g, ctx.upload(g)
        lr_bc1 = lr / (1.0 - b1 ** t)
        inv_sqrt_bc2 = 1.0 / math.sqrt(1.0 - b2 ** t)
        clip = 1.0 if t != 2 else 0.37
        K.adamw8bit_step(p, g_seen, qm, qv, am, av, qm_map, qv_map, 1.0 - lr * wd, lr_bc1, b1, b2, eps, decay_n, t == 1,
                         inv_sqrt_bc2, clip_coef=clip)
        ctx.call("agrad_adamw8bit_step", dt, vp(d_p), vp(d_g), vp(d_qm), vp(d_qv), vp(d_am), vp(d_av), vp(d_mapm),
                 vp(d_mapv), n, decay_n, 1.0 - lr * wd, lr_bc1, b1, b2, eps, inv_sqrt_bc2, clip, int(t == 1))
        ctx.synchronize()
        np.testing.assert_array_equal(d_am.download(), am, err_msg=f"absmax_m, step {t}")
        np.testing.assert_array_equal(d_av.download(), av, err_msg=f"absmax_v, step {t}")
        np.testing.assert_array_equal(d_qm.download(), qm, err_msg=f"qm, step {t}")
        np.testing.assert_array_equal(d_qv.download(), qv, err_msg=f"qv, step {t}")
        np.testing.assert_array_equal(d_p.download(), p, err_msg=f"p, step {t}")
        d_g.free()
    for d in (d_p, d_qm, d_qv, d_am, d_av, d_mapm, d_mapv):
        d.free()


def test_adamw8bit_unaligned_slices_and_argument_errors(ctx):
    """a slice of a slab that starts at an odd element (no 16-byte alignment: the
    element-wise path) gives the same bits as the aligned call"""
    rng = np.random.default_rng(99)
    n, off = 1500, 3
    qm_map, qv_map = K.dynamic_map(True), K.dynamic_map(False)
    p = rng.standard_normal(n + off).astype(np.float32)
    g = rng.standard_normal(n + off).astype(np.float32)
    qm, qv = np.zeros(n, np.uint8), np.zeros(n, np.uint8)
    am, av = np.zeros(6, np.float32), np.zeros(6, np.float32)
    d_p, d_g = ctx.upload(p), ctx.upload(g)
    d_qm, d_qv = ctx.zeros((n + off,), np.uint8), ctx.zeros((n + off,), np.uint8)
    d_am, d_av = ctx.zeros((6,), np.float32), ctx.zeros((6,), np.float32)
    d_mapm, d_mapv = ctx.upload(qm_map), ctx.upload(qv_map)
    want = p.copy()
    K.adamw8bit_step(want[off:], g[off:], qm, qv, am, av, qm_map, qv_map, 0.999, 1e-2, 0.9, 0.99, 1e-8, n, True, 3.0)
    ctx.call("agrad_adamw8bit_step", capi.F32, vp(d_p, 4 * off), vp(d_g, 4 * off), vp(d_qm, off), vp(d_qv, off), vp(d_am),
             vp(d_av), vp(d_mapm), vp(d_mapv), n, n, 0.999, 1e-2, 0.9, 0.99, 1e-8, 3.0, 1.0, 1)
    ctx.synchronize()
    np.testing.assert_array_equal(d_p.download(), want)
    np.testing.assert_array_equal(d_qm.download()[off:], qm)
    np.testing.assert_array_equal(d_qv.download()[off:], qv)
    np.testing.assert_array_equal(d_am.download(), am)
    assert (d_qm.download()[:off] == 0).all()
    with pytest.raises(capi.AgradError):      # decay_numel beyond numel
        ctx.call("agrad_adamw8bit_step", capi.F32, vp(d_p), vp(d_g), vp(d_qm), vp(d_qv), vp(d_am), vp(d_av), vp(d_mapm),
                 vp(d_mapv), 8, 9, 1.0, 1e-3, 0.9, 0.99, 1e-8, 1.0, 1.0, 1)
    with pytest.raises(capi.AgradError):      # a missing map
        ctx.call("agrad_adamw8bit_step", capi.F32, vp(d_p), vp(d_g), vp(d_qm), vp(d_qv), vp(d_am), vp(d_av), None,
                 vp(d_mapv), 8, 0, 1.0, 1e-3, 0.9, 0.99, 1e-8, 1.0, 1.0, 1)
    ctx.call("agrad_adamw8bit_step", capi.F32, vp(d_p), vp(d_g), vp(d_qm), vp(d_qv), vp(d_am), vp(d_av), vp(d_mapm),
             vp(d_mapv), 0, 0, 1.0, 1e-3, 0.9, 0.99, 1e-8, 1.0, 1.0, 1)      # empty: no launch
    ctx.synchronize()
    for d in (d_p, d_g, d_qm, d_qv, d_am, d_av, d_mapm, d_mapv):
        d.free()


def test_adamw_8bit_state_over_the_runtime():
    """AdamW(state_mode="8bit") on the hip device: the embedding table (V*C >= 4096
    elements) gets byte moments, gamma and beta (64 elements) keep fp32 ones
    (optimizer.py:205-222).  Expectation: the restated kernels applied per parameter
    to the gradients the device produced -- identical bits, three steps, with the
    clip coefficient passed into the step."""
    rng = np.random.default_rng(81)
    B, T, C_, V = 2, 16, 64, 80
    ids_np = rng.integers(0, V, (B, T), dtype=np.int32)
    rt = Runtime(device="hip")
    ids = Tensor(shape=(B, T), dtype=np.int32, device="hip", requires_grad=False, init_val=ids_np, name="ids")
    wte = Tensor(shape=(V, C_), dtype=np.float32, device="hip", requires_grad=True,
                 init_val=(0.5 * rng.standard_normal((V, C_))).astype(np.float32), name="wte")
    gamma = Tensor(shape=(C_,), dtype=np.float32, device="hip", requires_grad=True,
                   init_val=(1 + 0.1 * rng.standard_normal(C_)).astype(np.float32), name="gamma")
    beta = Tensor(shape=(C_,), dtype=np.float32, device="hip", requires_grad=True,
                  init_val=(0.1 * rng.standard_normal(C_)).astype(np.float32), name="beta")
    out = GELUOp()(LayerNormOp(eps=1e-5)(GatherOp()(ids, wte), gamma, beta))
    rt.loss = out
    rt.build_topo(out)
    rt.bind_memory()
    lr, betas, eps, wd = 1e-2, (0.9, 0.95), 1e-8, 0.1
    opt = AdamW([wte, gamma, beta], lr=lr, betas=betas, eps=eps, weight_decay=wd, runtime=rt, state_mode="8bit")
    assert [d[0] for d in opt.dispatches] == ["q8", "fp32", "fp32"]
    np.testing.assert_array_equal(rt.backend.storage_to_host(opt.qmap_m), K.dynamic_map(True))
    np.testing.assert_array_equal(rt.backend.storage_to_host(opt.qmap_v), K.dynamic_map(False))
    clip = opt.build_grad_clip()
    params = {"wte": wte, "gamma": gamma, "beta": beta}
    host = {k: rt.backend.copy_to_host(t).copy() for k, t in params.items()}
    mom = {k: (np.zeros_like(a), np.zeros_like(a)) for k, a in host.items() if k != "wte"}
    n = V * C_
    qm, qv = np.zeros(n, np.uint8), np.zeros(n, np.uint8)
    am, av = np.zeros(n // 256, np.float32), np.zeros(n // 256, np.float32)
    upstream = rng.standard_normal((B, T, C_)).astype(np.float32)
    for t in range(1, 4):
        rt.forward()
        rt.zero_grad()
        rt.backend.copy_from_host(out.grad, upstream)
        rt.backward_graph()
        rt.backend.synchronize()
        grads = {k: rt.backend.copy_to_host(p.grad).copy() for k, p in params.items()}
        _, coef = clip(1.0)
        opt.step(grad_scale=coef)
        lr_bc1 = lr / (1.0 - betas[0] ** t)
        inv_sqrt_bc2 = 1.0 / math.sqrt(1.0 - betas[1] ** t)
        K.adamw8bit_step(host["wte"].reshape(-1), grads["wte"].reshape(-1), qm, qv, am, av, K.dynamic_map(True),
                         K.dynamic_map(False), np.float32(1.0 - lr * wd), lr_bc1, betas[0], betas[1], eps, n, t == 1,
                         inv_sqrt_bc2, clip_coef=coef)
        for k in ("gamma", "beta"):
            m, v = mom[k]
            K.adamw_step_split(host[k], grads[k], m, v, 0.0, betas[0], betas[1], eps, lr_bc1, inv_sqrt_bc2, coef)
        for k in params:
            np.testing.assert_array_equal(rt.backend.copy_to_host(params[k]), host[k], err_msg=f"{k} at step {t}")
        np.testing.assert_array_equal(rt.backend.storage_to_host(opt.m[0]), qm, err_msg=f"codes of m at step {t}")
        np.testing.assert_array_equal(rt.backend.storage_to_host(opt.v[0]), qv, err_msg=f"codes of v at step {t}")
    opt.release()
    rt.release()
