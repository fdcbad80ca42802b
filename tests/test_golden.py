"""The frozen vectors of tests/golden/layer_ops_small.npz against the CPU
restatement (no GPU) and against the HIP kernels through the C ABI (gpu)."""
import sys
from pathlib import Path

import numpy as np
import pytest

from autograd_amd import capi
from tests.helpers import assert_fp32_close, assert_fp32_parity

GOLDEN = Path(__file__).parent / "golden" / "layer_ops_small.npz"


@pytest.fixture(scope="module")
def vec():
    return dict(np.load(GOLDEN, allow_pickle=False))


def test_restatement_reproduces_the_frozen_vectors(vec):
    sys.path.insert(0, str(GOLDEN.parent))
    import make_vectors
    now = make_vectors.build()
    assert set(now) == set(vec)
    for name, want in vec.items():
        got = now[name]
        assert got.dtype == want.dtype and got.shape == want.shape, name
        if want.dtype.kind in "iu":
            np.testing.assert_array_equal(got, want, err_msg=name)
        else:
            # libm differences between numpy builds are a few ulp of exp / tanh
            assert_fp32_close(got, want, name, rtol=2e-6, atol=2e-7)


@pytest.mark.gpu
def test_kernels_reproduce_the_frozen_vectors(ctx, vec):
    from oracle import closed_form as cf
    from tests import gpu_ops as G
    v = vec
    y, _ = G.norm_forward(ctx, capi.NORM_LAYER, v["x"], v["gamma"], v["beta"], 1e-5)
    assert_fp32_close(y, v["ln_y"], "layernorm y")
    out = G.norm_backward(ctx, capi.NORM_LAYER, v["x"], v["gamma"], v["dy"], 1e-5)
    assert_fp32_close(out["dx"], v["ln_dx"], "layernorm dx")
    _, dg64, db64 = cf.layernorm_grads(v["x"], v["gamma"], v["dy"], 1e-5)
    assert_fp32_parity(out["dgamma"], v["ln_dgamma"], dg64.reshape(v["ln_dgamma"].shape), "layernorm dgamma")
    assert_fp32_parity(out["dbeta"], v["ln_dbeta"], db64.reshape(v["ln_dbeta"].shape), "layernorm dbeta")
    y, _ = G.norm_forward(ctx, capi.NORM_RMS, v["x"], v["gamma"], None, 1e-6)
    assert_fp32_close(y, v["rms_y"], "rmsnorm y")
    out = G.norm_backward(ctx, capi.NORM_RMS, v["x"], v["gamma"], v["dy"], 1e-6, want_dbeta=False)
    assert_fp32_close(out["dx"], v["rms_dx"], "rmsnorm dx")
    assert_fp32_parity(out["dgamma"], v["rms_dgamma"], cf.rmsnorm_grads(v["x"], v["gamma"], v["dy"], 1e-6)[1].reshape(v["rms_dgamma"].shape),
                       "rmsnorm dgamma")
    y, h = G.norm_forward(ctx, capi.NORM_LAYER, v["x"], v["gamma"], v["beta"], 1e-5, residual=v["res"], want_h=True)
    np.testing.assert_array_equal(h, v["addln_h"])
    assert_fp32_close(y, v["addln_y"], "add+layernorm y")
    assert_fp32_close(G.unary(ctx, "agrad_gelu_forward", v["act_x"]), v["gelu_y"], "gelu y")
    assert_fp32_parity(G.unary_backward(ctx, "agrad_gelu_backward", v["act_x"], v["act_dy"]), v["gelu_dx"],
                       cf.gelu_grad(v["act_x"]) * v["act_dy"].astype(np.float64), "gelu dx")
    np.testing.assert_array_equal(G.unary(ctx, "agrad_relu2_forward", v["act_x"]), v["relu2_y"])
    np.testing.assert_array_equal(G.unary_backward(ctx, "agrad_relu2_backward", v["act_x"], v["act_dy"]), v["relu2_dx"])
    assert_fp32_close(G.swiglu_forward(ctx, v["gu"]), v["swiglu_h"], "swiglu h")
    assert_fp32_close(G.swiglu_backward(ctx, v["gu"], v["act_dy"]), v["swiglu_dgu"], "swiglu dgu")
    q2, k2 = G.rope(ctx, v["rope_q"], v["rope_k"], v["rope_cos"], v["rope_sin"], 1)
    np.testing.assert_array_equal(q2, v["rope_q_out"])
    np.testing.assert_array_equal(k2, v["rope_k_out"])
    np.testing.assert_array_equal(G.gather_forward(ctx, v["ids"], v["W"]), v["gather_out"])
    np.testing.assert_array_equal(G.gather_forward(ctx, v["ids"], v["W"], v["wpe"]), v["embsum_out"])
    dW = G.embedding_backward(ctx, v["ids"], v["dy"], v["W"].shape[0])
    assert_fp32_close(dW, v["emb_dW"], "embedding dW", atol=2e-6)
    np.testing.assert_array_equal(G.pos_embedding_backward(ctx, v["dy"]), v["emb_dwpe"])
    # cross-entropy and AdamW have no numpy wrapper: straight through the C ABI
    import ctypes as C

    def vp(d):
        return C.c_void_p(d.ptr)
    logits, ids, dloss = v["logits"], v["ids"], v["dloss"]
    rows, V = ids.size, logits.shape[-1]
    d_x, d_l, d_g = ctx.upload(logits), ctx.upload(ids.astype(np.int32)), ctx.upload(dloss)
    d_loss, d_lse, d_dx = ctx.empty((rows,), np.float32), ctx.empty((rows,), np.float32), ctx.empty(logits.shape, np.float32)
    ctx.call("agrad_cross_entropy_forward", capi.F32, vp(d_x), vp(d_l), vp(d_loss), vp(d_lse), rows, V)
    ctx.call("agrad_cross_entropy_backward", capi.F32, vp(d_x), vp(d_l), vp(d_g), vp(d_lse), vp(d_dx), rows, V, 0)
    ctx.synchronize()
    assert_fp32_close(d_loss.download().reshape(ids.shape), v["ce_loss"], "cross-entropy loss")
    assert_fp32_close(d_dx.download(), v["ce_dlogits"], "cross-entropy dlogits")
    p, g = ctx.upload(v["adam_p0"]), ctx.upload(v["adam_g"])
    m, s2 = ctx.zeros(v["adam_p0"].shape, np.float32), ctx.zeros(v["adam_p0"].shape, np.float32)
    n = v["adam_p0"].size
    ctx.call("agrad_adamw_step", capi.F32, vp(p), vp(g), vp(m), vp(s2), n, n, 1e-3 * 0.1, 0.9, 1.0 - 0.9, 0.999,
             1.0 - 0.999, 1e-8, 1e-3 * np.sqrt(1 - 0.999) / (1 - 0.9), 1.0, 1.0)
    ctx.synchronize()
    np.testing.assert_array_equal(p.download(), v["adam_p1"])
    np.testing.assert_array_equal(m.download(), v["adam_m1"])
    np.testing.assert_array_equal(s2.download(), v["adam_v1"])
    for d in (d_x, d_l, d_g, d_loss, d_lse, d_dx, p, g, m, s2):
        d.free()
