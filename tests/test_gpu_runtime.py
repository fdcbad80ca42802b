"""The same graph on the numpy oracle device ("cpu") and on "hip", compared.

This is the reference's own method: run_single_op builds a graph, runs forward,
zeroes grads, writes an upstream gradient into out.grad, runs backward_graph and
reads outputs and gradients back (check_tiny_gpt2_kernel.py:473-490), once per
device.  The hip side goes Tensor -> Op -> HipBackend -> hip_ext.HipContext ->
agrad_dispatch (C ABI) -> kernel.
"""
import numpy as np
import pytest

from autograd_amd.device import Device
from autograd_amd.op import (AddLayerNormOp, AddOp, AddRMSNormOp, EmbeddingSumOp, GatherOp, GELUOp,
                             LayerNormOp, ReLUSquaredOp, RMSNormOp, RopeOp, SwiGLUOp)
from autograd_amd.runtime import ExecutionPlan, Runtime, bind_plans
from autograd_amd.tensor import Tensor
from autograd_amd.utils import BF16
from oracle import cpu_device
from oracle import cpu_ops as ref
from tests.helpers import assert_bf16_close, assert_chain_close, assert_fp32_close

pytestmark = pytest.mark.gpu
SEED = 1333
cpu_device.register()


def make_tensor(shape, dtype, device, requires_grad, value, name=""):
    return Tensor(shape=tuple(shape), dtype=dtype, device=device, requires_grad=requires_grad,
                  init_val=np.asarray(value), name=name)


def run_single_op(device, build_fn, upstream=None, fuse=True):
    rt = Runtime(device=device, fuse_grad_zeroing=fuse)
    out, tracked = build_fn(device)
    outs = out if isinstance(out, (tuple, list)) else (out,)
    rt.loss = outs[0]
    rt.build_topo(outs[0])
    rt.bind_memory()
    rt.forward()
    rt.backend.synchronize()
    if upstream is not None:
        rt.zero_grad()
        rt.backend.copy_from_host(outs[0].grad, np.asarray(upstream, dtype=np.float32))
        rt.backward_graph()
        rt.backend.synchronize()
    host = [rt.backend.copy_to_host(o) for o in outs]
    grads = {k: (None if t.grad is None else rt.backend.copy_to_host(t.grad)) for k, t in tracked.items()}
    rt.release()
    return host, grads


def both(build_fn, upstream, fuse=True):
    cpu = run_single_op("cpu", build_fn, upstream)
    hip = run_single_op("hip", build_fn, upstream, fuse=fuse)
    return cpu, hip


def test_probe_layernorm():
    """probe_layernorm (check_tiny_gpt2_kernel.py:758-782)."""
    rng = np.random.default_rng(SEED + 4)
    B, T, C = 2, 16, 64
    x_np = rng.standard_normal((B, T, C), dtype=np.float32)
    g_np = rng.standard_normal((C,), dtype=np.float32)
    b_np = rng.standard_normal((C,), dtype=np.float32)
    upstream = rng.standard_normal((B, T, C), dtype=np.float32)

    def build(device):
        x = make_tensor(x_np.shape, np.float32, device, True, x_np)
        g = make_tensor(g_np.shape, np.float32, device, True, g_np)
        b = make_tensor(b_np.shape, np.float32, device, True, b_np)
        return LayerNormOp(eps=1e-5)(x, g, b), {"x": x, "gamma": g, "beta": b}

    for fuse in (True, False):
        (c_out, c_g), (h_out, h_g) = both(build, upstream, fuse)
        assert_fp32_close(h_out[0], c_out[0], "forward")
        for name in ("x", "gamma", "beta"):
            assert_fp32_close(h_g[name], c_g[name], f"{name}.grad fuse={fuse}")


def test_probe_gelu():
    """probe_gelu (check_tiny_gpt2_kernel.py:783-794)."""
    rng = np.random.default_rng(SEED + 5)
    x_np = rng.standard_normal((2, 16, 64), dtype=np.float32)
    upstream = rng.standard_normal(x_np.shape, dtype=np.float32)

    def build(device):
        x = make_tensor(x_np.shape, np.float32, device, True, x_np)
        return GELUOp()(x), {"x": x}

    (c_out, c_g), (h_out, h_g) = both(build, upstream)
    assert_fp32_close(h_out[0], c_out[0], "forward")
    assert_fp32_close(h_g["x"], c_g["x"], "x.grad")


def test_probe_gather_position_table():
    """probe_gather: GatherOp on a position table with pos_ids = tile(arange(T))
    (check_tiny_gpt2_kernel.py:282, 875-890)."""
    rng = np.random.default_rng(SEED + 6)
    B, T, C = 2, 32, 256
    pos_ids = np.tile(np.arange(T, dtype=np.int32), (B, 1))
    w_np = (0.02 * rng.standard_normal((T, C))).astype(np.float32)
    upstream = rng.standard_normal((B, T, C), dtype=np.float32)

    def build(device):
        idx = make_tensor(pos_ids.shape, np.int32, device, False, pos_ids)
        w = make_tensor(w_np.shape, np.float32, device, True, w_np)
        return GatherOp()(idx, w), {"w": w}

    (c_out, c_g), (h_out, h_g) = both(build, upstream)
    np.testing.assert_array_equal(h_out[0].view(np.uint32), c_out[0].view(np.uint32))
    assert_fp32_close(h_g["w"], c_g["w"], "w.grad")


def test_probe_fill_and_copy():
    """probe_fill (check_tiny_gpt2_kernel.py:795-810) plus copy round trips."""
    rt = Runtime(device="hip")
    t = Tensor(shape=(8,), dtype=np.float32, requires_grad=False, device="hip")
    t.storage = rt.allocator.alloc(t.shape, t.dtype)
    rt.backend.copy_from_host(t, np.full((8,), 9.0, dtype=np.float32))
    for v in (0.0, 1.0, -2.5):
        rt.backend.begin_pass()
        rt.backend.fill(t, v)
        rt.backend.end_pass()
        np.testing.assert_array_equal(rt.backend.copy_to_host(t), np.full((8,), v, np.float32))
    # odd sizes and offsets through the arena view path
    big = rt.allocator.alloc((1000,), np.float32)
    rt.backend.fill_storage(big, 3.0)
    view = rt.allocator.view(big, 4 * 3, (77,), np.float32)
    rt.backend.fill_storage(view, 5.0)
    host = rt.backend.ctx.copy_to_host(big.ptr.buffer_id, 0, [1000], "float32")
    want = np.full(1000, 3.0, np.float32)
    want[3:80] = 5.0
    np.testing.assert_array_equal(host, want)
    with pytest.raises(RuntimeError):
        rt.allocator.view(big, 4 * 990, (11,), np.float32)
    # bf16 storage: copy_from_host rounds to nearest even, copy_to_host widens
    tb = Tensor(shape=(5,), dtype=BF16, requires_grad=False, device="hip")
    tb.storage = rt.allocator.alloc(tb.shape, tb.dtype)
    vals = np.array([1.0, 1.00390625, 3.14159, -2.7e-3, 65504.0], np.float32)
    rt.backend.copy_from_host(tb, vals)
    np.testing.assert_array_equal(rt.backend.copy_to_host(tb), ref.round_bf16(vals))
    rt.backend.fill(tb, 0.1)
    np.testing.assert_array_equal(rt.backend.copy_to_host(tb), np.full(5, ref.round_bf16(np.float32(0.1))))


def test_unknown_device_and_kernel():
    with pytest.raises(ValueError):
        Device.get_backend("mps")
    ctx = Device.get_backend("hip").ctx
    with pytest.raises(RuntimeError):
        ctx.dispatch_with_args_3d("sdpa_forward", [], [], [], 1, 1, 1, 1)     # attention is not part of this library
    with pytest.raises(ValueError):      # wrong operand count
        ctx.dispatch_with_args_3d("gelu_forward_kernel", [0], [0], [0, 1, 0], 1, 1, 1, 1)
    buf = ctx.alloc(64)
    with pytest.raises(ValueError):      # range outside the buffer
        ctx.dispatch_with_args_3d("gelu_forward_kernel", [buf, buf], [0, 0], [0, 1000, 0], 1, 1, 1, 1)
    ctx.free(buf)


def test_config1_tiny_gpt2_chain():
    """The tiny-gpt2 chain (benchmark configuration 0): ids -> wte + wpe gather-sum ->
    LayerNorm (gamma 1, beta 0) -> GELU, B=4 T=128 C=128 V=50257, fp32, forward then backward."""
    rng = np.random.default_rng(SEED + 0)
    B, T, C, V = 4, 128, 128, 50257
    ids_np = rng.integers(0, V, size=(B, T), dtype=np.int32)
    wte_np = (0.02 * rng.standard_normal((V, C))).astype(np.float32)
    wpe_np = (0.02 * rng.standard_normal((T, C))).astype(np.float32)
    upstream = rng.standard_normal((B, T, C), dtype=np.float32)

    def build(device):
        ids = make_tensor((B, T), np.int32, device, False, ids_np)
        wte = make_tensor((V, C), np.float32, device, True, wte_np, "wte")
        wpe = make_tensor((T, C), np.float32, device, True, wpe_np, "wpe")
        g = make_tensor((C,), np.float32, device, True, np.ones(C, np.float32))
        b = make_tensor((C,), np.float32, device, True, np.zeros(C, np.float32))
        x0 = EmbeddingSumOp()(ids, wte, wpe)
        y = LayerNormOp(eps=1e-5)(x0, g, b)
        return GELUOp()(y), {"wte": wte, "wpe": wpe, "gamma": g, "beta": b}

    (c_out, c_g), (h_out, h_g) = both(build, upstream)
    assert_fp32_close(h_out[0], c_out[0], "config 1 forward")
    # Three ops deep, and LayerNorm of rows with std 0.03 multiplies dy by ~35:
    # an element where that cancels to O(1) carries the rounding of O(35) terms,
    # so the absolute budget is set on the gradient's own scale.
    scale = max(1.0, float(np.abs(c_g["wte"]).max()))
    assert_fp32_close(h_g["wte"], c_g["wte"], "wte.grad", rtol=1e-5, atol=2e-6 * scale)
    assert_fp32_close(h_g["wpe"], c_g["wpe"], "wpe.grad", rtol=1e-5, atol=2e-6 * scale)
    atol = 1e-6 * np.sqrt(B * T)
    assert_fp32_close(h_g["gamma"], c_g["gamma"], "gamma.grad", rtol=1e-5, atol=atol)
    assert_fp32_close(h_g["beta"], c_g["beta"], "beta.grad", rtol=1e-5, atol=atol)

    # the unfused reference composition gives the same numbers: Gather x2 + Add
    def build_unfused(device):
        ids = make_tensor((B, T), np.int32, device, False, ids_np)
        pos = make_tensor((B, T), np.int32, device, False, np.tile(np.arange(T, dtype=np.int32), (B, 1)))
        wte = make_tensor((V, C), np.float32, device, True, wte_np)
        wpe = make_tensor((T, C), np.float32, device, True, wpe_np)
        g = make_tensor((C,), np.float32, device, True, np.ones(C, np.float32))
        b = make_tensor((C,), np.float32, device, True, np.zeros(C, np.float32))
        x0 = AddOp()(GatherOp()(ids, wte), GatherOp()(pos, wpe))
        return GELUOp()(LayerNormOp(eps=1e-5)(x0, g, b)), {"wte": wte, "wpe": wpe}

    u_out, u_g = run_single_op("hip", build_unfused, upstream)
    np.testing.assert_array_equal(u_out[0], h_out[0])
    np.testing.assert_array_equal(u_g["wpe"], h_g["wpe"])
    np.testing.assert_array_equal(u_g["wte"], h_g["wte"])


@pytest.mark.parametrize("dtype", [np.float32, BF16])
def test_transformer_block_slice(dtype):
    """A chain that uses every op once: gather -> add+RMSNorm -> rope on q/k views
    is not expressible without GEMMs, so the slices are chained directly:
    gather -> AddRMSNorm(residual) -> SwiGLU -> ReLU^2 -> AddLayerNorm -> Add."""
    rng = np.random.default_rng(SEED + 7)
    B, T, C, V = 2, 24, 256, 97
    ids_np = rng.integers(0, V, size=(B, T), dtype=np.int32)
    w_np = rng.standard_normal((V, C)).astype(np.float32)
    r_np = rng.standard_normal((B, T, C)).astype(np.float32)
    g1 = (1 + 0.02 * rng.standard_normal(C)).astype(np.float32)
    g2 = (1 + 0.02 * rng.standard_normal(C // 2)).astype(np.float32)
    b2 = (0.02 * rng.standard_normal(C // 2)).astype(np.float32)
    upstream = rng.standard_normal((B, T, C // 2)).astype(np.float32)

    def build(device):
        ids = make_tensor((B, T), np.int32, device, False, ids_np)
        w = make_tensor((V, C), dtype, device, True, w_np)
        r = make_tensor((B, T, C), dtype, device, True, r_np)
        ga = make_tensor((C,), np.float32, device, True, g1)
        gb = make_tensor((C // 2,), np.float32, device, True, g2)
        bb = make_tensor((C // 2,), np.float32, device, True, b2)
        x = GatherOp()(ids, w)
        h, y = AddRMSNormOp(eps=1e-6)(x, r, ga)
        s = SwiGLUOp()(y)                    # [B,T,C/2]
        a = ReLUSquaredOp()(s)
        h2, y2 = AddLayerNormOp(eps=1e-5)(a, s, gb, bb)
        out = AddOp()(h2, y2)
        return out, {"w": w, "r": r, "ga": ga, "gb": gb, "bb": bb}

    (c_out, c_g), (h_out, h_g) = both(build, upstream)
    if dtype is BF16:
        assert_bf16_close(h_out[0], c_out[0], "block forward", rel=2e-2)
        for k in ("r",):
            assert_bf16_close(h_g[k], c_g[k], f"{k}.grad", rel=3e-2)
    else:
        # six kernels forward; a gradient has those and up to six backward kernels behind it; the
        # table's rows and the norm parameters are sums over up to B * T rows
        assert_chain_close(h_out[0], c_out[0], "block forward", kernels=6)
        assert_chain_close(h_g["r"], c_g["r"], "r.grad", kernels=12)
        assert_chain_close(h_g["w"], c_g["w"], "w.grad", kernels=12, sum_rows=B * T)
        for k in ("ga", "gb", "bb"):
            assert_chain_close(h_g[k], c_g[k], f"{k}.grad", kernels=12, sum_rows=B * T)
    # fused zeroing and fill-then-accumulate agree bit for bit
    n_out, n_g = run_single_op("hip", build, upstream, fuse=False)
    np.testing.assert_array_equal(n_out[0], h_out[0])
    for k in h_g:
        np.testing.assert_array_equal(n_g[k] + 0.0, h_g[k] + 0.0)


@pytest.mark.parametrize("sign", [1, -1])
def test_rope_op_in_graph(sign):
    """RopeOp on leaves (copy, then rotate) and on activations (aliased, in place)."""
    rng = np.random.default_rng(SEED + 8)
    B, T, H, HKV, D = 2, 16, 4, 2, 64
    q_np = rng.standard_normal((B, T, H, D)).astype(np.float32)
    k_np = rng.standard_normal((B, T, HKV, D)).astype(np.float32)
    cos_np, sin_np = ref.rope_tables(32, D, 1e4)
    up = rng.standard_normal((B, T, H, D)).astype(np.float32)

    def build_leaf(device):
        q = make_tensor(q_np.shape, np.float32, device, True, q_np)
        k = make_tensor(k_np.shape, np.float32, device, True, k_np)
        c = make_tensor(cos_np.shape, np.float32, device, False, cos_np)
        s = make_tensor(sin_np.shape, np.float32, device, False, sin_np)
        q2, k2 = RopeOp(rope_sign=sign)(q, k, c, s)
        return (q2, k2), {"q": q, "k": k}

    def build_act(device):
        q = make_tensor(q_np.shape, np.float32, device, True, q_np)
        k = make_tensor(k_np.shape, np.float32, device, True, k_np)
        c = make_tensor(cos_np.shape, np.float32, device, False, cos_np)
        s = make_tensor(sin_np.shape, np.float32, device, False, sin_np)
        qa, ka = ReLUSquaredOp()(q), ReLUSquaredOp()(k)
        q2, k2 = RopeOp(rope_sign=sign)(qa, ka, c, s)
        out = AddOp()(q2, q2)
        return (out, k2), {"q": q, "k": k}

    want_q, want_k = q_np.copy(), k_np.copy()
    ref.rope_signed(want_q, want_k, cos_np, sin_np, sign, False)
    (c_out, c_g), (h_out, h_g) = both(build_leaf, up)
    np.testing.assert_array_equal(h_out[0], want_q)
    np.testing.assert_array_equal(c_out[0], want_q)
    assert_fp32_close(h_g["q"], c_g["q"], "q.grad (leaf)")
    back = up.copy()
    ref.rope_signed(back, np.zeros_like(k_np), cos_np, sin_np, sign, True)
    np.testing.assert_array_equal(h_g["q"], back)

    (c_out, c_g), (h_out, h_g) = both(build_act, up)
    assert_fp32_close(h_out[0], c_out[0], "rope on activations")
    assert_fp32_close(h_g["q"], c_g["q"], "q.grad (aliased)")


@pytest.mark.parametrize("dim", [0, 1, 2, -1])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_softmax_over_any_axis_in_a_graph(dim, dtype):
    """SoftmaxOp(dim) for every axis of a [B, T, C] activation on both devices
    (cpu_softmax_forward / backward take any axis, backend.py:354-374): forward,
    the gradient into an activation, and a second pass over the same arena"""
    from autograd_amd.utils import BF16
    rng = np.random.default_rng(SEED + 50 + (dim % 3))
    B, T, C = 5, 70, 24
    x_np = rng.standard_normal((B, T, C), dtype=np.float32)
    g_np = (1 + 0.1 * rng.standard_normal(C)).astype(np.float32)
    upstream = rng.standard_normal((B, T, C), dtype=np.float32)
    dt = BF16 if dtype == "bf16" else np.float32

    def build(device):
        x = make_tensor(x_np.shape, dt, device, True, x_np, "x")
        g = make_tensor(g_np.shape, np.float32, device, True, g_np, "g")
        return x.rms_norm(g).softmax(dim), {"x": x}

    (c_out, c_g), (h_out, h_g) = both(build, upstream)
    if dtype == "bf16":
        assert_bf16_close(h_out[0], c_out[0], f"softmax dim={dim}")
        scale = float(np.abs(c_g["x"]).max())
        assert np.abs(h_g["x"] - c_g["x"]).max() <= 3e-2 * scale
    else:
        # norm, (layout change,) softmax forward; the gradient has their backward kernels behind it as well
        assert_chain_close(h_out[0], c_out[0], f"softmax dim={dim}", kernels=2)
        assert_chain_close(h_g["x"], c_g["x"], "x.grad", kernels=4)
        np.testing.assert_allclose(h_out[0].sum(axis=dim), 1.0, rtol=0, atol=2e-6)


def test_embedding_table_with_bf16_gradient_storage():
    """an fp32 table whose gradient is kept in bf16 (Tensor(grad_dtype=BF16); the
    reference's bf16 gradient store, backend.py:2808-2812): the backward pass rounds each
    row's fp32 sum once; two passes accumulate in bf16, on both devices; AdamW then reads
    the bf16 gradient"""
    from autograd_amd.optimizer import AdamW
    from autograd_amd.utils import BF16
    rng = np.random.default_rng(SEED + 60)
    B, T, V, C = 4, 96, 300, 64
    ids_np = rng.integers(0, V, (B, T), dtype=np.int32)
    w_np = (0.5 * rng.standard_normal((V, C))).astype(np.float32)
    upstream = rng.standard_normal((B, T, C)).astype(np.float32)
    results = {}
    for device in ("cpu", "hip"):
        rt = Runtime(device=device)
        ids = Tensor(shape=(B, T), dtype=np.int32, device=device, requires_grad=False, init_val=ids_np)
        w = Tensor(shape=(V, C), dtype=np.float32, device=device, requires_grad=True, init_val=w_np, grad_dtype=BF16)
        out = ids.gather(w).relu2()
        rt.loss = out
        rt.build_topo(out)
        rt.bind_memory()
        rt.accumulate_parameter_grads = True
        rt.backend.accumulate_parameter_grads = True
        rt.zero_grad()
        for _ in range(2):
            rt.forward()
            rt.backend.copy_from_host(out.grad, upstream)
            rt.backward_graph()
        rt.backend.synchronize()
        assert np.dtype(w.grad.storage.dtype) == np.dtype(np.uint16)
        grad = rt.backend.copy_to_host(w.grad).copy()
        opt = AdamW([w], lr=1e-2, weight_decay=0.0, runtime=rt)
        opt.step()
        results[device] = (grad, rt.backend.copy_to_host(w).copy())
        opt.release()
        rt.release()
    (c_grad, c_w), (h_grad, h_w) = results["cpu"], results["hip"]
    x = np.maximum(w_np[ids_np], 0)
    once = np.zeros((V, C), np.float64)
    np.add.at(once, ids_np.reshape(-1), (2 * x * upstream).reshape(-1, C).astype(np.float64))
    assert_bf16_close(h_grad, 2 * once, "bf16 table gradient vs float64", rel=2e-2)
    assert_bf16_close(h_grad, c_grad, "bf16 table gradient, hip vs cpu", rel=1.6e-2)
    assert np.abs(h_w - c_w).max() <= 2.1e-2          # a first Adam step moves by lr * sign(g): same side, or a zero gradient


def test_norm_parameters_with_bf16_gradient_storage():
    """gamma / beta and a bias under a broadcast Add with grad_dtype=BF16 under fp32
    activations, on both devices"""
    from autograd_amd.utils import BF16
    rng = np.random.default_rng(SEED + 61)
    B, T, C = 6, 40, 96
    x_np = rng.standard_normal((B, T, C), dtype=np.float32)
    g_np = (1 + 0.1 * rng.standard_normal(C)).astype(np.float32)
    b_np = (0.1 * rng.standard_normal(C)).astype(np.float32)
    upstream = rng.standard_normal((B, T, C), dtype=np.float32)

    def build(device):
        x = make_tensor(x_np.shape, np.float32, device, True, x_np, "x")
        g = Tensor(shape=(C,), dtype=np.float32, device=device, requires_grad=True, init_val=g_np, grad_dtype=BF16)
        b = Tensor(shape=(C,), dtype=np.float32, device=device, requires_grad=True, init_val=b_np, grad_dtype=BF16)
        bias = Tensor(shape=(C,), dtype=np.float32, device=device, requires_grad=True, init_val=b_np, grad_dtype=BF16)
        return x.relu2().layer_norm(g, b) + bias, {"x": x, "g": g, "b": b, "bias": bias}

    (c_out, c_g), (h_out, h_g) = both(build, upstream)
    assert_chain_close(h_out[0], c_out[0], "forward", kernels=3)       # relu2, norm, add
    assert_chain_close(h_g["x"], c_g["x"], "x.grad", kernels=6)        # ... and their backward kernels
    for name in ("g", "b", "bias"):
        assert_bf16_close(h_g[name], c_g[name], f"{name}.grad stored as bf16", rel=1.6e-2)


def test_rope_op_bhtd_layout_in_graph():
    """RopeOp(layout="bhtd") on [B,H,T,D] activations equals the default layout on the
    transposed tensors, forward and gradients, on both devices"""
    rng = np.random.default_rng(SEED + 9)
    B, T, H, HKV, D = 2, 12, 4, 2, 32
    q_np = rng.standard_normal((B, H, T, D)).astype(np.float32)
    k_np = rng.standard_normal((B, HKV, T, D)).astype(np.float32)
    cos_np, sin_np = ref.rope_tables(16, D, 1e4)
    up = rng.standard_normal((B, H, T, D)).astype(np.float32)

    def build(device):
        q = make_tensor(q_np.shape, np.float32, device, True, q_np)
        k = make_tensor(k_np.shape, np.float32, device, True, k_np)
        c = make_tensor(cos_np.shape, np.float32, device, False, cos_np)
        s = make_tensor(sin_np.shape, np.float32, device, False, sin_np)
        q2, k2 = RopeOp(rope_sign=1, layout="bhtd")(ReLUSquaredOp()(q), ReLUSquaredOp()(k), c, s)
        return (AddOp()(q2, q2), k2), {"q": q, "k": k}

    (c_out, c_g), (h_out, h_g) = both(build, up)
    qa = np.maximum(q_np, 0) ** 2
    want = np.ascontiguousarray(qa.transpose(0, 2, 1, 3))
    ref.rope_signed(want, np.zeros((B, T, 1, D), np.float32), cos_np, sin_np, 1, False)
    np.testing.assert_array_equal(h_out[0], 2 * want.transpose(0, 2, 1, 3))
    np.testing.assert_array_equal(c_out[0], h_out[0])
    assert_fp32_close(h_g["q"], c_g["q"], "q.grad, bhtd")
    with pytest.raises(ValueError):
        RopeOp(layout="thbd")


def test_accumulate_parameter_grads_and_rerun():
    """Two backward passes with accumulate_parameter_grads give twice the
    parameter gradient; without it the second pass starts from zero."""
    rng = np.random.default_rng(SEED + 9)
    x_np = rng.standard_normal((32, 384)).astype(np.float32)
    g_np = (1 + 0.02 * rng.standard_normal(384)).astype(np.float32)
    rt = Runtime(device="hip")
    x = make_tensor(x_np.shape, np.float32, "hip", True, x_np)
    g = make_tensor(g_np.shape, np.float32, "hip", True, g_np)
    out = RMSNormOp(eps=1e-6)(x, g)
    rt.backward(out, grad_scale=0.5)
    first = rt.backend.copy_to_host(g.grad)
    dx_first = rt.backend.copy_to_host(x.grad)
    rt.backward(out, grad_scale=0.5)
    np.testing.assert_array_equal(rt.backend.copy_to_host(g.grad), first)
    rt.backward(out, grad_scale=0.5, accumulate_parameter_grads=True)
    assert_fp32_close(rt.backend.copy_to_host(g.grad), 2 * first, "accumulated gamma.grad", atol=2e-6)
    assert_fp32_close(rt.backend.copy_to_host(x.grad), 2 * dx_first, "accumulated x.grad", atol=2e-6)
    dx = np.zeros_like(x_np)
    dg = np.zeros_like(g_np)
    ref.rmsnorm_backward_into(x_np, g_np, np.full_like(x_np, 0.5), 1e-6, dx, dg)
    assert_fp32_close(first, dg, "gamma.grad", atol=4e-6)
    assert_fp32_close(dx_first, dx, "x.grad")
    rt.release()


def test_tied_gamma_with_separate_betas_over_two_steps():
    """Two LayerNorms share gamma and own a beta each.  gamma.grad is first written by the
    later node, so the earlier one accumulates its parameter gradients -- including its own
    beta's, which therefore must have been zero-filled: a second step gives the first
    step's numbers again, and they are the CPU device's."""
    rng = np.random.default_rng(SEED + 21)
    x_np = rng.standard_normal((4, 16, 64)).astype(np.float32)
    g_np = (1 + 0.1 * rng.standard_normal(64)).astype(np.float32)
    up = rng.standard_normal(x_np.shape).astype(np.float32)
    grads = {}
    for device in ("cpu", "hip"):
        x = make_tensor(x_np.shape, np.float32, device, True, x_np)
        gamma = make_tensor((64,), np.float32, device, True, g_np)
        beta_a = make_tensor((64,), np.float32, device, True, np.zeros(64, np.float32))
        beta_b = make_tensor((64,), np.float32, device, True, np.zeros(64, np.float32))
        out = LayerNormOp(eps=1e-5)(GELUOp()(LayerNormOp(eps=1e-5)(x, gamma, beta_a)), gamma, beta_b)
        rt = Runtime(device=device)
        rt.loss = out
        rt.build_topo(out)
        rt.bind_memory()
        steps = []
        for _ in range(2):
            rt.forward()
            rt.zero_grad()
            rt.backend.copy_from_host(out.grad, up)
            rt.backward_graph()
            rt.backend.synchronize()
            steps.append({k: rt.backend.copy_to_host(t.grad) for k, t in
                          (("x", x), ("gamma", gamma), ("beta_a", beta_a), ("beta_b", beta_b))})
        for k in steps[0]:
            np.testing.assert_array_equal(steps[1][k], steps[0][k], err_msg=f"{device}: {k}.grad changed on step 2")
        grads[device] = steps[1]
        rt.release()
    for k in grads["cpu"]:
        assert_fp32_close(grads["hip"][k], grads["cpu"][k], f"{k}.grad", atol=4e-6)


def test_rope_after_an_op_that_saves_its_output():
    """q = exp(x) is read again by Exp's backward, so Rope must not rotate it in place."""
    from autograd_amd.op import ExpOp
    rng = np.random.default_rng(SEED + 22)
    B, T, H, D = 2, 8, 2, 64
    x_np = (0.5 * rng.standard_normal((B, T, H, D))).astype(np.float32)
    k_np = rng.standard_normal((B, T, H, D)).astype(np.float32)
    cos_np, sin_np = ref.rope_tables(T, D, 1e4)
    up = rng.standard_normal((B, T, H, D)).astype(np.float32)

    def build(device):
        x = make_tensor(x_np.shape, np.float32, device, True, x_np)
        k = make_tensor(k_np.shape, np.float32, device, True, k_np)
        c = make_tensor(cos_np.shape, np.float32, device, False, cos_np)
        s = make_tensor(sin_np.shape, np.float32, device, False, sin_np)
        q2, k2 = RopeOp(rope_sign=1)(ExpOp()(x), GELUOp()(k), c, s)
        return AddOp()(q2, k2), {"x": x, "k": k}

    (c_out, c_g), (h_out, h_g) = both(build, up)
    assert_fp32_close(h_out[0], c_out[0], "forward")
    assert_fp32_close(h_g["x"], c_g["x"], "x.grad through exp", atol=2e-6)
    assert_fp32_close(h_g["k"], c_g["k"], "k.grad through gelu", atol=3e-6)
    # and against the formula: d/dx of rope(exp(x)) is rope^T(up) * exp(x)
    back = up.copy()
    ref.rope_signed(back, np.zeros_like(back), cos_np, sin_np, 1, True)
    assert_fp32_close(h_g["x"], back * np.exp(x_np), "x.grad closed form", rtol=2e-5, atol=2e-6)


def test_add_with_a_broadcast_operand():
    """x[B, T, C] + bias[C] and + table[T, C]: forward and both gradients through the
    runtime on both devices (the broadcasting branch of cpu_add_backward,
    backend.py:78-105; lead = 144 rows takes the two-stage column sum)."""
    rng = np.random.default_rng(SEED + 30)
    B, T, C = 9, 16, 48
    x_np = rng.standard_normal((B, T, C), dtype=np.float32)
    bias_np = rng.standard_normal((C,), dtype=np.float32)
    tab_np = rng.standard_normal((T, C), dtype=np.float32)
    upstream = rng.standard_normal((B, T, C), dtype=np.float32)

    def build(device):
        x = make_tensor(x_np.shape, np.float32, device, True, x_np)
        bias = make_tensor(bias_np.shape, np.float32, device, True, bias_np)
        tab = make_tensor(tab_np.shape, np.float32, device, True, tab_np)
        return ReLUSquaredOp()((x + bias) + tab), {"x": x, "bias": bias, "tab": tab}

    (c_out, c_g), (h_out, h_g) = both(build, upstream)
    assert_fp32_close(h_out[0], c_out[0], "forward")
    assert_fp32_close(h_g["x"], c_g["x"], "x.grad")
    assert_fp32_close(h_g["tab"], c_g["tab"], "tab.grad", atol=4e-6)
    assert_fp32_close(h_g["bias"], c_g["bias"], "bias.grad", atol=2e-5)


@pytest.mark.parametrize("dtype", [np.float32, BF16])
def test_layout_ops_in_a_graph(dtype):
    """reshape -> permute -> contiguous around compute ops, a transposed parameter and
    a transposed activation gradient, on both devices: forward and every gradient.
    Layout changes move bits, so the two devices differ only where GELU does."""
    rng = np.random.default_rng(SEED + 31)
    B, T, H, D = 3, 40, 6, 32
    x_np = rng.standard_normal((B, T, H * D), dtype=np.float32)
    w_np = rng.standard_normal((D, T), dtype=np.float32)
    upstream = rng.standard_normal((B, H, D, T), dtype=np.float32)

    def build(device):
        x = make_tensor(x_np.shape, dtype, device, True, x_np)
        w = make_tensor(w_np.shape, dtype, device, True, w_np)
        a = ReLUSquaredOp()(x)
        heads = a.reshape(B, T, H, D).permute(0, 2, 1, 3).contiguous()       # [B, H, T, D]: rows kernel
        y = heads + w.transpose(0, 1).contiguous()                             # [T, D] under [B, H]: tile kernel
        out = ReLUSquaredOp()(y).transpose(2, 3).contiguous()                  # [B, H, D, T]
        return out.view(B, H, D * T).reshape(B, H, D, T), {"x": x, "w": w}

    (c_out, c_g), (h_out, h_g) = both(build, upstream)
    if dtype is BF16:
        assert_bf16_close(h_out[0], c_out[0], "forward")
        assert_bf16_close(h_g["x"], c_g["x"], "x.grad")
        assert_bf16_close(h_g["w"], c_g["w"], "w.grad")
    else:
        np.testing.assert_array_equal(h_out[0], c_out[0])
        np.testing.assert_array_equal(h_g["x"], c_g["x"])
        assert_fp32_close(h_g["w"], c_g["w"], "w.grad", atol=2e-5)
    if dtype is not BF16:
        a_np = ref.relu2_forward(x_np)
        y_np = np.transpose(a_np.reshape(B, T, H, D), (0, 2, 1, 3)) + w_np.T
        np.testing.assert_array_equal(c_out[0], np.swapaxes(ref.relu2_forward(y_np), 2, 3))


def test_execution_plans_share_one_arena():
    """training plan + forward-only plan at another length over the same parameters,
    bound into one device arena (ExecutionPlan, runtime.py:857-892): alternating runs
    reproduce the oracle device's results for each plan"""
    rng = np.random.default_rng(SEED + 32)
    V, C = 301, 96
    w_np = (0.5 * rng.standard_normal((V, C))).astype(np.float32)
    g_np = (1 + 0.1 * rng.standard_normal(C)).astype(np.float32)
    feeds = {"train": rng.integers(0, V, (4, 48), dtype=np.int32), "eval": rng.integers(0, V, (1, 20), dtype=np.int32)}

    def plans(device):
        w = make_tensor((V, C), np.float32, device, True, w_np, "w")
        g = make_tensor((C,), np.float32, device, True, g_np, "g")
        out = {}
        for mode, ids_np in feeds.items():
            fwd_only = mode == "eval"
            ids = Tensor(shape=ids_np.shape, dtype=np.int32, device=device, requires_grad=False, name=mode)
            x = ids.gather(w)
            h, y = AddRMSNormOp(eps=1e-6)(x, ReLUSquaredOp()(x), g)
            o = (h + y).reshape(ids_np.size, C)
            rt = Runtime(device=device, forward_only=fwd_only, owns_params=not fwd_only)
            out[mode] = ExecutionPlan(runtime=rt, input_ids=ids, output=o, seq_len=ids_np.shape[1], mode=mode).prepare()
        arena = bind_plans(out.values())
        assert arena.nbytes == max(p.runtime.arena_bytes for p in out.values())
        return out, w, g, arena

    results = {}
    for device in ("cpu", "hip"):
        ps, w, g, arena = plans(device)
        runs = []
        for _ in range(2):
            ps["train"].set_inputs(feeds["train"])
            ps["train"].backward()
            be = ps["train"].runtime.backend
            be.synchronize()
            runs.append((be.copy_to_host(ps["train"].output), be.copy_to_host(w.grad), be.copy_to_host(g.grad)))
            ps["eval"].set_inputs(feeds["eval"])
            runs.append((ps["eval"].forward(),))
        results[device] = runs
        ps["train"].runtime.release()
        ps["eval"].runtime.release()
        if hasattr(ps["train"].runtime.allocator, "release"):
            ps["train"].runtime.allocator.release(arena)     # bind_plans' arena belongs to the caller
    for c_run, h_run in zip(results["cpu"], results["hip"]):
        for c_arr, h_arr in zip(c_run, h_run):
            assert_fp32_close(h_arr, c_arr, "plan result", atol=5e-6)
    # the second round equals the first on the device, bit for bit
    for a, b in zip(results["hip"][:2], results["hip"][2:]):
        for x0, x1 in zip(a, b):
            np.testing.assert_array_equal(x0, x1)


def test_primitive_ops_in_a_graph():
    """Mul in all four broadcast kinds (one of them x * x), Softmax, Exp, Log and Rsqrt
    chained in one graph on both devices (the reference probes them one at a time:
    check_tiny_gpt2_kernel.py:699-724, verify_ops.py:47-91)"""
    rng = np.random.default_rng(SEED + 33)
    B, T, C = 3, 70, 96
    x_np = rng.standard_normal((B, T, C), dtype=np.float32)
    w_np = (1 + 0.2 * rng.standard_normal(C)).astype(np.float32)
    s_np = np.array([0.37], np.float32)
    c_np = rng.uniform(0.5, 1.5, (B, T, 1)).astype(np.float32)
    upstream = rng.standard_normal((B, T, C), dtype=np.float32)

    def build(device):
        x = make_tensor(x_np.shape, np.float32, device, True, x_np, "x")
        w = make_tensor(w_np.shape, np.float32, device, True, w_np, "w")
        sc = make_tensor(s_np.shape, np.float32, device, True, s_np, "s")
        cv = make_tensor(c_np.shape, np.float32, device, True, c_np, "c")
        p = (x * w).softmax(-1)            # row kind, softmax
        r = (p * sc).exp()                 # scalar kind, exp: a little above 1
        u = (x * x) + r                    # same kind with both operands one tensor; >= 1
        out = ((u.log() + r) * cv).rsqrt()   # log, col kind, rsqrt (every step well-conditioned)
        return out, {"x": x, "w": w, "s": sc, "c": cv}

    (c_out, c_g), (h_out, h_g) = both(build, upstream)
    assert_chain_close(h_out[0], c_out[0], "forward", kernels=10)      # ten primitive kernels in the chain
    assert_chain_close(h_g["x"], c_g["x"], "x.grad", kernels=20)       # ... and as many backward
    for name, terms in (("w", B * T), ("s", B * T * C), ("c", C)):
        ref_g = c_g[name]
        bound = 1e-5 * np.sqrt(terms) * (np.abs(ref_g).max() + 1.0)
        assert np.abs(h_g[name] - ref_g).max() <= bound, (name, np.abs(h_g[name] - ref_g).max(), bound)
    # float64 check of the forward value, so that both devices agreeing is not the only evidence
    x64, w64 = x_np.astype(np.float64), w_np.astype(np.float64)
    a = x64 * w64
    p64 = np.exp(a - a.max(-1, keepdims=True))
    p64 /= p64.sum(-1, keepdims=True)
    r64 = np.exp(p64 * float(s_np[0]))
    want = ((np.log(x64 * x64 + r64) + r64) * c_np.astype(np.float64)) ** -0.5
    np.testing.assert_allclose(h_out[0], want, rtol=2e-5, atol=1e-6)


@pytest.mark.parametrize("bias_grad", [True, False])
def test_bias_gelu_in_a_graph_equals_add_then_gelu(bias_grad):
    """x.bias_gelu(b) against (x + b).gelu() -- the way the reference writes it
    (op.py:47-59, 241-245) -- on both devices, twice over the same arena; with the
    bias frozen the fused backward needs no workspace"""
    rng = np.random.default_rng(SEED + 41)
    B, T, C = 4, 50, 192
    x_np = rng.standard_normal((B, T, C), dtype=np.float32)
    b_np = rng.standard_normal(C).astype(np.float32)
    g_np = (1 + 0.1 * rng.standard_normal(C)).astype(np.float32)
    upstream = rng.standard_normal((B, T, C), dtype=np.float32)

    def build_with(fused):
        def build(device):
            x = make_tensor(x_np.shape, np.float32, device, True, x_np, "x")
            b = make_tensor(b_np.shape, np.float32, device, bias_grad, b_np, "b")
            g = make_tensor(g_np.shape, np.float32, device, True, g_np, "g")
            h = x.rms_norm(g)                       # an activation feeds the fused op
            out = h.bias_gelu(b) if fused else (h + b).gelu()
            return out, {"x": x, "b": b, "g": g} if bias_grad else {"x": x, "g": g}
        return build

    (c_out, c_g), (h_out, h_g) = both(build_with(True), upstream)
    (p_out, p_g), (q_out, q_g) = both(build_with(False), upstream)
    assert_fp32_close(h_out[0], c_out[0], "fused forward, hip vs cpu", rtol=2e-5, atol=2e-6)
    np.testing.assert_array_equal(c_out[0], p_out[0])         # the oracle's fused op IS the composition
    assert_fp32_close(h_out[0], q_out[0], "fused vs add->gelu on hip", rtol=2e-5, atol=2e-6)
    for name in c_g:
        terms = B * T if name in ("b", "g") else 1
        bound = 2e-5 * np.sqrt(terms) * (np.abs(c_g[name]).max() + 1.0)
        assert np.abs(h_g[name] - c_g[name]).max() <= bound, name
        assert np.abs(h_g[name] - q_g[name]).max() <= bound, name


def test_captured_graph_replays_match_eager():
    """Record forward + zero_grad + upstream copy + backward of the tiny GPT-2 chain
    once, replay it several times with eager work and synchronisations in between,
    and compare every replay with the eager result bit for bit."""
    rng = np.random.default_rng(SEED + 40)
    B, T, C, V = 4, 32, 64, 500
    ids_np = rng.integers(0, V, (B, T), dtype=np.int32)
    dev = "hip"
    rt = Runtime(device=dev)
    ids = make_tensor(ids_np.shape, np.int32, dev, False, ids_np)
    wte = make_tensor((V, C), np.float32, dev, True, (0.5 * rng.standard_normal((V, C))).astype(np.float32))
    wpe = make_tensor((T, C), np.float32, dev, True, (0.5 * rng.standard_normal((T, C))).astype(np.float32))
    g = make_tensor((C,), np.float32, dev, True, (1 + 0.1 * rng.standard_normal(C)).astype(np.float32))
    b = make_tensor((C,), np.float32, dev, True, (0.1 * rng.standard_normal(C)).astype(np.float32))
    up = make_tensor((B, T, C), np.float32, dev, False, rng.standard_normal((B, T, C)).astype(np.float32))
    out = GELUOp()(LayerNormOp(eps=1e-5)(EmbeddingSumOp()(ids, wte, wpe), g, b))
    rt.loss = out
    rt.build_topo(out)
    rt.bind_memory()
    up.storage = rt.allocator.alloc(up.shape, up.dtype)
    rt.backend.init(up)

    def step():
        rt.forward()
        rt.zero_grad()
        rt.backend._launch("copy_kernel", [up, out.grad], [up.numel * 4, 0])   # device-side upstream gradient
        rt.backward_graph()

    def read():
        rt.backend.synchronize()
        return [rt.backend.copy_to_host(t).copy() for t in (out, wte.grad, wpe.grad, g.grad, b.grad)]

    step()
    eager = read()
    graph = rt.capture(step)
    for replay in range(3):
        # eager work between replays: scribble over the outputs and the gradients
        for t in (out, wte.grad, g.grad):
            rt.backend.fill(t, float(replay + 1))
        rt.backend.synchronize()
        graph.launch()
        got = read()
        for a, e in zip(got, eager):
            np.testing.assert_array_equal(a, e, err_msg=f"replay {replay}")
    # calls that wait for the GPU are refused while recording, and the recording survives that
    rt.backend.capture_begin()
    with pytest.raises((RuntimeError, ValueError)):
        rt.backend.ctx.synchronize()
    rt.forward()
    g2 = rt.backend.capture_end()
    rt.backend.graph_launch(g2)
    rt.backend.synchronize()
    np.testing.assert_array_equal(rt.backend.copy_to_host(out), eager[0])
    rt.backend.graph_destroy(g2)
    graph.destroy()
    with pytest.raises(RuntimeError):
        graph.launch()
    rt.release()


@pytest.mark.parametrize("with_wpe", [False, True])
def test_ids_ordered_with_the_zero_fill(with_wpe):
    """zero_grad(order_ids=True) lets the id ordering ride with the zero fill of the table's gradient,
    and the forward pass then gathers with the plain kernel; without it the forward call orders the
    ids.  Same outputs and the same gradient bits either way, step after step with new ids."""
    rng = np.random.default_rng(SEED + 90)
    B, T, C, V = 8, 256, 96, 1000
    dev = "hip"
    results = {}
    for mode in ("execute", "protocol"):
        r2 = np.random.default_rng(SEED + 91)
        ids = make_tensor((B, T), np.int32, dev, False, r2.integers(0, V, (B, T), dtype=np.int32))
        wte = make_tensor((V, C), np.float32, dev, True, (0.5 * r2.standard_normal((V, C))).astype(np.float32))
        g = make_tensor((C,), np.float32, dev, True, np.ones(C, np.float32))
        if with_wpe:
            wpe = make_tensor((T, C), np.float32, dev, True, (0.5 * r2.standard_normal((T, C))).astype(np.float32))
            x0 = EmbeddingSumOp()(ids, wte, wpe)
        else:
            x0 = GatherOp()(ids, wte)
        out = RMSNormOp(eps=1e-6)(x0, g)
        rt = Runtime(device=dev)
        rt.loss = out
        rt.build_topo(out)
        rt.bind_memory()
        emb = x0.op
        steps = []
        for step in range(3):
            rt.backend.copy_from_host(ids, np.random.default_rng(SEED + 92 + step).integers(0, V, (B, T), dtype=np.int32))
            rt.zero_grad(order_ids=(mode == "execute"))
            assert emb.order_ready == (mode == "execute")
            rt.forward()
            rt.backend.fill(out.grad, 0.5)
            rt.backward_graph()
            rt.backend.synchronize()
            assert not emb.order_ready          # consumed by the backward kernel
            steps.append([rt.backend.copy_to_host(t).copy() for t in (out, wte.grad, g.grad)]
                         + ([rt.backend.copy_to_host(wpe.grad).copy()] if with_wpe else []))
        results[mode] = steps
        rt.release()
    for a, b in zip(results["execute"], results["protocol"]):
        for x, y in zip(a, b):
            np.testing.assert_array_equal(x, y)


def _launch_log(rt):
    """records the kernel names the runtime's backend launches from now on"""
    names = []
    plain = rt.backend._launch

    def logged(name, tensors, args):
        names.append(name)
        plain(name, tensors, args)
    rt.backend._launch = logged
    return names, lambda: setattr(rt.backend, "_launch", plain)


@pytest.mark.parametrize("with_wpe", [False, True])
@pytest.mark.parametrize("protocol", ["execute", "nowait", "manual", "graph"])
def test_table_gradient_cleared_by_rows_over_steps(with_wpe, protocol):
    """From the second step on zero_grad clears the rows of the last pass's ids in the table's
    gradient instead of filling the table; the gradients are those of a runtime that fills, bit
    for bit, step after step with new ids -- through execute (with and without the wait at the
    step's end), through the reference's manual protocol with the ids changed between zero_grad
    and forward, and through replays of a recorded execute."""
    B, T, C, V = 8, 256, 96, 1000
    dev = "hip"
    results = {}
    for row_reset in (True, False):
        r2 = np.random.default_rng(SEED + 101)
        ids = make_tensor((B, T), np.int32, dev, False, r2.integers(0, V, (B, T), dtype=np.int32))
        wte = make_tensor((V, C), np.float32, dev, True, (0.5 * r2.standard_normal((V, C))).astype(np.float32))
        g = make_tensor((C,), np.float32, dev, True, np.ones(C, np.float32))
        if with_wpe:
            wpe = make_tensor((T, C), np.float32, dev, True, (0.5 * r2.standard_normal((T, C))).astype(np.float32))
            x0 = EmbeddingSumOp()(ids, wte, wpe)
        else:
            x0 = GatherOp()(ids, wte)
        out = RMSNormOp(eps=1e-6)(x0, g)
        rt = Runtime(device=dev, row_reset=row_reset)
        rt.loss = out
        rt.grad_scale = 0.5
        rt.build_topo(out)
        rt.bind_memory()
        assert (x0.op.kept_ids is not None) == row_reset
        names, restore = _launch_log(rt)
        graph = None
        steps = []
        for step in range(4):
            new_ids = np.random.default_rng(SEED + 102 + step).integers(0, V, (B, T), dtype=np.int32)
            del names[:]
            if protocol == "manual":
                rt.zero_grad()
                rt.backend.copy_from_host(ids, new_ids)
                rt.forward()
                rt.backend.fill(out.grad, 0.5)
                rt.backward_graph()
            elif protocol == "graph" and step >= 2:
                rt.backend.copy_from_host(ids, new_ids)
                if graph is None:
                    graph = rt.capture(rt.execute)
                    assert ("embedding_grad_reset" in names) == row_reset
                graph.launch()
            else:
                rt.backend.copy_from_host(ids, new_ids)
                rt.execute(wait=(protocol != "nowait"))
            rt.backend.synchronize()
            if graph is None:
                assert ("embedding_grad_reset" in names) == (row_reset and step > 0), names
            dW = rt.backend.copy_to_host(wte.grad).copy()
            absent = np.ones(V, bool)
            absent[new_ids.reshape(-1)] = False
            assert not dW[absent].any(), f"step {step}: rows of ids that are not in this pass"
            steps.append([rt.backend.copy_to_host(t).copy() for t in (out, g.grad)] + [dW]
                         + ([rt.backend.copy_to_host(wpe.grad).copy()] if with_wpe else []))
        results[row_reset] = steps
        restore()
        if graph is not None:
            graph.destroy()
        rt.release()
    for a, b in zip(results[True], results[False]):
        for x, y in zip(a, b):
            np.testing.assert_array_equal(x, y)


def test_row_reset_falls_back_to_the_fill():
    """The rows to clear are known only while embedding nodes' backward passes are all that wrote the
    table's gradient since it was last zero: two micro-steps that accumulate or a host write into
    the gradient end in the plain fill.  A table that two embeddings share is cleared by both
    lists."""
    B, T, C, V = 4, 128, 64, 500
    dev = "hip"
    r2 = np.random.default_rng(SEED + 111)
    ids_a = make_tensor((B, T), np.int32, dev, False, r2.integers(0, V, (B, T), dtype=np.int32))
    ids_b = make_tensor((B, T), np.int32, dev, False, r2.integers(0, V, (B, T), dtype=np.int32))
    wte = make_tensor((V, C), np.float32, dev, True, (0.5 * r2.standard_normal((V, C))).astype(np.float32))
    g = make_tensor((C,), np.float32, dev, True, np.ones(C, np.float32))
    xa, xb = GatherOp()(ids_a, wte), GatherOp()(ids_b, wte)
    out = RMSNormOp(eps=1e-6)(AddOp()(xa, xb), g)
    rt = Runtime(device=dev)
    rt.loss = out
    rt.grad_scale = 0.25
    rt.build_topo(out)
    rt.bind_memory()
    names, restore = _launch_log(rt)

    def run(a, b):
        rt.backend.copy_from_host(ids_a, a)
        rt.backend.copy_from_host(ids_b, b)
        del names[:]
        rt.execute()
        rt.backend.synchronize()
        return rt.backend.copy_to_host(wte.grad).copy()

    def new_ids(k):
        r = np.random.default_rng(SEED + 112 + k)
        return r.integers(0, V, (B, T), dtype=np.int32), r.integers(0, V, (B, T), dtype=np.int32)

    def rows_of(*id_arrays):
        m = np.zeros(V, bool)
        for a in id_arrays:
            m[a.reshape(-1)] = True
        return m
    a0, b0 = new_ids(0)
    run(a0, b0)
    assert "embedding_grad_reset" not in names
    a1, b1 = new_ids(1)
    dW = run(a1, b1)
    assert names.count("embedding_grad_reset") == 2          # one list per embedding
    assert not dW[~rows_of(a1, b1)].any() and dW[rows_of(a1, b1)].any()
    # two micro-steps that accumulate: the union of their rows is in no list
    rt.accumulate_parameter_grads = True
    rt.zero_grad()
    a2, b2 = new_ids(2)
    run(a2, b2)
    a3, b3 = new_ids(3)
    dW = run(a3, b3)
    assert dW[rows_of(a2, b2) & ~rows_of(a3, b3)].any()      # rows of the first micro-step are still there
    del names[:]
    rt.zero_grad()
    rt.backend.synchronize()
    assert "embedding_grad_reset" not in names
    assert not rt.backend.copy_to_host(wte.grad).any()
    rt.accumulate_parameter_grads = False
    # a host write into the gradient
    a4, b4 = new_ids(4)
    run(a4, b4)
    rt.backend.copy_from_host(wte.grad, np.full((V, C), 3.0, np.float32))
    a5, b5 = new_ids(5)
    dW = run(a5, b5)
    assert "embedding_grad_reset" not in names
    assert not dW[~rows_of(a5, b5)].any()
    a6, b6 = new_ids(6)
    dW = run(a6, b6)
    assert names.count("embedding_grad_reset") == 2
    assert not dW[~rows_of(a6, b6)].any()
    restore()
    rt.release()
