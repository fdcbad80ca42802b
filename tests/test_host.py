"""Host-side logic and the native library's load / export surface, no GPU needed."""
import ctypes
import re
from pathlib import Path

import numpy as np
import pytest

from autograd_amd import capi
from autograd_amd.device import Device
from autograd_amd.op import (AddLayerNormOp, AddOp, AddRMSNormOp, EmbeddingSumOp, GatherOp, GELUOp,
                             LayerNormOp, RMSNormOp, RopeOp, SwiGLUOp)
from autograd_amd.runtime import ExecutionPlan, MemoryPlanner, Runtime, bind_plans
from autograd_amd.tensor import Tensor
from autograd_amd.utils import BF16, bf16_bits, broadcast_shape, contiguous_strides, f32_bits, itemsize
from oracle import cpu_device

ROOT = Path(__file__).resolve().parents[1]
cpu_device.register()


def T(shape, dtype=np.float32, requires_grad=True, val=None):
    return Tensor(shape=shape, dtype=dtype, device="cpu", requires_grad=requires_grad, init_val=val)


# ---- native library: loads without a GPU and exports what the header declares ----
def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "autograd_hip.h").read_text()
    declared = set(re.findall(r"\b(agrad_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 35
    lib = ctypes.CDLL(str(capi.LIB_PATH))
    missing = [name for name in sorted(declared) if not hasattr(lib, name)]
    assert not missing, f"declared but not exported: {missing}"
    assert declared == set(capi.SIGNATURES), declared ^ set(capi.SIGNATURES)


def test_header_compiles_as_plain_c(tmp_path):
    """include/autograd_hip.h is a C header: gcc -std=c99 -pedantic accepts a
    translation unit that includes it and takes the address of every declared function"""
    import subprocess
    header = (ROOT / "include" / "autograd_hip.h").read_text()
    names = sorted(set(re.findall(r"\b(agrad_[a-z0-9_]+)\s*\(", header)) - {"agrad_ctx"})
    src = tmp_path / "use_header.c"
    src.write_text('#include "autograd_hip.h"\n' + "void* table[] = {\n"
                   + "".join(f"    (void*)(unsigned long){n},\n" for n in names) + "};\n")
    proc = subprocess.run(["gcc", "-std=c99", "-Wall", "-pedantic", "-fsyntax-only", f"-I{ROOT / 'include'}", str(src)],
                          capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr
    assert len(names) >= len(capi.SIGNATURES)


def test_index_divider_matches_the_machines_division(tmp_path):
    """The kernels split a flat index into (row, column) with a multiply-high divider prepared
    on the host (csrc/fastdiv.hpp); tests/c_abi/fastdiv_check.cpp, compiled here with g++,
    compares it with / and % over strides of all 32-bit dividends, edges and random pairs."""
    import subprocess
    exe = tmp_path / "fastdiv_check"
    proc = subprocess.run(["g++", "-O2", "-std=c++17", f"-I{ROOT / 'autograd_amd' / 'csrc'}",
                           str(ROOT / "tests" / "c_abi" / "fastdiv_check.cpp"), "-o", str(exe)], capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr
    proc = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout + proc.stderr


def test_library_reports_errors_without_gpu_or_kernel():
    lib = capi.load_library()
    assert lib.agrad_kernel_count() == 47
    names = [lib.agrad_kernel_name(i).decode() for i in range(lib.agrad_kernel_count())]
    for n in ("layernorm_forward", "layernorm_backward_kernel", "rmsnorm_forward", "rmsnorm_backward",
              "gelu_forward_kernel", "gelu_backward_kernel", "swiglu_forward_kernel", "rope_qk_inplace",
              "gather_forward_kernel", "gather_backward_kernel", "pos_emb_grad", "fill_scalar_kernel",
              "fp32_to_bf16", "add_residual_forward"):
        assert n in names
    assert lib.agrad_kernel_signature(b"nope") is None
    assert b"eps_bits" in lib.agrad_kernel_signature(b"layernorm_forward")
    assert lib.agrad_kernel_name(-1) is None and lib.agrad_kernel_name(999) is None
    # null context is refused, not dereferenced
    assert lib.agrad_synchronize(None) == capi.EINVAL
    assert b"null context" in lib.agrad_last_error()
    assert lib.agrad_dispatch(None, b"x", None, None, 0, None, 0, 0, 0, 0, 0) == capi.EINVAL


def test_pybind_module_imports_and_hip_device_is_loud_without_gpu():
    from autograd_amd import hip_ext
    assert hip_ext.F32 == 0 and hip_ext.BF16 == 1
    if hip_ext.device_count() == 0:
        with pytest.raises(RuntimeError):
            hip_ext.HipContext(0)
        with pytest.raises(RuntimeError):
            Device.get_backend("hip")       # no silent CPU path


def test_device_registry():
    with pytest.raises(ValueError):
        Device.get_allocator("mps")
    with pytest.raises(ValueError):
        Device.get_backend("cuda")
    assert Device.get_backend("cpu") is Device.get_backend("cpu")
    assert Device.get_allocator("cpu").device == "cpu"


# ---- utils ------------------------------------------------------------------------
def test_utils():
    assert contiguous_strides((2, 3, 4)) == (12, 4, 1)
    assert broadcast_shape((4, 1, 3), (5, 3)) == (4, 5, 3)
    with pytest.raises(RuntimeError):
        broadcast_shape((2, 3), (4, 3))
    assert f32_bits(1.0) == 0x3F800000 and f32_bits(1e-5) == 0x3727C5AC
    assert bf16_bits(1.0) == 0x3F80 and bf16_bits(float("inf")) == 0x7F80 and bf16_bits(float("nan")) & 0x7FC0 == 0x7FC0
    assert itemsize(BF16) == 2 and itemsize(np.float32) == 4 and itemsize(np.int32) == 4


# ---- ops: shape inference and error behaviour (op.py:219-267) ------------------------
def test_op_shapes_and_errors():
    ids = T((2, 5), np.int32, False)
    w = T((11, 8))
    assert GatherOp()(ids, w).shape == (2, 5, 8)
    with pytest.raises(ValueError):
        GatherOp()(T((10,), np.int32, False), w)
    with pytest.raises(ValueError):
        GatherOp()(ids, T((11, 8, 2)))
    x = T((2, 5, 8))
    g, b = T((8,)), T((8,))
    y = LayerNormOp(eps=1e-5)(x, g, b)
    assert y.shape == x.shape and y.op.op.eps == 1e-5 and y.op.inputs == (x, g, b)
    assert LayerNormOp().eps == 1e-6          # the op's default (op.py:249)
    assert x.layer_norm(g, b).op.op.eps == 1e-5   # the Tensor sugar's default (tensor.py:97)
    with pytest.raises(ValueError):
        LayerNormOp()(x, T((7,)), T((7,)))
    with pytest.raises(ValueError):
        LayerNormOp()(x, g, T((7,)))
    with pytest.raises(ValueError):
        RMSNormOp()(x, T((7,)))
    assert RMSNormOp()(x).shape == x.shape and len(RMSNormOp()(x).op.inputs) == 1
    assert SwiGLUOp()(x).shape == (2, 5, 4)
    with pytest.raises(ValueError):
        SwiGLUOp()(T((2, 5, 7)))
    h, yy = AddLayerNormOp()(x, T((2, 5, 8)), g, b)
    assert h.op is yy.op and h.op.outputs == (h, yy)
    with pytest.raises(ValueError):
        AddRMSNormOp()(x, T((2, 5, 4)))
    q, k = T((2, 5, 4, 8)), T((2, 5, 2, 8))
    c, s = T((16, 4), requires_grad=False), T((16, 4), requires_grad=False)
    q2, k2 = RopeOp(rope_sign=-1)(q, k, c, s)
    assert q2.shape == q.shape and k2.shape == k.shape
    with pytest.raises(ValueError):
        RopeOp(rope_sign=0)
    with pytest.raises(ValueError):
        RopeOp()(q, k, T((3, 4)), T((3, 4)))     # table shorter than T
    assert EmbeddingSumOp()(ids, w, T((5, 8))).shape == (2, 5, 8)
    with pytest.raises(ValueError):
        EmbeddingSumOp()(ids, w, T((4, 8)))
    assert (x + x).op.op.op_name == "Add" and x.gelu().op.op.op_name == "GELU"
    # requires_grad propagates; gather ignores the integer operand
    assert not GatherOp()(ids, T((11, 8), requires_grad=False)).requires_grad


def test_primitive_op_shapes_and_errors():
    """Mul's broadcast kinds are the reference's (utils.py:134-143); Softmax takes any axis of its input"""
    from autograd_amd.utils import mul_bcast_kind
    x = T((2, 3, 8))
    assert (x * T((2, 3, 8))).shape == (2, 3, 8) and (x * T((8,))).shape == (2, 3, 8)
    assert (x * T((2, 3, 1))).shape == (2, 3, 8) and (x * T((1,))).op.op.op_name == "Mul"
    assert [mul_bcast_kind((2, 3, 8), s) for s in ((2, 3, 8), (8,), (2, 3, 1), (1,), ())] == \
        ["same", "row", "col", "scalar", "scalar"]
    with pytest.raises(RuntimeError):
        x * T((3, 8))                  # no kernel for a middle-axes broadcast
    with pytest.raises(RuntimeError):
        T((8,)) * x                    # the broadcast operand goes second
    assert x.exp().shape == x.log().shape == x.rsqrt().shape == x.shape
    assert x.softmax(-1).op.op.dim == -1 and x.softmax(2).shape == x.shape
    assert x.softmax(1).op.op.axis(x) == 1 and x.softmax(-3).op.op.axis(x) == 0      # any axis (backend.py:356)
    with pytest.raises(ValueError):
        x.softmax(3)
    assert x.exp().op.op.save_for_backward((x,), ("y",)) == ["y"]
    assert x.log().op.op.save_for_backward((x,), ("y",)) == [x]


def test_layout_ops_shapes_strides_and_errors():
    """View / Reshape / Permute / Transpose are views with the reference's shape and
    stride rules (op.py:89-171, utils.py:85-109); only Contiguous reads through strides"""
    x = T((2, 3, 4, 5))
    assert x.strides == (60, 20, 5, 1) and x.is_contiguous
    p = x.permute(0, 2, 1, 3)
    assert p.shape == (2, 4, 3, 5) and p.strides == (60, 5, 20, 1) and not p.is_contiguous
    t = x.transpose(1, 3)
    assert t.shape == (2, 5, 4, 3) and t.strides == (60, 1, 5, 20) and not t.is_contiguous
    assert p.transpose(-1, -2).strides == (60, 5, 1, 20)          # views compose
    r = x.reshape(6, -1)
    assert r.shape == (6, 20) and r.strides == (20, 1) and r.is_contiguous
    assert x.view(-1).shape == (120,) and x.view(2, 60).op.op.op_name == "View"
    c = p.contiguous()
    assert c.shape == p.shape and c.is_contiguous and c.strides == contiguous_strides(p.shape)
    for bad in (lambda: x.reshape(7, -1), lambda: x.reshape(-1, -1), lambda: x.reshape(3, 5), lambda: x.reshape(0, -1)):
        with pytest.raises(ValueError):
            bad()
    with pytest.raises(ValueError):
        x.permute(0, 1, 1, 3)
    with pytest.raises(RuntimeError):
        p.reshape(2, 60)            # reshape view requires contiguous input (utils.py:106-107)
    with pytest.raises(RuntimeError):
        p.view(2, 60)
    with pytest.raises(RuntimeError):
        p.gelu()                    # compute kernels read dense tensors
    with pytest.raises(RuntimeError):
        AddOp()(p, p)
    assert p.contiguous().gelu().shape == p.shape
    assert not T((2, 3), requires_grad=False).permute(1, 0).requires_grad


def test_layout_ops_in_a_graph_on_the_oracle_device():
    """x -> reshape -> permute -> contiguous -> gelu and a transpose branch of a
    parameter: forward values and gradients against numpy written out directly;
    views own no arena memory and an in-place consumer never writes through one"""
    rng = np.random.default_rng(5)
    B, Tn, H, D = 2, 6, 3, 4
    x_np = rng.standard_normal((B, Tn, H * D)).astype(np.float32)
    w_np = rng.standard_normal((D, Tn)).astype(np.float32)
    up = rng.standard_normal((B, H, Tn, D)).astype(np.float32)
    x, w = T((B, Tn, H * D), val=x_np), T((D, Tn), val=w_np)
    a = x.gelu()                                     # an activation, so that its views live in the arena
    heads = a.reshape(B, Tn, H, D).permute(0, 2, 1, 3)
    dense = heads.contiguous()
    out = dense + w.transpose(0, 1).contiguous()     # [Tn, D] broadcast over [B, H]
    rt = Runtime(device="cpu")
    rt.loss = out
    rt.build_topo(out)
    rt.bind_memory()
    rt.forward()
    from oracle import cpu_ops as K
    a_np = K.gelu_forward(x_np)
    want = np.transpose(a_np.reshape(B, Tn, H, D), (0, 2, 1, 3)) + w_np.T
    np.testing.assert_array_equal(rt.backend.copy_to_host(out), want)
    # the reshape and permute outputs are the gelu output's bytes
    assert np.shares_memory(heads.storage.data, a.storage.data)
    assert heads.grad.storage.data.shape == heads.shape       # a dense gradient of its own
    rt.zero_grad()
    rt.backend.copy_from_host(out.grad, up)
    rt.backward_graph()
    da = np.transpose(up, (0, 2, 1, 3)).reshape(B, Tn, H * D)
    dx = np.zeros_like(x_np)
    K.gelu_backward_into(x_np, np.ascontiguousarray(da), dx)
    np.testing.assert_array_equal(rt.backend.copy_to_host(x.grad), dx)
    np.testing.assert_allclose(rt.backend.copy_to_host(w.grad), up.sum((0, 1)).T, rtol=1e-5, atol=1e-6)
    # second run: same numbers
    rt.zero_grad()
    rt.forward()
    rt.backend.copy_from_host(out.grad, up)
    rt.backward_graph()
    np.testing.assert_array_equal(rt.backend.copy_to_host(x.grad), dx)


def _plan_graph(device, w, g, B, Tn, forward_only, owns_params=None):
    ids = Tensor(shape=(B, Tn), dtype=np.int32, device=device, requires_grad=False, name=f"ids_{Tn}")
    x = ids.gather(w)
    h, y = x.add_rms_norm(x.gelu(), g)
    out = (h + y).reshape(B * Tn, -1)
    rt = Runtime(device=device, forward_only=forward_only,
                 owns_params=(not forward_only) if owns_params is None else owns_params)
    return ExecutionPlan(runtime=rt, input_ids=ids, output=out, seq_len=Tn, mode="eval" if forward_only else "train")


def test_execution_plans_share_one_arena_on_the_oracle_device():
    """a training plan and a forward-only plan at another length over the same
    parameters, prepared separately and bound into one arena sized for the larger
    (ExecutionPlan.prepare / bind_to, runtime.py:857-892; engine.py:133-170): each
    gives what a runtime of its own gives"""
    rng = np.random.default_rng(11)
    V, C = 29, 16
    w_np = rng.standard_normal((V, C)).astype(np.float32)
    g_np = (1 + 0.1 * rng.standard_normal(C)).astype(np.float32)
    ids_train = rng.integers(0, V, (2, 8), dtype=np.int32)
    ids_eval = rng.integers(0, V, (1, 5), dtype=np.int32)

    def solo(ids_np, forward_only):
        w, g = T((V, C), val=w_np), T((C,), val=g_np)
        plan = _plan_graph("cpu", w, g, *ids_np.shape, forward_only, owns_params=True)
        rt = plan.runtime
        rt.loss = plan.output
        rt.build_topo(plan.output)
        rt.bind_memory()
        rt.is_compiled = True
        rt.backend.copy_from_host(plan.input_ids, ids_np)
        if forward_only:
            return plan.forward(), None
        plan.backward()
        return rt.backend.copy_to_host(plan.output), rt.backend.copy_to_host(w.grad)

    want_train, want_dw = solo(ids_train, False)
    want_eval, _ = solo(ids_eval, True)

    w, g = T((V, C), val=w_np), T((C,), val=g_np)
    train = _plan_graph("cpu", w, g, 2, 8, False).prepare()       # owns the parameters
    evalp = _plan_graph("cpu", w, g, 1, 5, True).prepare()        # borrows them
    assert train.runtime.arena_bytes > evalp.runtime.arena_bytes > 0
    with pytest.raises(RuntimeError):
        train.forward()                                           # planned, not bound
    arena = bind_plans([train, evalp])
    assert arena.nbytes == train.runtime.arena_bytes
    assert train.runtime.unified_arena is arena and evalp.runtime.unified_arena is arena
    for _ in range(2):                                            # alternate: each plan re-runs cleanly
        train.set_inputs(ids_train)
        train.backward()
        np.testing.assert_array_equal(train.runtime.backend.copy_to_host(train.output), want_train)
        np.testing.assert_array_equal(train.runtime.backend.copy_to_host(w.grad), want_dw)
        evalp.set_inputs(ids_eval)
        np.testing.assert_array_equal(evalp.forward(), want_eval)
    with pytest.raises(ValueError):
        evalp.backward()
    with pytest.raises(ValueError):
        evalp.set_targets(ids_eval)
    small = train.runtime.allocator.empty((evalp.runtime.arena_bytes,), np.uint8)
    with pytest.raises(RuntimeError):
        train.bind_to(small)


# ---- planner ------------------------------------------------------------------------
def test_memory_planner_first_fit():
    p = MemoryPlanner()
    assert p.alloc("a", 100) == 0 and p.alloc("b", 300) == 256 and p.alloc("c", 10) == 768
    p.free("a")
    assert p.alloc("d", 200) == 0           # reuses the lowest hole that fits
    p.free("b")
    assert p.alloc("e", 512) == 256         # hole of 512 between d and c
    assert p.alloc("f", 1) == 1024
    assert p.peak == 1280 and p.alloc("a", 5) == 0   # known keys keep their offset
    for off in p.offsets.values():
        assert off % 256 == 0


def test_planner_property_no_live_overlap():
    rng = np.random.default_rng(7)
    for _ in range(20):
        n = 40
        start = rng.integers(0, 30, n)
        length = rng.integers(1, 10, n)
        size = rng.integers(1, 5000, n)
        p = MemoryPlanner()
        end = start + length
        for step in range(int(end.max()) + 1):
            for i in range(n):
                if end[i] == step - 1:
                    p.free(i)
            for i in range(n):
                if start[i] == step:
                    p.alloc(i, int(size[i]))
        for i in range(n):
            for j in range(i + 1, n):
                if start[i] <= end[j] and start[j] <= end[i]:       # lifetimes intersect
                    a0, a1 = p.offsets[i], p.offsets[i] + size[i]
                    b0, b1 = p.offsets[j], p.offsets[j] + size[j]
                    assert a1 <= b0 or b1 <= a0
        assert p.peak >= max(p.offsets[i] + size[i] for i in range(n))


def test_runtime_arena_views_and_execution_on_oracle_device():
    rng = np.random.default_rng(3)
    B, Tn, C, V = 2, 6, 16, 23
    ids_np = rng.integers(0, V, (B, Tn), dtype=np.int32)
    w_np = rng.standard_normal((V, C)).astype(np.float32)
    ids, w = T((B, Tn), np.int32, False, ids_np), T((V, C), val=w_np)
    g, b = T((C,), val=np.ones(C, np.float32)), T((C,), val=np.zeros(C, np.float32))
    x = ids.gather(w)
    h, y = x.add_layer_norm(x.gelu(), g, b)
    out = h + y
    rt = Runtime(device="cpu")
    rt.backward(out, grad_scale=1.0)
    # every activation and activation gradient is a view of the one arena
    arena = rt.unified_arena.data
    lo, hi = arena.ctypes.data, arena.ctypes.data + arena.nbytes
    seen = []
    for node in rt.topo:
        for t in node.outputs:
            for u in (t, t.grad):
                if u is None:
                    continue
                a = u.storage.data
                assert lo <= a.ctypes.data and a.ctypes.data + a.nbytes <= hi
                assert (a.ctypes.data - lo) % 256 == 0
                seen.append(u)
    assert rt.arena_bytes == arena.nbytes and rt.arena_bytes % 256 == 0
    # gradients flow: d(out)/dw is non-zero exactly on the gathered rows
    dw = rt.backend.copy_to_host(w.grad)
    used = np.zeros(V, bool)
    used[ids_np.ravel()] = True
    assert np.abs(dw[used]).sum() > 0 and not dw[~used].any()
    # a second execute gives the same numbers (grads are re-zeroed)
    rt.backward(out, grad_scale=1.0)
    np.testing.assert_array_equal(rt.backend.copy_to_host(w.grad), dw)
    # an output nobody consumes gets no gradient tensor
    h2, y2 = x.add_rms_norm(x.gelu())
    rt2 = Runtime(device="cpu")
    rt2.build_topo(y2)
    assert h2.grad is None and y2.grad is not None


def test_partly_first_written_parameter_grads_are_all_zero_filled():
    """Two LayerNorms share gamma and have their own betas.  The backward kernel has one
    store-or-accumulate choice for (dgamma, dbeta), and gamma's gradient is first written
    by the LATER node (backward runs in reverse), so the earlier node must accumulate --
    and then its own beta's gradient has to be zero-filled like everything else."""
    rng = np.random.default_rng(5)
    x_np = rng.standard_normal((4, 8, 16)).astype(np.float32)
    g_np = (1 + 0.1 * rng.standard_normal(16)).astype(np.float32)
    x = T(x_np.shape, val=x_np)
    gamma = T((16,), val=g_np)
    beta_a, beta_b = T((16,), val=np.zeros(16, np.float32)), T((16,), val=np.zeros(16, np.float32))
    a = LayerNormOp(eps=1e-5)(x, gamma, beta_a)
    out = LayerNormOp(eps=1e-5)(a.gelu(), gamma, beta_b)
    rt = Runtime(device="cpu")
    rt.fuse_grad_zeroing = True        # the first-writer analysis as the hip device runs it (planning only)
    rt.loss = out
    rt.build_topo(out)
    rt.plan_memory()
    first, last = rt.topo[0], rt.topo[-1]
    assert first.inputs[2] is beta_a and last.inputs[2] is beta_b
    # the last node writes gamma.grad and beta_b.grad first: both may be stored
    assert {id(gamma.grad), id(beta_b.grad)} <= last.overwrite_grads
    # the first node accumulates onto gamma.grad, so beta_a.grad may not skip its fill
    assert id(gamma.grad) not in first.overwrite_grads
    assert id(beta_a.grad) not in first.overwrite_grads
    assert id(beta_a.grad) not in rt._stored_leaf_grads
    assert id(x.grad) not in first.overwrite_grads        # x is a leaf of the same node: same treatment


def test_inplace_op_leaves_a_tensor_its_producer_saved_alone():
    """Rope rotates its input in place when nobody else reads it -- but Exp's backward
    reads Exp's OUTPUT, so q = exp(x) must keep its values and Rope gets its own memory."""
    rng = np.random.default_rng(6)
    B, Tn, H, D = 1, 4, 2, 8
    x = T((B, Tn, H, D), val=rng.standard_normal((B, Tn, H, D)).astype(np.float32))
    k = T((B, Tn, H, D), val=rng.standard_normal((B, Tn, H, D)).astype(np.float32))
    from oracle import cpu_ops
    cos_np, sin_np = cpu_ops.rope_tables(Tn, D, 1e4)
    cos, sin = T(cos_np.shape, requires_grad=False, val=cos_np), T(sin_np.shape, requires_grad=False, val=sin_np)
    q = x.exp()
    kk = k.gelu()                      # GELU saves its input, not kk: kk may be rotated in place
    q2, k2 = RopeOp(rope_sign=1)(q, kk, cos, sin)
    out = q2 + k2
    rt = Runtime(device="cpu")
    rt.loss = out
    rt.build_topo(out)
    rt._resolve_aliases()
    assert id(q2) not in rt._alias_of
    assert rt._alias_of.get(id(k2)) is kk
    fwd_only = Runtime(device="cpu", forward_only=True)
    fwd_only.loss = out
    fwd_only.build_topo(out)
    fwd_only._resolve_aliases()
    assert fwd_only._alias_of.get(id(q2)) is q       # nothing is read back without a backward pass


def test_runtime_rejects_ops_without_kernels():
    class Bare(GELUOp):
        pass
    x = T((2, 4), val=np.zeros((2, 4), np.float32))
    y = Bare()(x)
    with pytest.raises(RuntimeError):
        Runtime(device="cpu").build_topo(y)      # lookup is by exact type (backend.py:4938-4950)


def test_adamw_host_logic_on_oracle_device():
    """AdamW over a runtime on the oracle device: per-parameter dispatches, decay on
    matrices only, step-size bookkeeping, clip coefficient (optimizer.py:443-500)."""
    import math
    from autograd_amd.optimizer import AdamW
    from oracle import cpu_ops as K
    rng = np.random.default_rng(5)
    B, Tn, C, V = 2, 6, 16, 23
    ids = T((B, Tn), np.int32, False, rng.integers(0, V, (B, Tn), dtype=np.int32))
    w = T((V, C), val=rng.standard_normal((V, C)).astype(np.float32))
    g = T((C,), val=np.ones(C, np.float32))
    b = T((C,), val=np.zeros(C, np.float32))
    out = ids.gather(w).layer_norm(g, b).gelu()
    rt = Runtime(device="cpu")
    rt.backward(out, grad_scale=1.0)
    with pytest.raises(ValueError):
        AdamW([w], state_mode="4bit", runtime=rt)
    with pytest.raises(NotImplementedError):
        AdamW([w], state_mode="mini", runtime=rt)
    lr, betas, eps, wd = 1e-2, (0.9, 0.95), 1e-8, 0.1
    opt = AdamW([w, g, b, ids], lr=lr, betas=betas, eps=eps, weight_decay=wd, runtime=rt)
    assert len(opt.params) == 3                       # ids needs no gradient
    assert [d[5] for d in opt.dispatches] == [V * C, 0, 0]
    clip = opt.build_grad_clip()
    want = {k: rt.backend.copy_to_host(t) for k, t in (("w", w), ("g", g), ("b", b))}
    mom = {k: (np.zeros_like(a), np.zeros_like(a)) for k, a in want.items()}
    for t in range(1, 3):
        rt.backward(out, grad_scale=1.0)
        grads = {k: rt.backend.copy_to_host(p.grad) for k, p in (("w", w), ("g", g), ("b", b))}
        norm, coef = clip(0.5)
        total = math.sqrt(sum(float((a.astype(np.float64) ** 2).sum()) for a in grads.values()))
        assert norm == pytest.approx(total, rel=1e-6) and coef == pytest.approx(min(1.0, 0.5 / (total + 1e-6)))
        opt.step()
        lr_t = lr * math.sqrt(1 - betas[1] ** t) / (1 - betas[0] ** t)
        for k, p in (("w", w), ("g", g), ("b", b)):
            K.adamw_step(want[k], grads[k], *mom[k], lr, lr_t, betas[0], betas[1], eps, wd if p.ndim > 1 else 0.0)
            np.testing.assert_array_equal(rt.backend.copy_to_host(p), want[k])
    assert opt.t == 2
    opt.zero_grad()
    assert not rt.backend.copy_to_host(w.grad).any()


def test_adamw_8bit_state_on_the_oracle_device():
    """AdamW(state_mode="8bit") drives the oracle device through the same calls as the hip
    one: large parameters get byte moments and per-block scales, small ones fp32 moments
    (optimizer.py:205-222); its code books are the reference's; "mini" is refused"""
    from autograd_amd.optimizer import AdamW, build_dynamic_map
    from oracle import cpu_ops as K
    for signed in (True, False):
        np.testing.assert_array_equal(build_dynamic_map(signed), K.dynamic_map(signed))
    rng = np.random.default_rng(21)
    V, C = 80, 64
    w = T((V, C), val=rng.standard_normal((V, C)).astype(np.float32))
    g = T((C,), val=np.ones(C, np.float32))
    ids = Tensor(shape=(2, 9), dtype=np.int32, device="cpu", requires_grad=False,
                 init_val=rng.integers(0, V, (2, 9), dtype=np.int32))
    out = ids.gather(w).rms_norm(g)
    rt = Runtime(device="cpu")
    rt.loss = out
    rt.build_topo(out)
    rt.bind_memory()
    opt = AdamW([w, g], lr=1e-2, weight_decay=0.1, runtime=rt, state_mode="8bit")
    assert [d[0] for d in opt.dispatches] == ["q8", "fp32"]
    assert opt.m[0].data.dtype == np.uint8 and opt.m[0].data.size == V * C and opt.dispatches[0][5].data.size == V * C // 256
    before = rt.backend.copy_to_host(w).copy()
    up = rng.standard_normal((2, 9, C)).astype(np.float32)
    for _ in range(2):
        rt.forward()
        rt.zero_grad()
        rt.backend.copy_from_host(out.grad, up)
        rt.backward_graph()
        opt.step()
    after = rt.backend.copy_to_host(w)
    touched = np.unique(rt.backend.copy_to_host(ids))
    moved = np.abs(after - before * np.float32(1 - 1e-2 * 0.1) ** 2).max(axis=1)
    assert (moved[touched] > 5e-3).all()                       # rows with a gradient took Adam-sized steps
    rest = np.setdiff1d(np.arange(V), touched)
    assert (moved[rest] < 1e-6).all()                          # the others only decayed
    with pytest.raises(NotImplementedError):
        AdamW([w, g], runtime=rt, state_mode="mini")


def test_hip_backend_refuses_a_gradient_type_no_kernel_can_write():
    """fp32 values with a bf16 gradient are for embedding tables, norm parameters and biases; the
    second operand of a Mul is refused when the graph is planned, not corrupted when it runs
    (checked on the planning hook alone: no device is needed)"""
    from autograd_amd.backend import HipBackend
    from autograd_amd.utils import BF16
    backend = HipBackend.__new__(HipBackend)          # no context: plan-time checks only
    x = Tensor(shape=(4, 8), dtype=np.float32, device="hip", requires_grad=True)
    bias = Tensor(shape=(8,), dtype=np.float32, device="hip", requires_grad=True, grad_dtype=BF16)
    for t in (x, bias):
        t.grad = Tensor(shape=t.shape, dtype=t.grad_dtype, device="hip", requires_grad=False)
    backend._check_gradient_storage((x + bias).op)                # a bias under a broadcast Add may
    out = x * bias
    with pytest.raises(RuntimeError, match="another type"):
        backend._check_gradient_storage(out.op)                   # Mul's second operand may not
    gamma = Tensor(shape=(8,), dtype=np.float32, device="hip", requires_grad=True, grad_dtype=BF16)
    gamma.grad = Tensor(shape=(8,), dtype=BF16, device="hip", requires_grad=False)
    backend._check_gradient_storage(x.rms_norm(gamma).op)         # a norm parameter may
