"""Cross-entropy on the GPU against the CPU restatement of
cpu_crossentropy_forward / backward (backend.py:489-524), through the C ABI and
through the runtime.  fp32: rtol 1e-5 / atol 1e-6; bf16 logits: 1e-2 relative on
the gradient (loss, log-sum-exp and dloss are fp32 on both sides)."""
import ctypes as C

import numpy as np
import pytest

from autograd_amd import capi
from autograd_amd.op import CrossEntropyLossOp
from autograd_amd.runtime import Runtime
from autograd_amd.tensor import Tensor
from oracle import closed_form as cf
from oracle import cpu_device
from oracle import cpu_ops as K
from tests.helpers import assert_bf16_close, assert_fp32_close, from_bf16_bits, to_bf16_bits

pytestmark = pytest.mark.gpu
cpu_device.register()


def vp(d, off=0):
    return C.c_void_p(d.ptr + off) if d is not None else None


def run_ce(ctx, x_store, labels, dloss, dtype, use_lse=True, dx_init=None, flags=0, offset_elems=0):
    rows, V = labels.size, x_store.shape[-1]
    esz = x_store.dtype.itemsize
    pad = np.zeros(offset_elems, x_store.dtype)
    dx_ = ctx.upload(np.concatenate([pad, x_store.reshape(-1)]))
    dl = ctx.upload(labels.reshape(-1).astype(np.int32))
    loss = ctx.upload(np.full(rows, -7.0, np.float32))
    lse = ctx.upload(np.full(rows, -7.0, np.float32))
    dg = ctx.upload(dloss.reshape(-1).astype(np.float32))
    init = dx_init if dx_init is not None else np.full(x_store.shape, 3, x_store.dtype)
    dout = ctx.upload(np.concatenate([pad, init.reshape(-1)]))
    off = offset_elems * esz
    ctx.call("agrad_cross_entropy_forward", dtype, vp(dx_, off), vp(dl), vp(loss), vp(lse) if use_lse else None, rows, V)
    ctx.call("agrad_cross_entropy_backward", dtype, vp(dx_, off), vp(dl), vp(dg), vp(lse) if use_lse else None,
             vp(dout, off), rows, V, flags)
    ctx.synchronize()
    out = loss.download(), lse.download(), dout.download()[offset_elems:].reshape(x_store.shape)
    for d in (dx_, dl, loss, lse, dg, dout):
        d.free()
    return out


@pytest.mark.parametrize("rows,V", [(1, 1), (3, 7), (5, 64), (4, 1000), (6, 4099), (2, 50257), (3, 32768)])
@pytest.mark.parametrize("use_lse", [True, False])
def test_cross_entropy_fp32(ctx, rows, V, use_lse):
    rng = np.random.default_rng(90 + V)
    x = (4.0 * rng.standard_normal((rows, V))).astype(np.float32)
    labels = rng.integers(0, V, rows, dtype=np.int32)
    dloss = rng.standard_normal(rows).astype(np.float32)
    loss, lse, dx = run_ce(ctx, x, labels, dloss, capi.F32, use_lse)
    assert_fp32_close(loss, K.cross_entropy_forward(x, labels), "loss")
    assert np.abs(loss - cf.cross_entropy(x, labels)).max() <= 2e-6 * max(1.0, np.abs(loss).max())
    if use_lse:
        from scipy.special import logsumexp
        assert np.abs(lse - logsumexp(x.astype(np.float64), axis=-1)).max() <= 2e-6 * max(1.0, np.abs(lse).max())
    ref = np.zeros_like(x)
    K.cross_entropy_backward_into(x, labels, dloss, ref)
    assert_fp32_close(dx, ref, "dlogits")
    assert np.abs(dx.sum(-1, dtype=np.float64)).max() <= 1e-5 * max(1.0, np.abs(dloss).max())


def test_cross_entropy_unaligned_rows_accumulate_and_extremes(ctx):
    rng = np.random.default_rng(95)
    rows, V = 5, 1003                       # odd row length: rows start at every alignment
    x = (3.0 * rng.standard_normal((rows, V))).astype(np.float32)
    x[1, 17] = 80.0                          # one class dominates
    x[2, :] = -60.0                          # uniform far below zero
    x[3, 5] = -np.inf                        # a masked class
    labels = np.array([0, 17, 9, 1002, 500], np.int32)
    dloss = np.array([1.0, -2.0, 0.5, 1.5, 0.0], np.float32)
    base = rng.standard_normal((rows, V)).astype(np.float32)
    for off in (0, 1, 3):                   # tensor start 0 / 4 / 12 bytes past a 16-byte boundary
        loss, _, dx = run_ce(ctx, x, labels, dloss, capi.F32, True, dx_init=base, flags=capi.ACC_INPUT_GRAD,
                             offset_elems=off)
        assert_fp32_close(loss, K.cross_entropy_forward(x, labels), f"loss off={off}")
        ref = base.copy()
        K.cross_entropy_backward_into(x, labels, dloss, ref)
        assert_fp32_close(dx, ref, f"dlogits off={off}")
        assert dx[3, 5] == base[3, 5]        # exp(-inf) contributes exactly nothing
        np.testing.assert_array_equal(dx[4], base[4])   # zero upstream gradient adds zeros


def test_cross_entropy_bf16_logits(ctx):
    rng = np.random.default_rng(96)
    rows, V = 7, 5003
    xb = to_bf16_bits((3.0 * rng.standard_normal((rows, V))).astype(np.float32))
    x = from_bf16_bits(xb)
    labels = rng.integers(0, V, rows, dtype=np.int32)
    dloss = rng.standard_normal(rows).astype(np.float32)
    for use_lse in (True, False):
        loss, _, dxb = run_ce(ctx, xb, labels, dloss, capi.BF16, use_lse, dx_init=np.zeros((rows, V), np.uint16))
        ref_loss = K.cross_entropy_forward(x, labels)
        assert np.abs(loss - ref_loss).max() <= 1e-4 * max(1.0, np.abs(ref_loss).max())   # fp32 output, hardware exp2
        ref = np.zeros_like(x)
        K.cross_entropy_backward_into(x, labels, dloss, ref)
        assert_bf16_close(from_bf16_bits(dxb), ref, "bf16 dlogits")


def test_cross_entropy_label_out_of_range(ctx):
    x = np.zeros((2, 8), np.float32)
    dx_, dl = ctx.upload(x), ctx.upload(np.array([3, 8], np.int32))
    loss = ctx.upload(np.full(2, -7.0, np.float32))
    ctx.call("agrad_cross_entropy_forward", capi.F32, vp(dx_), vp(dl), vp(loss), None, 2, 8)
    with pytest.raises(IndexError):
        ctx.synchronize()
    got = loss.download()
    assert got[0] == pytest.approx(np.log(8.0), rel=1e-6) and got[1] == 0.0
    with pytest.raises(capi.AgradError):
        ctx.call("agrad_cross_entropy_forward", capi.F32, vp(dx_), vp(dl), vp(loss), None, 2, 0)
    ctx.call("agrad_cross_entropy_forward", capi.F32, vp(dx_), vp(dl), vp(loss), None, 0, 8)   # no rows: no-op
    ctx.synchronize()
    for d in (dx_, dl, loss):
        d.free()


def test_cross_entropy_through_the_runtime():
    """CrossEntropyLossOp on "hip" against the oracle device: same graph, same
    upstream gradient (the reference's run_single_op protocol,
    check_tiny_gpt2_kernel.py:473-490)."""
    rng = np.random.default_rng(97)
    B, Tn, V = 2, 9, 301
    x_np = (2.0 * rng.standard_normal((B, Tn, V))).astype(np.float32)
    lab_np = rng.integers(0, V, (B, Tn), dtype=np.int32)
    up = rng.standard_normal((B, Tn)).astype(np.float32)
    results = {}
    for device in ("cpu", "hip"):
        rt = Runtime(device=device)
        x = Tensor(shape=x_np.shape, dtype=np.float32, device=device, requires_grad=True, init_val=x_np)
        lab = Tensor(shape=lab_np.shape, dtype=np.int32, device=device, requires_grad=False, init_val=lab_np)
        loss = CrossEntropyLossOp()(x, lab)
        rt.loss = loss
        rt.build_topo(loss)
        rt.bind_memory()
        rt.forward()
        rt.zero_grad()
        rt.backend.copy_from_host(loss.grad, up)
        rt.backward_graph()
        rt.backend.synchronize()
        results[device] = (rt.backend.copy_to_host(loss), rt.backend.copy_to_host(x.grad))
        rt.release()
    assert_fp32_close(results["hip"][0], results["cpu"][0], "loss")
    assert_fp32_close(results["hip"][1], results["cpu"][1], "dlogits")


# ---- loss and gradient in one launch, in place (fused_linear_ce_logits_to_dlogits) ---------------
def run_fused(ctx, x_store, targets, dtype, scale=1.0, row_scale=None, row_base=0, write_grad=1, offset_elems=0,
              want_loss=True, want_lse=True):
    rows, V = x_store.shape
    esz = x_store.dtype.itemsize
    pad = np.zeros(offset_elems, x_store.dtype)
    d_x = ctx.upload(np.concatenate([pad, x_store.reshape(-1)]))
    total = row_base + rows
    tg = np.full(total, -5, np.int32)
    tg[row_base:] = targets
    d_t = ctx.upload(tg)
    loss = ctx.upload(np.full(total, -7.0, np.float32))
    lse = ctx.upload(np.full(total, -7.0, np.float32))
    d_rs = None
    if row_scale is not None:
        full = np.zeros(total, np.float32)
        full[row_base:] = row_scale
        d_rs = ctx.upload(full)
    ctx.call("agrad_cross_entropy_fused", dtype, vp(d_x, offset_elems * esz), vp(d_t), vp(loss) if want_loss else None,
             vp(lse) if want_lse else None, vp(d_rs), rows, V, row_base, float(scale), write_grad)
    ctx.synchronize()
    out = loss.download(), lse.download(), d_x.download()[offset_elems:].reshape(x_store.shape)
    for d in (d_x, d_t, loss, lse, d_rs):
        if d is not None:
            d.free()
    return out


# every register geometry (4 ... 20 vectors a thread), the second pass from memory (fp32 beyond 81920 classes),
# odd row lengths (rows start at any alignment), tiny rows (element by element)
FUSED_SHAPES = [(1, 1), (3, 7), (5, 64), (4, 1000), (6, 4099), (3, 32768), (2, 50257), (2, 65536), (2, 81920), (1, 128256),
                (2, 151936)]


@pytest.mark.parametrize("rows,V", FUSED_SHAPES)
def test_fused_cross_entropy_fp32(ctx, rows, V):
    rng = np.random.default_rng(190 + V)
    x = (4.0 * rng.standard_normal((rows, V))).astype(np.float32)
    t = rng.integers(0, V, rows, dtype=np.int32)
    if rows >= 3:
        t[1] = -1                       # an ignored position
    scale = 1.0 / 16384
    loss, lse, dx = run_fused(ctx, x, t, capi.F32, scale=scale, row_base=5)
    w_loss, w_lse, w_dx = K.cross_entropy_fused(x, t, np.float32(scale))
    assert_fp32_close(loss[5:], w_loss, "loss")
    assert_fp32_close(lse[5:], w_lse, "lse")
    np.testing.assert_array_equal(loss[:5], np.full(5, -7.0, np.float32))      # rows before row_base are not touched
    # the gradient against the restatement at the scale's size (values are p * 6e-5), and against float64
    assert_fp32_close(dx / np.float32(scale), w_dx / np.float32(scale), "dlogits")
    ok = t >= 0
    if ok.any():
        assert np.abs(dx[ok] / scale - cf.cross_entropy_grad(x[ok], t[ok], np.ones(int(ok.sum()), np.float32))).max() <= 2e-6
    assert not dx[~ok].any()


@pytest.mark.parametrize("rows,V", [(5, 64), (4, 1000), (3, 32768), (2, 50257), (3, 65536), (2, 128256), (2, 151936)])
def test_fused_cross_entropy_bf16(ctx, rows, V):
    rng = np.random.default_rng(290 + V)
    x = from_bf16_bits(to_bf16_bits((4.0 * rng.standard_normal((rows, V))).astype(np.float32)))
    t = rng.integers(0, V, rows, dtype=np.int32)
    rs = rng.standard_normal(rows).astype(np.float32)
    loss, lse, dx = run_fused(ctx, to_bf16_bits(x), t, capi.BF16, row_scale=rs)
    w_loss, w_lse, w_dx = K.cross_entropy_fused(x, t, 1.0, row_scale=rs)
    np.testing.assert_allclose(loss, w_loss, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(lse, w_lse, rtol=2e-5, atol=2e-5)
    assert_bf16_close(from_bf16_bits(dx), w_dx, "dlogits (bf16)")


def test_fused_cross_entropy_masks_unaligned_and_loss_only(ctx):
    rng = np.random.default_rng(391)
    rows, V = 6, 1537
    x = (3.0 * rng.standard_normal((rows, V))).astype(np.float32)
    x[2, 10:40] = -np.inf               # masked classes
    x[4, :] = -np.inf                   # a row with no finite logit: zero row, loss 0
    t = rng.integers(0, V, rows, dtype=np.int32)
    t[5] = V                            # out of range above
    for off in (0, 1, 3):               # the tensor itself starts 0, 4 or 12 bytes past a 16-byte boundary
        loss, lse, dx = run_fused(ctx, x, t, capi.F32, scale=0.5, offset_elems=off)
        w_loss, w_lse, w_dx = K.cross_entropy_fused(x, t, np.float32(0.5))
        assert_fp32_close(loss, w_loss, f"loss off={off}")
        assert_fp32_close(lse, w_lse, f"lse off={off}")
        assert_fp32_close(dx, w_dx, f"dlogits off={off}")
        assert not dx[4].any() and not dx[5].any() and not np.isnan(dx).any()
    # write_grad = 0: the logits stay as they were
    loss, lse, same = run_fused(ctx, x, t, capi.F32, write_grad=0)
    np.testing.assert_array_equal(same, x)
    assert_fp32_close(loss, w_loss, "loss only")
    # NULL loss / lse outputs are allowed
    _, _, dx = run_fused(ctx, x, t, capi.F32, scale=0.5, want_loss=False, want_lse=False)
    assert_fp32_close(dx, w_dx, "dlogits without loss outputs")
    with pytest.raises(capi.AgradError):
        run_fused(ctx, x, t, capi.F32, write_grad=2)


@pytest.mark.parametrize("dtype,rows,V", [("f32", 300, 90001), ("f32", 37, 151936), ("bf16", 150, 170001)])
def test_fused_cross_entropy_rows_shared_by_a_team_of_workgroups(ctx, dtype, rows, V):
    """Rows too long for one workgroup's registers (fp32 beyond 81920 classes, bf16 beyond 163840)
    are held by a team of workgroups, a slice each, which exchange their (max, sum) pairs through
    memory.  More rows than teams, so that every team takes several rows in turn (the pairs
    alternate between two sets of slots); an odd row length, so that rows start at every
    alignment; a slice that is all -inf, a row that is, an ignored and an out-of-range target;
    per-row scales, a row base, the loss-only form."""
    rng = np.random.default_rng(490 + V)
    x = (4.0 * rng.standard_normal((rows, V))).astype(np.float32)
    if dtype == "bf16":
        x = from_bf16_bits(to_bf16_bits(x))
    x[2, :9000] = -np.inf               # one member's whole slice
    x[3, V // 2:] = -np.inf
    x[4, :] = -np.inf                   # no finite logit: zero row, loss 0
    x[6, 5] = 60.0                      # one class takes all the mass
    t = rng.integers(0, V, rows, dtype=np.int32)
    t[1] = -1
    t[5] = V
    t[7] = V - 1
    t[8] = 0
    rs = rng.standard_normal(rows).astype(np.float32)
    store = to_bf16_bits(x) if dtype == "bf16" else x
    dt = capi.BF16 if dtype == "bf16" else capi.F32
    loss, lse, dx = run_fused(ctx, store, t, dt, row_scale=rs, row_base=3)
    w_loss, w_lse, w_dx = K.cross_entropy_fused(x, t, 1.0, row_scale=rs)
    if dtype == "bf16":
        np.testing.assert_allclose(loss[3:], w_loss, rtol=2e-5, atol=2e-5)
        np.testing.assert_allclose(lse[3:], w_lse, rtol=2e-5, atol=2e-5)
        assert_bf16_close(from_bf16_bits(dx), w_dx, "dlogits (bf16, team)")
        dx = from_bf16_bits(dx)
    else:
        assert_fp32_close(loss[3:], w_loss, "loss (team)")
        assert_fp32_close(lse[3:], w_lse, "lse (team)")
        assert_fp32_close(dx, w_dx, "dlogits (team)")
    np.testing.assert_array_equal(loss[:3], np.full(3, -7.0, np.float32))
    assert not dx[1].any() and not dx[4].any() and not dx[5].any() and not np.isnan(dx).any()
    # twice in a row: the words of the first call's rows are cleared in front of the second
    loss2, lse2, dx2 = run_fused(ctx, store, t, dt, row_scale=rs, row_base=3)
    np.testing.assert_array_equal(loss2, loss)
    np.testing.assert_array_equal(lse2, lse)
    np.testing.assert_array_equal(from_bf16_bits(dx2) if dtype == "bf16" else dx2, dx)
    # the loss alone leaves the logits as they were
    loss3, _, same = run_fused(ctx, store, t, dt, row_base=3, write_grad=0)
    np.testing.assert_array_equal(same, store)
    np.testing.assert_array_equal(loss3, loss)


def test_fused_cross_entropy_team_wait_is_bounded(ctx):
    """A member of a team waits for the others a bounded number of polls.  With the bound set to
    one poll from the host, members give up at once: the launch still ends, the pass boundary
    says that the gradient is not valid (or, if every pair happened to be there in time, the
    numbers are right), and with the default bound back the same call is right again."""
    rng = np.random.default_rng(591)
    rows, V = 96, 151936
    x = (4.0 * rng.standard_normal((rows, V))).astype(np.float32)
    t = rng.integers(0, V, rows, dtype=np.int32)
    w_loss, w_lse, w_dx = K.cross_entropy_fused(x, t, np.float32(1.0))
    ctx.call("agrad_set_team_wait_polls", 1)
    try:
        try:
            loss, lse, dx = run_fused(ctx, x, t, capi.F32)
        except capi.AgradError as e:
            assert "team" in str(e)
        else:
            assert_fp32_close(dx, w_dx, "dlogits (every pair in time)")
    finally:
        ctx.call("agrad_set_team_wait_polls", 0)
    ctx.synchronize()                       # the error has been reported once and is gone
    loss, lse, dx = run_fused(ctx, x, t, capi.F32)
    assert_fp32_close(loss, w_loss, "loss")
    assert_fp32_close(dx, w_dx, "dlogits")


def test_fused_cross_entropy_through_the_name_dispatch(ctx):
    """the reference's kernel names and argument order (backend.py:3175-3179)"""
    import ctypes as C
    from autograd_amd.utils import f32_bits
    rng = np.random.default_rng(392)
    rows, V = 7, 2048
    x = (2.0 * rng.standard_normal((rows, V))).astype(np.float32)
    t = rng.integers(0, V, rows, dtype=np.int32)
    rs = rng.standard_normal(rows).astype(np.float32)
    for scaled in (False, True):
        d_x, d_t = ctx.upload(x), ctx.upload(t)
        loss, lse = ctx.upload(np.zeros(rows, np.float32)), ctx.upload(np.zeros(rows, np.float32))
        d_rs = ctx.upload(rs)
        bufs = [d_x, d_t, loss, lse] + ([d_rs] if scaled else [])
        ids = (C.c_uint64 * len(bufs))(*[b.ptr for b in bufs])
        offs = (C.c_uint64 * len(bufs))(*([0] * len(bufs)))
        args = [rows, V, 0, rows if scaled else f32_bits(0.25), 1, capi.F32, 0b1111]
        a = (C.c_uint32 * len(args))(*args)
        name = b"fused_linear_ce_logits_to_dlogits_row_scaled" if scaled else b"fused_linear_ce_logits_to_dlogits"
        ctx.call("agrad_dispatch", name, ids, offs, len(bufs), a, len(args), 0, 0, 0, 0)
        ctx.synchronize()
        w_loss, w_lse, w_dx = K.cross_entropy_fused(x, t, np.float32(0.25), row_scale=rs if scaled else None)
        assert_fp32_close(loss.download(), w_loss, "loss")
        assert_fp32_close(d_x.download(), w_dx, "dlogits")
        for b in bufs + ([] if scaled else [d_rs]):
            b.free()
