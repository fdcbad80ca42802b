"""Pins the CPU restatement (oracle/cpu_ops.py) without a GPU.

Each check is chosen so that a plausible mistake -- a dropped term, a wrong
sign, a transposed operand, population vs sample variance, eps inside vs outside
the square root -- fails it: float64 closed forms written independently
(oracle/closed_form.py, after verify_model.py:127-135 and
debug/check_qwen_kernel.py:195-342, 577-645), central finite differences
(verify_model.py:65-77), algebraic invariants, and brute force on small inputs.
"""
import numpy as np
import pytest

from oracle import closed_form as cf
from oracle import cpu_ops as K

SEED = 1333


def rng(k):
    return np.random.default_rng(SEED + k)


def close(a, b, rtol=1e-5, atol=1e-6):
    np.testing.assert_allclose(np.asarray(a, np.float64), np.asarray(b, np.float64), rtol=rtol, atol=atol)


# ---- GELU ---------------------------------------------------------------------
def test_gelu_matches_closed_form_and_special_values():
    x = rng(5).standard_normal((2, 16, 64), dtype=np.float32)      # probe_gelu recipe
    close(K.gelu_forward(x), cf.gelu(x))
    sp = np.array([0.0, 30.0, -30.0], np.float32)
    y = K.gelu_forward(sp)
    assert y[0] == 0 and y[1] == 30 and y[2] == 0
    dx = np.zeros(3, np.float32)
    K.gelu_backward_into(sp, np.ones(3, np.float32), dx)
    assert dx[0] == 0.5 and dx[1] == 1.0 and dx[2] == 0.0
    # the constants are the reference's (backend.py:18-20)
    assert K.GELU_C == 0.7978845608028654 and K.GELU_A == 0.044715 and K.GELU_A3 == 0.134145
    assert abs(K.GELU_C - np.sqrt(2 / np.pi)) < 1e-15 and abs(K.GELU_A3 - 3 * K.GELU_A) < 1e-15


def test_gelu_backward_finite_difference_and_accumulate():
    r = rng(5)
    x = r.standard_normal((7, 33), dtype=np.float32)
    dy = r.standard_normal((7, 33), dtype=np.float32)
    dx = np.zeros_like(x)
    K.gelu_backward_into(x, dy, dx)
    close(dx, dy * cf.gelu_grad(x), rtol=2e-5, atol=2e-6)
    idx = r.choice(x.size, 25, replace=False)
    fd = cf.finite_diff(lambda a: float((cf.gelu(a) * dy).sum()), x, idx, eps=1e-4)
    close(dx.reshape(-1)[idx], fd, rtol=1e-4, atol=1e-5)
    base = r.standard_normal(x.shape, dtype=np.float32)
    acc = base.copy()
    K.gelu_backward_into(x, dy, acc)            # "grad += ..." (backend.py:414)
    close(acc, base + dx, atol=2e-6)


def test_bias_gelu_is_gelu_of_the_sum_and_its_bias_gradient_is_the_row_sum():
    r = rng(23)
    h = r.standard_normal((4, 9, 33), dtype=np.float32)
    b = r.standard_normal(33, dtype=np.float32)
    dy = r.standard_normal(h.shape, dtype=np.float32)
    close(K.bias_gelu_forward(h, b), cf.gelu(h.astype(np.float64) + b))
    dh = np.zeros_like(h)
    db = np.zeros_like(b)
    K.bias_gelu_backward_into(h, b, dy, dh=dh, db=db)
    slope = cf.gelu_grad(h.astype(np.float64) + b)
    close(dh, dy * slope, rtol=2e-5, atol=2e-6)
    by_rows = np.zeros(33)
    for i in range(4):                     # the bias gradient, row by row
        for j in range(9):
            by_rows += dy[i, j] * slope[i, j]
    close(db, by_rows, rtol=2e-5, atol=2e-5)
    # finite differences: in one element of h, and in one element of b (which moves a whole column)
    loss = lambda hh, bb: float((cf.gelu(hh + bb) * dy).sum())
    h64, b64 = h.astype(np.float64), b.astype(np.float64)
    for idx in ((0, 0, 0), (3, 8, 32), (1, 4, 17)):
        e = np.zeros_like(h64); e[idx] = 1e-5
        close(dh[idx], (loss(h64 + e, b64) - loss(h64 - e, b64)) / 2e-5, rtol=1e-4, atol=1e-5)
    for c in (0, 17, 32):
        e = np.zeros_like(b64); e[c] = 1e-5
        close(db[c], (loss(h64, b64 + e) - loss(h64, b64 - e)) / 2e-5, rtol=1e-4, atol=2e-5)
    # "grad += ..." on both, and either alone
    dh2, db2 = dh.copy(), db.copy()
    K.bias_gelu_backward_into(h, b, dy, dh=dh2)
    K.bias_gelu_backward_into(h, b, dy, db=db2)
    close(dh2, 2 * dh, atol=4e-6)
    close(db2, 2 * db, atol=4e-5)


# ---- ReLU^2 (closed form only: the reference has none) ---------------------------
def test_relu2():
    r = rng(11)
    x = r.standard_normal((5, 40), dtype=np.float32)
    dy = r.standard_normal((5, 40), dtype=np.float32)
    close(K.relu2_forward(x), cf.relu2(x))
    dx = np.zeros_like(x)
    K.relu2_backward_into(x, dy, dx)
    close(dx, dy * cf.relu2_grad(x))
    assert (K.relu2_forward(np.array([-1.0, 0.0, -0.0, 2.0], np.float32)) == [0, 0, 0, 4]).all()


# ---- LayerNorm ------------------------------------------------------------------
def _ln_case(k=4, shape=(2, 16, 64)):
    r = rng(k)
    C = shape[-1]
    return (r.standard_normal(shape, dtype=np.float32), r.standard_normal(C, dtype=np.float32),
            r.standard_normal(C, dtype=np.float32), r.standard_normal(shape, dtype=np.float32))


def test_layernorm_forward_closed_form_and_invariants():
    x, g, b, _ = _ln_case()
    y64, _, _ = cf.layernorm(x, g, b, 1e-5)
    close(K.layernorm_forward(x, g, b, 1e-5), y64, rtol=2e-5, atol=2e-6)
    plain = K.layernorm_forward(x, np.ones_like(g), np.zeros_like(b), 1e-5)
    assert np.abs(plain.mean(-1)).max() < 1e-6          # mean 0
    assert np.abs(plain.var(-1) - 1).max() < 1e-4       # population variance 1 (not the sample one: 64/63)
    # eps sits inside the square root: a constant row maps to beta
    const = np.full((3, 8), 2.5, np.float32)
    close(K.layernorm_forward(const, np.ones(8, np.float32), np.full(8, 0.25, np.float32), 1e-5), 0.25)


def test_layernorm_backward_closed_form_fd_and_invariants():
    x, g, b, dy = _ln_case()
    dx, dg, db = np.zeros_like(x), np.zeros_like(g), np.zeros_like(b)
    K.layernorm_backward_into(x, g, dy, 1e-5, dx, dg, db)
    dx64, dg64, db64 = cf.layernorm_grads(x, g, dy, 1e-5)
    close(dx, dx64, rtol=2e-5, atol=2e-6)
    close(dg, dg64, rtol=2e-5, atol=5e-6)
    close(db, db64, rtol=2e-5, atol=5e-6)
    r = rng(40)
    idx = r.choice(x.size, 20, replace=False)
    fd = cf.finite_diff(lambda a: float((cf.layernorm(a, g, b, 1e-5)[0] * dy).sum()), x, idx, eps=1e-4)
    close(dx.reshape(-1)[idx], fd, rtol=2e-3, atol=2e-4)
    # gamma = 1: each row of dx sums to zero and is orthogonal to x_hat
    one = np.ones_like(g)
    dx1 = np.zeros_like(x)
    K.layernorm_backward_into(x, one, dy, 1e-5, dx1, None, None)
    _, _, xh = cf.layernorm(x, one, np.zeros_like(b), 1e-5)
    assert np.abs(dx1.sum(-1)).max() < 2e-5
    assert np.abs((dx1 * xh).sum(-1)).max() < 1e-3      # exact up to eps / (var + eps)
    # accumulation into existing grads
    base = r.standard_normal(x.shape, dtype=np.float32)
    acc = base.copy()
    K.layernorm_backward_into(x, g, dy, 1e-5, acc, None, None)
    close(acc, base + dx, atol=3e-6)


# ---- RMSNorm ----------------------------------------------------------------------
def test_rmsnorm_forward_backward():
    r = rng(6)
    x = (0.02 * r.standard_normal((2, 8, 96))).astype(np.float32)   # x ~ 0.02 N (check_qwen_kernel.py:1097-1139)
    g = (1 + 0.02 * r.standard_normal(96)).astype(np.float32)
    g[0] = 0.0
    dz = r.standard_normal(x.shape, dtype=np.float32)
    z64, _, _ = cf.rmsnorm(x, g, 1e-6)
    close(K.rmsnorm_forward(x, g, 1e-6), z64, rtol=2e-5, atol=2e-6)
    close(K.rmsnorm_forward(x, None, 1e-6), cf.rmsnorm(x, None, 1e-6)[0], rtol=2e-5, atol=2e-6)
    dx, dg = np.zeros_like(x), np.zeros_like(g)
    K.rmsnorm_backward_into(x, g, dz, 1e-6, dx, dg)
    dx64, dg64 = cf.rmsnorm_grads(x, g, dz, 1e-6)
    close(dx, dx64, rtol=5e-5, atol=1e-4 * np.abs(dx64).max())
    close(dg, dg64, rtol=2e-5, atol=1e-5)
    idx = r.choice(x.size, 20, replace=False)
    fd = cf.finite_diff(lambda a: float((cf.rmsnorm(a, g, 1e-6)[0] * dz).sum()), x, idx, eps=1e-6)
    close(dx.reshape(-1)[idx], fd, rtol=5e-3, atol=5e-3 * np.abs(fd).max())
    # gamma = 1 and eps -> 0: dx is orthogonal to x row by row
    xb = r.standard_normal((5, 64), dtype=np.float32)
    d1 = np.zeros_like(xb)
    K.rmsnorm_backward_into(xb, None, dz.reshape(-1, 96)[:5, :64].copy(), 0.0, d1, None)
    assert np.abs((d1 * xb).sum(-1)).max() < 1e-4
    # unit-RMS rows come back unchanged
    u = np.ones((2, 16), np.float32)
    close(K.rmsnorm_forward(u, None, 0.0), u)


def test_add_norm_is_add_then_norm():
    r = rng(9)
    x, res = r.standard_normal((4, 32), dtype=np.float32), r.standard_normal((4, 32), dtype=np.float32)
    g, b = r.standard_normal(32, dtype=np.float32), r.standard_normal(32, dtype=np.float32)
    h, y = K.add_norm_forward("layer", x, res, g, b, 1e-5)
    assert np.array_equal(h, x + res) and np.array_equal(y, K.layernorm_forward(x + res, g, b, 1e-5))
    h, z = K.add_norm_forward("rms", x, res, g, None, 1e-6)
    assert np.array_equal(z, K.rmsnorm_forward(x + res, g, 1e-6))


# ---- SwiGLU -------------------------------------------------------------------------
def test_swiglu():
    r = rng(12)
    gu = (2 * r.standard_normal((6, 2 * 40))).astype(np.float32)
    dh = r.standard_normal((6, 40), dtype=np.float32)
    close(K.swiglu_forward(gu), cf.swiglu(gu), rtol=2e-5, atol=2e-6)
    dgu = K.swiglu_backward(gu, dh)
    close(dgu, cf.swiglu_grads(gu, dh), rtol=2e-5, atol=2e-6)
    idx = r.choice(gu.size, 30, replace=False)
    fd = cf.finite_diff(lambda a: float((cf.swiglu(a) * dh).sum()), gu, idx, eps=1e-5)
    close(dgu.reshape(-1)[idx], fd, rtol=1e-4, atol=1e-5)
    # gate = first half, up = second half; silu(0) = 0; the up gradient of a zero gate is 0
    z = np.zeros((1, 8), np.float32)
    z[0, 4:] = 3.0
    assert not K.swiglu_forward(z).any()
    d = K.swiglu_backward(z, np.ones((1, 4), np.float32))
    close(d[0, :4], 0.5 * 3.0)       # d/dg silu(g) u at g = 0 is u / 2
    assert not d[0, 4:].any()


# ---- RoPE -----------------------------------------------------------------------------
def test_rope_tables():
    cos, sin = K.rope_tables(16, 8, 1e4)
    assert cos.shape == (16, 4) and cos.dtype == np.float32
    assert (cos[0] == 1).all() and (sin[0] == 0).all()
    inv = 1e4 ** (-np.arange(0, 8, 2) / 8)
    close(cos, np.cos(np.arange(16)[:, None] * inv), atol=2e-6)
    close(sin, np.sin(np.arange(16)[:, None] * inv), atol=2e-6)


@pytest.mark.parametrize("sign", [1, -1])
def test_rope_signed_closed_form_and_invariants(sign):
    r = rng(15)
    B, T, H, HKV, D = 2, 9, 3, 1, 16
    q = r.standard_normal((B, T, H, D), dtype=np.float32)
    k = r.standard_normal((B, T, HKV, D), dtype=np.float32)
    cos, sin = K.rope_tables(T, D, 1e6)
    fq, fk = q.copy(), k.copy()
    K.rope_signed(fq, fk, cos, sin, sign, False)
    close(fq, cf.rope(q, cos, sin, sign), atol=2e-6)
    close(fk, cf.rope(k, cos, sin, sign), atol=2e-6)
    assert np.array_equal(fq[:, 0], q[:, 0])                 # position 0 is the identity
    h = D // 2
    close(fq[..., :h] ** 2 + fq[..., h:] ** 2, q[..., :h] ** 2 + q[..., h:] ** 2, atol=1e-5)
    bq, bk = fq.copy(), fk.copy()
    K.rope_signed(bq, bk, cos, sin, sign, True)              # backward is the transpose = inverse
    close(bq, q, atol=2e-6)
    iq, ik = fq.copy(), fk.copy()
    K.rope_signed(iq, ik, cos, sin, -sign, False)            # the two conventions are mutual inverses
    close(iq, q, atol=2e-6)
    # <R x, g> = <x, R^T g>
    g = r.standard_normal(q.shape, dtype=np.float32)
    tg, _ = g.copy(), None
    K.rope_signed(tg, k.copy(), cos, sin, sign, True)
    assert abs(float((fq.astype(np.float64) * g).sum() - (q.astype(np.float64) * tg).sum())) < 1e-3


def test_rope_nanochat_is_sign_minus_one():
    r = rng(16)
    q = r.standard_normal((2, 7, 2, 8), dtype=np.float32)
    k = r.standard_normal((2, 7, 1, 8), dtype=np.float32)
    cos, sin = K.rope_tables(7, 8, 1e5)
    for backward in (False, True):
        a, b = q.copy(), k.copy()
        K.rope_nanochat(a, b, cos, sin, backward)
        c, d = q.copy(), k.copy()
        K.rope_signed(c, d, cos, sin, -1, backward)
        assert np.array_equal(a, c) and np.array_equal(b, d)
    # the sign: with cos = 0, sin = 1 the nanochat forward maps (lo, hi) -> (hi, -lo)
    one = np.ones((1, 1), np.float32)
    x = np.array([[[[2.0, 5.0]]]], np.float32)
    y = x.copy()
    K.rope_nanochat(y, None, 0 * one, one, False)
    assert (y.ravel() == [5.0, -2.0]).all()
    y = x.copy()
    K.rope_signed(y, None, 0 * one, one, 1, False)           # HF: (lo, hi) -> (-hi, lo)
    assert (y.ravel() == [-5.0, 2.0]).all()


# ---- embedding -----------------------------------------------------------------------
def test_gather_reference_vectors():
    """verify_model.py:298-318 (seed 1234, B,T,V,C = 2,3,11,4)."""
    r = np.random.default_rng(1234)
    B, T, V, C = 2, 3, 11, 4
    idx = r.integers(0, V, size=(B, T), dtype=np.int32)
    w = (r.standard_normal((V, C)) * 0.1).astype(np.float32)
    out = K.gather_forward(idx, w)
    for b in range(B):
        for t in range(T):
            assert np.array_equal(out[b, t], w[idx[b, t]])
    # d/dw of sum(out) counts occurrences (the scalar loss of the reference's case)
    dW = np.zeros_like(w)
    K.gather_backward_into(idx, np.ones((B, T, C), np.float32), dW)
    assert np.array_equal(dW[:, 0], np.bincount(idx.ravel(), minlength=V).astype(np.float32))


def test_gather_backward_is_row_order_loop():
    r = rng(20)
    B, T, V, C = 3, 50, 7, 5
    ids = r.integers(0, V, size=(B, T), dtype=np.int32)
    dY = r.standard_normal((B, T, C), dtype=np.float32)
    dW = np.zeros((V, C), np.float32)
    K.gather_backward_into(ids, dY, dW)
    brute = np.zeros((V, C), np.float32)
    for n, t in enumerate(ids.ravel()):
        brute[t] += dY.reshape(-1, C)[n]              # fp32, ascending row order
    assert np.array_equal(dW, brute)
    close(dW.sum(0), dY.reshape(-1, C).sum(0), atol=1e-4)
    close(dW, cf.gather_backward(ids, dY, V), atol=1e-5)
    with pytest.raises(IndexError):
        K.gather_forward(np.array([[V]], np.int32), np.zeros((V, C), np.float32))


def test_embedding_sum():
    r = rng(19)
    B, T, V, C = 2, 6, 13, 4
    ids = r.integers(0, V, size=(B, T), dtype=np.int32)
    wte = r.standard_normal((V, C), dtype=np.float32)
    wpe = r.standard_normal((T, C), dtype=np.float32)
    out = K.embedding_sum_forward(ids, wte, wpe)
    assert np.array_equal(out, wte[ids] + wpe[None, :, :])
    dY = r.standard_normal((B, T, C), dtype=np.float32)
    dwte, dwpe = np.zeros_like(wte), np.zeros_like(wpe)
    K.embedding_sum_backward_into(ids, dY, dwte, dwpe)
    seq = np.zeros_like(wpe)
    for b in range(B):
        seq += dY[b]
    assert np.array_equal(dwpe, seq)                 # sum over batch, b ascending
    ref = np.zeros_like(wte)
    K.gather_backward_into(ids, dY, ref)
    assert np.array_equal(dwte, ref)


def test_add_backward_broadcast():
    r = rng(21)
    g = r.standard_normal((3, 4, 5), dtype=np.float32)
    same, bc = np.zeros((3, 4, 5), np.float32), np.zeros((4, 5), np.float32)
    K.add_backward_into(g, same)
    K.add_backward_into(g, bc)
    assert np.array_equal(same, g)
    close(bc, g.sum(0), atol=1e-6)


# ---- bf16 ---------------------------------------------------------------------------
def _bf16_scalar(bits):
    """integer restatement of utils.py:20-27 on a uint32 bit pattern"""
    if bits & 0x7F800000 == 0x7F800000:
        return ((bits >> 16) | (0x0040 if bits & 0x007FFFFF else 0)) & 0xFFFF
    return ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) & 0xFFFF


def test_bf16_rounding_rule():
    cases = {
        0x3F800000: 0x3F80,   # 1.0
        0x3F808000: 0x3F80,   # tie, even mantissa -> down
        0x3F818000: 0x3F82,   # tie, odd mantissa -> up
        0x3F808001: 0x3F81,   # just above the tie
        0x7F800000: 0x7F80,   # +inf kept
        0xFF800000: 0xFF80,   # -inf kept
        0x7F800001: 0x7FC0,   # signalling NaN -> quiet
        0x7FC00000: 0x7FC0,
        0x7F7FFFFF: 0x7F80,   # max finite rounds to inf
        0x80000000: 0x8000,   # -0
        0x00000001: 0x0000,
    }
    bits = np.array(list(cases), dtype=np.uint32)
    got = K.f32_to_bf16_bits(bits.view(np.float32))
    assert got.tolist() == list(cases.values())
    # dense sample of all 2^32 patterns against the scalar rule, plus every exponent edge
    r = rng(30)
    sample = np.concatenate([r.integers(0, 2 ** 32, size=200_000, dtype=np.uint64).astype(np.uint32),
                             (np.arange(512, dtype=np.uint32) << 23)[:, None].repeat(4, 1).ravel()
                             + np.tile(np.array([0, 0x7FFF, 0x8000, 0x8001], np.uint32), 512)])
    got = K.f32_to_bf16_bits(sample.view(np.float32))
    want = np.array([_bf16_scalar(int(b)) for b in sample], dtype=np.uint16)
    assert np.array_equal(got, want)
    # widening is exact and rounding is idempotent
    back = K.bf16_bits_to_f32(got)
    finite = np.isfinite(back)
    assert np.array_equal(K.f32_to_bf16_bits(back[finite]), got[finite])
    # product-side helpers implement the same rule
    from autograd_amd import utils
    assert np.array_equal(utils.f32_array_to_bf16_bits(sample.view(np.float32)), want)
    assert all(utils.bf16_bits(float(np.uint32(b).view(np.float32))) == w
               for b, w in cases.items() if not np.isnan(np.uint32(b).view(np.float32)))


# ---------------------------------------------------------------------------
# AdamW (cpu_adamw_step, backend.py:2013-2038)
# ---------------------------------------------------------------------------
def _adam_case(k, n=513):
    r = rng(k)
    p = r.standard_normal(n).astype(np.float32)
    grads = [r.standard_normal(n).astype(np.float32) for _ in range(5)]
    return p, grads


def test_adamw_first_step_is_lr_times_sign_and_matches_textbook():
    import math
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.999, 1e-8, 0.0
    p0, grads = _adam_case(40)
    p, m, v = p0.copy(), np.zeros_like(p0), np.zeros_like(p0)
    lr_t = lr * math.sqrt(1.0 - b2) / (1.0 - b1)
    K.adamw_step(p, grads[0], m, v, lr, lr_t, b1, b2, eps, wd)
    # from zero moments the first Adam step is lr * sign(g) (eps only matters for |g| ~ 1e-8)
    big = np.abs(grads[0]) > 1e-3
    assert np.abs((p0 - p)[big] - lr * np.sign(grads[0])[big]).max() < 2e-7
    # several steps, with weight decay, against the float64 recurrence
    wd = 0.1
    p, m, v = p0.copy(), np.zeros_like(p0), np.zeros_like(p0)
    for t, g in enumerate(grads, start=1):
        lr_t = lr * math.sqrt(1.0 - b2 ** t) / (1.0 - b1 ** t)
        K.adamw_step(p, g, m, v, lr, lr_t, b1, b2, eps, wd)
    p64, m64, v64 = cf.adamw_reference(p0, grads, lr, b1, b2, eps, wd)
    close(p, p64)
    close(m, m64, 1e-5, 1e-7)
    close(v, v64, 1e-5, 1e-7)
    # decoupled decay: with zero gradients only the (1 - lr*wd)^t shrink remains
    p, m, v = p0.copy(), np.zeros_like(p0), np.zeros_like(p0)
    zero = np.zeros_like(p0)
    for t in range(1, 4):
        K.adamw_step(p, zero, m, v, lr, lr, b1, b2, eps, wd)
    close(p, p0.astype(np.float64) * (1 - lr * wd) ** 3)
    assert not m.any() and not v.any()


def test_softmax_over_an_inner_axis_is_softmax_of_the_moved_axis():
    import scipy.special as sp
    r = rng(61)
    x = r.standard_normal((3, 5, 4, 6), dtype=np.float32)
    g = r.standard_normal(x.shape, dtype=np.float32)
    for axis in (0, 1, 2, -3):
        y = K.softmax_forward(x, axis=axis)
        close(y, sp.softmax(x.astype(np.float64), axis=axis))
        close(y.sum(axis=axis), np.ones_like(y.sum(axis=axis)), atol=1e-6)
        dx = np.zeros_like(x)
        K.softmax_backward_into(y, g, dx, axis=axis)
        moved_y, moved_g = np.moveaxis(y, axis, -1), np.moveaxis(g, axis, -1)
        want = np.zeros_like(moved_y)
        K.softmax_backward_into(np.ascontiguousarray(moved_y), np.ascontiguousarray(moved_g), want)
        close(dx, np.moveaxis(want, -1, axis), atol=1e-7)
        close(dx.sum(axis=axis), np.zeros_like(dx.sum(axis=axis)), atol=1e-6)      # rows of the Jacobian sum to zero


def test_dynamic_maps_have_the_defining_shape():
    """optimizer.py:144-179: 256 sorted values; the signed map is symmetric with two zero
    codes and extremes -1 / +1, the unsigned one starts at 0, ends at 1 and is strictly
    increasing; seven decades: the smallest non-zero magnitude is a few 1e-7"""
    sm, um = K.dynamic_map(True), K.dynamic_map(False)
    for q in (sm, um):
        assert q.shape == (256,) and q.dtype == np.float32 and (np.diff(q) >= 0).all()
    assert sm[0] == -1 and sm[-1] == 1 and (sm == 0).sum() == 2
    np.testing.assert_array_equal(sm, -sm[::-1])
    assert um[0] == 0 and um[-1] == 1 and (np.diff(um) > 0).all()
    assert 1e-7 < np.abs(sm[sm != 0]).min() < 1e-6 and 1e-8 < um[1] < 1e-6
    # each decade of the signed map holds twice the codes of the decade below
    pos = sm[sm > 0]
    counts = [int(((pos > 10.0 ** -(k + 1)) & (pos <= 10.0 ** -k)).sum()) for k in range(6)]
    assert all(a >= 1.6 * b for a, b in zip(counts, counts[1:])), counts


def test_nearest_code_is_the_nearest_entry_and_ties_go_down():
    r = rng(51)
    for q, lo in ((K.dynamic_map(True), -1.0), (K.dynamic_map(False), 0.0)):
        x = np.concatenate([r.uniform(lo, 1.0, 4000), r.uniform(-1, 1, 500) * 1e-4, q, [lo, 1.0, 0.0]]).astype(np.float32)
        x = np.clip(x, lo, 1.0)
        code = K.nearest_code(q, x)
        brute = np.abs(q[None, :].astype(np.float64) - x[:, None].astype(np.float64)).min(axis=1)
        got = np.abs(q[code].astype(np.float64) - x.astype(np.float64))
        # distances are compared as the kernel forms them, in fp32
        np.testing.assert_array_equal(np.abs(q[code] - x), np.abs(q[None, :] - x[:, None]).min(axis=1))
        assert (got <= brute + 1e-9).all()
        np.testing.assert_array_equal(q[K.nearest_code(q, q)], q)       # a map value is its own code's value
    q = K.dynamic_map(False)
    mid = ((q[200].astype(np.float64) + q[201]) / 2).astype(np.float32)
    if np.abs(q[201] - mid) == np.abs(q[200] - mid):                      # an exact tie in fp32
        assert K.nearest_code(q, np.array([mid]))[0] == 200
    assert K.nearest_code(q, np.array([np.nextafter(q[255], 0, dtype=np.float32)]))[0] in (254, 255)


def test_adamw8bit_tracks_fp32_adamw_within_the_quantisation_error():
    """Five steps of the 8-bit update beside the same update with fp32 moments
    (adamw_step_split with the Metal scalars): the first step is identical in p
    (both start from zero moments), later ones differ by what quantising m and v to
    the map costs -- a few percent of a step -- and the stored moments decode to the
    fp32 ones within the map's resolution.  Weight decay reaches the prefix only."""
    import math
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.95, 1e-8, 0.1
    n, decay_n = 1000, 600
    r = rng(52)
    p0 = r.standard_normal(n).astype(np.float32)
    grads = [r.standard_normal(n).astype(np.float32) for _ in range(5)]
    qm_map, qv_map = K.dynamic_map(True), K.dynamic_map(False)
    p8 = p0.copy()
    qm, qv = np.zeros(n, np.uint8), np.zeros(n, np.uint8)
    am, av = np.zeros(4, np.float32), np.zeros(4, np.float32)
    p32, m32, v32 = p0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    for t, g in enumerate(grads, 1):
        lr_bc1 = lr / (1.0 - b1 ** t)
        inv_sqrt_bc2 = 1.0 / math.sqrt(1.0 - b2 ** t)
        K.adamw8bit_step(p8, g, qm, qv, am, av, qm_map, qv_map, 1.0 - lr * wd, lr_bc1, b1, b2, eps, decay_n, t == 1,
                         inv_sqrt_bc2, clip_coef=0.5)
        K.adamw_step_split(p32, g, m32, v32, lr * wd, b1, b2, eps, lr_bc1, inv_sqrt_bc2, 0.5, decay_numel=decay_n)
        if t == 1:
            np.testing.assert_allclose(p8, p32, rtol=0, atol=6e-7)      # the two spell the same update differently: an ulp or two
            # the first step moves every weight by lr * sign(g) (after the decay factor)
            moved = p8 - p0 * np.where(np.arange(n) < decay_n, np.float32(1.0 - lr * wd), np.float32(1.0))
            np.testing.assert_allclose(moved, -lr * np.sign(g), rtol=1e-3, atol=1e-8)
        blk = np.arange(n) // 256
        m_dec, v_dec = am[blk] * qm_map[qm], av[blk] * qv_map[qv]
        assert np.abs(m_dec - m32).max() <= 0.03 * am.max() * t       # errors of earlier steps carry over, damped by b1
        assert np.abs(v_dec - v32).max() <= 0.03 * av.max() * t
        np.testing.assert_array_equal(am, [np.abs(m_dec[blk == b]).max() for b in range(4)])   # the block maximum is a code value 1
    assert np.abs(p8 - p32).max() < 0.25 * 5 * lr
    assert np.abs(p8[decay_n:] - p0[decay_n:]).max() <= 5.5 * lr       # no decay outside the prefix: only Adam-sized moves


def test_adamw_split_form_is_the_same_update():
    import math
    lr, b1, b2, eps, wd = 3e-4, 0.9, 0.95, 1e-8, 0.05
    p0, grads = _adam_case(41)
    a = [p0.copy(), np.zeros_like(p0), np.zeros_like(p0)]
    b = [p0.copy(), np.zeros_like(p0), np.zeros_like(p0)]
    c = [p0.copy(), np.zeros_like(p0), np.zeros_like(p0)]
    for t, g in enumerate(grads, start=1):
        lr_t = lr * math.sqrt(1.0 - b2 ** t) / (1.0 - b1 ** t)
        K.adamw_step(a[0], g, a[1], a[2], lr, lr_t, b1, b2, eps, wd)
        # neutral extra factors: the very same bits
        K.adamw_step_split(b[0], g, b[1], b[2], lr * wd, b1, b2, eps, lr_t, 1.0, 1.0)
        # the Metal path's split of the bias correction differs only in where eps sits
        K.adamw_step_split(c[0], g, c[1], c[2], lr * wd, b1, b2, eps, lr / (1.0 - b1 ** t),
                             1.0 / math.sqrt(1.0 - b2 ** t), 1.0)
    for x, y in zip(a, b):
        np.testing.assert_array_equal(x, y)
    close(c[0], a[0], 1e-5, 1e-6)
    # clipping by grad_scale is scaling the gradient; decay_numel limits the decay to a prefix
    g = grads[0]
    d = [p0.copy(), np.zeros_like(p0), np.zeros_like(p0)]
    e = [p0.copy(), np.zeros_like(p0), np.zeros_like(p0)]
    K.adamw_step_split(d[0], g, d[1], d[2], lr * wd, b1, b2, eps, lr, 1.0, 0.25, decay_numel=100)
    K.adamw_step_split(e[0][:100], g[:100] * np.float32(0.25), e[1][:100], e[2][:100], lr * wd, b1, b2, eps, lr, 1.0, 1.0)
    K.adamw_step_split(e[0][100:], g[100:] * np.float32(0.25), e[1][100:], e[2][100:], 0.0, b1, b2, eps, lr, 1.0, 1.0)
    for x, y in zip(d, e):
        np.testing.assert_array_equal(x, y)


def test_grad_norm_partials():
    r = rng(42)
    g = r.standard_normal(1000).astype(np.float32)
    part = K.grad_norm_partials(g)
    assert part.shape == (4,)
    assert abs(part.sum() - float(np.dot(g.astype(np.float64), g.astype(np.float64)))) < 1e-9
    assert abs(part[3] - float((g[768:].astype(np.float64) ** 2).sum())) < 1e-12


# ---------------------------------------------------------------------------
# cross-entropy (cpu_crossentropy_forward / backward, backend.py:489-524)
# ---------------------------------------------------------------------------
def test_cross_entropy_closed_form_fd_and_invariants():
    r = rng(50)
    B, Tn, V = 2, 5, 37
    x = (3.0 * r.standard_normal((B, Tn, V))).astype(np.float32)
    labels = r.integers(0, V, (B, Tn), dtype=np.int32)
    loss = K.cross_entropy_forward(x, labels)
    close(loss, cf.cross_entropy(x, labels))
    # uniform logits: every class has probability 1/V
    close(K.cross_entropy_forward(np.full((1, 1, V), 0.7, np.float32), np.array([[3]], np.int32)), np.log(V))
    # a dominant correct class costs nothing, a dominant wrong class costs the margin
    big = np.zeros((1, 2, V), np.float32)
    big[0, 0, 4] = 50.0
    big[0, 1, 9] = 50.0
    close(K.cross_entropy_forward(big, np.array([[4, 4]], np.int32)), [[0.0, 50.0]], atol=1e-5)
    # shifting a row changes nothing
    close(K.cross_entropy_forward(x + np.float32(5.0), labels), loss, atol=5e-6)
    dloss = r.standard_normal((B, Tn)).astype(np.float32)
    dx = np.zeros_like(x)
    K.cross_entropy_backward_into(x, labels, dloss, dx)
    close(dx, cf.cross_entropy_grad(x, labels, dloss))
    assert np.abs(dx.sum(-1, dtype=np.float64)).max() < 1e-6        # softmax sums to one
    base = np.ones_like(x)
    K.cross_entropy_backward_into(x, labels, dloss, base)            # accumulates
    close(base - 1.0, dx, atol=2e-6)
    where = [0, (1 * Tn + 3) * V + 7, (1 * Tn + 4) * V + int(labels[1, 4])]
    fd = cf.finite_diff(lambda a: float((cf.cross_entropy(a, labels) * dloss).sum()), x, where)
    for i, val in zip(where, fd):
        assert abs(val - dx.reshape(-1)[i]) < 2e-3 * max(1.0, abs(val))


def test_cross_entropy_fused_is_the_pair_with_ignored_rows_zeroed():
    """the one-kernel form (metal_ops.metal:8808-8996): scipy's logsumexp / softmax in float64 for
    the valid rows; an out-of-range target or a row of -inf gives loss 0, lse 0 and a zero row"""
    from scipy.special import logsumexp, softmax
    r = rng(51)
    rows, V = 9, 53
    x = (3.0 * r.standard_normal((rows, V))).astype(np.float32)
    t = r.integers(0, V, rows).astype(np.int32)
    t[2], t[5] = -1, V           # ignored positions
    x[7, :] = -np.inf            # no finite logit
    x[8, 3] = -np.inf            # a masked class in an ordinary row
    scale = np.float32(0.37)
    loss, lse, dx = K.cross_entropy_fused(x, t, scale)
    ok = np.array([i not in (2, 5, 7) for i in range(rows)])
    x64 = x.astype(np.float64)
    want_lse = logsumexp(x64[ok], axis=-1)
    close(lse[ok], want_lse)
    close(loss[ok], want_lse - x64[ok, t[ok]])
    p = softmax(x64[ok], axis=-1)
    p[np.arange(ok.sum()), t[ok]] -= 1.0
    close(dx[ok], p * float(scale))
    assert not loss[~ok].any() and not lse[~ok].any() and not dx[~ok].any()
    assert dx[8, 3] == 0.0
    # per-row scales, and the loss-only call
    rs = r.standard_normal(rows).astype(np.float32)
    _, _, dx2 = K.cross_entropy_fused(x, t, 1.0, row_scale=rs)
    close(dx2[ok], p * rs[ok, None].astype(np.float64))
    l3, s3, none = K.cross_entropy_fused(x, t, scale, write_grad=False)
    assert none is None
    np.testing.assert_array_equal(l3, loss)
    np.testing.assert_array_equal(s3, lse)


# ---------------------------------------------------------------------------
# strided views and the permute / transpose gradients: an explicit loop over every
# dense index with the index arithmetic written out
# ---------------------------------------------------------------------------
def _loop_gather(flat, shape, strides, offset):
    out = np.empty(shape, flat.dtype)
    for idx in np.ndindex(*shape):
        out[idx] = flat[offset + sum(c * s for c, s in zip(idx, strides))]
    return out


def test_strided_view_matches_the_index_loop():
    rng = np.random.default_rng(SEED + 70)
    flat = rng.standard_normal(600).astype(np.float32)
    for shape, strides, offset in [((3, 4, 5), (20, 5, 1), 0), ((5, 4, 3), (1, 5, 20), 0), ((4, 6), (0, 2), 3),
                                   ((2, 3, 4), (100, 1, 7), 11), ((7,), (3,), 2)]:
        got = K.contiguous_forward(flat, shape, strides, offset)
        assert got.flags["C_CONTIGUOUS"]
        np.testing.assert_array_equal(got, _loop_gather(flat, shape, strides, offset))


def test_permute_and_transpose_gradients_match_the_index_loop():
    rng = np.random.default_rng(SEED + 71)
    xshape = (2, 3, 4, 5)
    for dims in [(0, 2, 1, 3), (3, 2, 1, 0), (1, 3, 0, 2)]:
        oshape = tuple(xshape[d] for d in dims)
        g = rng.standard_normal(oshape).astype(np.float32)
        base = rng.standard_normal(xshape).astype(np.float32)
        want = base.copy()
        for idx in np.ndindex(*xshape):       # out[j] = x[idx] where j[i] = idx[dims[i]]
            want[idx] = base[idx] + g[tuple(idx[d] for d in dims)]
        got = base.copy()
        K.permute_backward_into(g, list(dims), got)
        np.testing.assert_array_equal(got, want)
    g = rng.standard_normal((2, 5, 4, 3)).astype(np.float32)
    base = rng.standard_normal(xshape).astype(np.float32)
    want = base.copy()
    for idx in np.ndindex(*xshape):
        want[idx] = base[idx] + g[idx[0], idx[3], idx[2], idx[1]]
    got = base.copy()
    K.transpose_backward_into(g, 1, 3, got)
    np.testing.assert_array_equal(got, want)


# ---------------------------------------------------------------------------
# Mul / Exp / Log / Rsqrt / Softmax: float64 closed forms, explicit loops,
# finite differences
# ---------------------------------------------------------------------------
def test_mul_gradients_match_the_index_loops():
    rng = np.random.default_rng(SEED + 80)
    x = rng.standard_normal((3, 4, 5)).astype(np.float32)
    g = rng.standard_normal((3, 4, 5)).astype(np.float32)
    for yshape in [(3, 4, 5), (5,), (3, 4, 1), (1,)]:
        y = rng.standard_normal(yshape).astype(np.float32)
        np.testing.assert_array_equal(K.mul_forward(x, y), x * y)
        dx0 = rng.standard_normal(x.shape).astype(np.float32)
        dy0 = rng.standard_normal(yshape).astype(np.float32)
        dx, dy = dx0.copy(), dy0.copy()
        K.mul_backward_into(g, x, y, dx=dx, dy=dy)
        yb = np.broadcast_to(y, x.shape)
        want_dx = dx0.astype(np.float64)
        want_dy = dy0.astype(np.float64).copy()
        for idx in np.ndindex(*x.shape):
            want_dx[idx] += float(g[idx]) * float(yb[idx])
            if yshape == x.shape:
                want_dy[idx] += float(g[idx]) * float(x[idx])
            elif yshape == (5,):
                want_dy[idx[2]] += float(g[idx]) * float(x[idx])
            elif yshape == (3, 4, 1):
                want_dy[idx[0], idx[1], 0] += float(g[idx]) * float(x[idx])
            else:
                want_dy[0] += float(g[idx]) * float(x[idx])
        np.testing.assert_allclose(dx, want_dx, rtol=1e-6, atol=1e-6)
        np.testing.assert_allclose(dy, want_dy, rtol=1e-5, atol=1e-5)
    with pytest.raises(RuntimeError):
        K.mul_kind((3, 4, 5), (4, 5))


def test_unary_primitives_against_float64_and_finite_differences():
    rng = np.random.default_rng(SEED + 81)
    x = rng.uniform(0.1, 3.0, (7, 9)).astype(np.float32)
    dy = rng.standard_normal((7, 9)).astype(np.float32)
    x64 = x.astype(np.float64)
    cases = [
        (K.exp_forward, K.exp_backward_into, True, np.exp, np.exp),
        (K.log_forward, K.log_backward_into, False, np.log, lambda v: 1.0 / v),
        (K.rsqrt_forward, K.rsqrt_backward_into, True, lambda v: v ** -0.5, lambda v: -0.5 * v ** -1.5),
    ]
    for fwd, bwd, saves_y, f64, d64 in cases:
        y = fwd(x)
        assert y.dtype == np.float32
        np.testing.assert_allclose(y, f64(x64), rtol=2e-7, atol=0)
        dx = np.zeros_like(x)
        bwd(dy, y if saves_y else x, dx)
        np.testing.assert_allclose(dx, dy * d64(x64), rtol=1e-6, atol=1e-7)
        h = 1e-4                                   # central difference of the float64 function
        fd = (f64(x64 + h) - f64(x64 - h)) / (2 * h)
        np.testing.assert_allclose(d64(x64), fd, rtol=1e-6, atol=1e-7)
    # rsqrt is sqrt then reciprocal, each correctly rounded (backend.py:342-345)
    np.testing.assert_array_equal(K.rsqrt_forward(x), np.float32(1.0) / np.sqrt(x))


def test_softmax_against_scipy_and_its_jacobian():
    from scipy.special import softmax as sp_softmax
    rng = np.random.default_rng(SEED + 82)
    x = (4.0 * rng.standard_normal((5, 6, 33))).astype(np.float32)
    g = rng.standard_normal(x.shape).astype(np.float32)
    y = K.softmax_forward(x)
    want = sp_softmax(x.astype(np.float64), axis=-1)
    np.testing.assert_allclose(y, want, rtol=2e-6, atol=1e-8)
    np.testing.assert_allclose(y.sum(-1), 1.0, rtol=0, atol=2e-6)
    # invariance to a per-row shift, and a row of equal logits gives 1/V
    np.testing.assert_allclose(K.softmax_forward(x + np.float32(3.0)), y, rtol=3e-6, atol=1e-8)
    np.testing.assert_allclose(K.softmax_forward(np.full((2, 8), 1.5, np.float32)), 0.125, rtol=1e-7)
    dx = np.zeros_like(x)
    K.softmax_backward_into(y, g, dx)
    # J = diag(y) - y y^T, dx = J g, written out per row in float64
    for r in np.ndindex(*x.shape[:-1]):
        yr, gr = want[r], g[r].astype(np.float64)
        J = np.diag(yr) - np.outer(yr, yr)
        np.testing.assert_allclose(dx[r], J @ gr, rtol=2e-5, atol=2e-7)
    np.testing.assert_allclose(dx.sum(-1), 0.0, atol=2e-6)      # rows of J sum to zero
    # masked logits: exp(-inf) = 0 and no NaN
    xm = x.copy()
    xm[..., 5:9] = -np.inf
    ym = K.softmax_forward(xm)
    assert np.isfinite(ym).all() and not ym[..., 5:9].any()
