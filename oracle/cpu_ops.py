"""CPU restatement of the reference's fused layer-op kernels (numpy, fp32).

TEST INFRASTRUCTURE ONLY.  This module is the checker for the HIP kernels: it is
imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of
bench.py, and by nothing in the autograd_amd package.

Each function performs the same sequence of whole-array fp32 numpy operations
as the reference function it cites (every step rounds to fp32, no FMA), so its
results are what the reference's "cpu" device produces with the same numpy.
Citations are file:line in the reference repository.

Pinning (what shows these functions are the right functions; tests/test_oracle.py):
  * layernorm / gelu: the reference's own independent numpy oracles
    (verify_model.py:127-135 restated in oracle/closed_form.py), float64 closed
    forms, finite differences, row invariants.
  * rmsnorm / swiglu / rope: the closed forms of debug/check_qwen_kernel.py:195-342,
    577-645 (restated in float64), finite differences, rotation invariants.
  * gather: numpy fancy indexing; backward: brute-force row loop.
  * bf16: bit-exact against an exhaustive integer restatement of utils.py:20-27.
  * cross-entropy: scipy.special.logsumexp / softmax in float64, finite
    differences, rows of the gradient sum to zero, uniform logits give log V.
  * strided views / permute gradients: an explicit loop over every dense index
    with the index arithmetic written out, on small shapes.
  * mul / exp / log / rsqrt / softmax: float64 closed forms (scipy.special.softmax,
    the softmax Jacobian written out), explicit index loops for the broadcast sums
    of the mul gradient, finite differences, rows of a softmax sum to one.
  * bias_gelu: the float64 closed form of GELU at h + b, finite differences in h and in b,
    an explicit row loop for the bias gradient.
  * adamw8bit: the maps against their defining properties (256 sorted values, extremes
    -1 / 0 / 1, seven decades), nearest_code against a brute-force argmin over all 256
    entries, and several steps against fp32-moment AdamW within the quantisation bound.
  * adamw: the textbook bias-corrected recurrence in float64 over several steps;
    the first step from zero moments moves every weight by lr * sign(g).
Parity unpinned by the reference:
  * adamw8bit_step -- the reference runs it on its GPU only and keeps no vectors for
    it; pinned by the properties above, not by reference outputs.
  * relu2_* -- the reference has no ReLU^2; pinned by its closed form only.
  * d(gamma), d(beta) at large row counts -- numpy sums rows sequentially in
    fp32 (backend.py:461,466); the value is pinned, its rounding noise (~1e-4
    absolute at N = 16384) is numpy behaviour that no GPU reduction order
    reproduces bit for bit.
"""
from __future__ import annotations

import numpy as np

F32 = np.float32

# backend.py:18-20
GELU_C = 0.7978845608028654
GELU_A = 0.044715
GELU_A3 = 0.134145


# --------------------------------------------------------------------------
# Add  (cpu_add_forward / cpu_add_backward, backend.py:74-105)
# --------------------------------------------------------------------------
def add_forward(x, y):
    return np.add(x, y)


def add_backward_into(g, grad):
    """grad += g, summing g over the leading axes it was broadcast along."""
    if g.shape == grad.shape:
        np.add(grad, g, out=grad)
        return
    lead = g.ndim - grad.ndim
    padded = (1,) * lead + grad.shape
    axes = tuple(i for i, (gi, ti) in enumerate(zip(g.shape, padded)) if ti == 1 and gi != 1)
    tmp = np.sum(g, axis=axes) if axes else g
    np.add(grad, tmp.reshape(grad.shape), out=grad)


# --------------------------------------------------------------------------
# Mul  (cpu_mul_forward / cpu_mul_backward, backend.py:107-146; mul_bcast_kind,
# utils.py:134-143)
# --------------------------------------------------------------------------
def mul_kind(x_shape, y_shape):
    x_shape, y_shape = tuple(x_shape), tuple(y_shape)
    if len(y_shape) == 0 or int(np.prod(y_shape)) == 1:
        return "scalar"
    if len(y_shape) == 1 and x_shape[-1] == y_shape[0]:
        return "row"
    if len(y_shape) == len(x_shape) and y_shape[:-1] == x_shape[:-1] and y_shape[-1] == 1:
        return "col"
    if y_shape == x_shape:
        return "same"
    raise RuntimeError(f"Mul backward: unsupported broadcast x={x_shape} y={y_shape}")


def mul_forward(x, y):
    return np.multiply(x, y)


def mul_backward_into(g, x, y, dx=None, dy=None):
    kind = mul_kind(g.shape, y.shape)
    if dx is not None:
        if kind == "scalar":
            s = y.reshape(())
            np.add(dx, g if s == 1 else np.multiply(g, s, dtype=g.dtype), out=dx)
        else:
            np.add(dx, np.multiply(g, y, dtype=g.dtype), out=dx)
    if dy is None:
        return
    full = np.multiply(g, x, dtype=dy.dtype)
    if kind == "scalar":
        red = np.empty(dy.shape, dy.dtype)
        red[...] = np.sum(full, dtype=dy.dtype)
    elif kind == "row":
        red = np.sum(full, axis=tuple(range(g.ndim - 1)))
    elif kind == "col":
        red = np.sum(full, axis=-1, keepdims=True)
    else:
        red = full
    np.add(dy, red.reshape(dy.shape), out=dy)


# --------------------------------------------------------------------------
# Exp, Log, Rsqrt, Softmax  (backend.py:320-374)
# --------------------------------------------------------------------------
def exp_forward(x):
    return np.exp(x)


def exp_backward_into(dy, y, dx):
    np.add(dx, dy * y, out=dx)


def log_forward(x):
    return np.log(x)


def log_backward_into(dy, x, dx):
    np.add(dx, dy / x, out=dx)


def rsqrt_forward(x):
    t = np.sqrt(x)
    return np.reciprocal(t)


def rsqrt_backward_into(dy, y, dx):
    np.add(dx, dy * (-0.5) * y * y * y, out=dx)


def softmax_forward(x, axis=-1):
    m = np.max(x, axis=axis, keepdims=True)
    e = np.subtract(x, m)
    np.exp(e, out=e)
    s = np.sum(e, axis=axis, keepdims=True)
    np.divide(e, s, out=e)
    return e


def softmax_backward_into(y, g, dx, axis=-1):
    t = np.multiply(g, y)
    dot = np.sum(t, axis=axis, keepdims=True)
    np.subtract(g, dot, out=t)
    np.multiply(y, t, out=t)
    np.add(dx, t, out=dx)


# --------------------------------------------------------------------------
# Views and layout changes  (tensor_to_numpy, utils.py:111-125;
# cpu_permute_backward / cpu_transpose_backward / cpu_contiguous_forward,
# backend.py:286-313)
# --------------------------------------------------------------------------
def strided_view(flat, shape, strides, offset=0):
    """the [shape] view of the flat buffer that starts `offset` elements in and
    steps `strides` elements per dimension"""
    flat = flat.reshape(-1)[offset:]
    byte_strides = tuple(int(s) * flat.itemsize for s in strides)
    return np.lib.stride_tricks.as_strided(flat, shape=tuple(shape), strides=byte_strides, writeable=False)


def contiguous_forward(flat, shape, strides, offset=0):
    return np.ascontiguousarray(strided_view(flat, shape, strides, offset))


def permute_backward_into(g_out, dims, grad):
    """grad += g_out with the permutation undone (out.shape[i] = x.shape[dims[i]])"""
    inv = [0] * len(dims)
    for i, d in enumerate(dims):
        inv[d] = i
    np.add(grad, np.ascontiguousarray(np.transpose(g_out, inv)), out=grad)


def transpose_backward_into(g_out, dim0, dim1, grad):
    np.add(grad, np.ascontiguousarray(np.swapaxes(g_out, dim0, dim1)), out=grad)


# --------------------------------------------------------------------------
# GELU-tanh  (cpu_gelu_forward / cpu_gelu_backward, backend.py:376-414)
# --------------------------------------------------------------------------
def _gelu_tanh(x):
    b = np.multiply(x, x)
    np.multiply(b, x, out=b)
    np.multiply(b, GELU_A, out=b)
    np.add(x, b, out=b)
    np.multiply(b, GELU_C, out=b)
    np.tanh(b, out=b)
    return b


def gelu_forward(x):
    b = _gelu_tanh(x)
    np.add(b, 1.0, out=b)
    np.multiply(x, b, out=b)
    return np.multiply(b, 0.5)


def gelu_backward_into(x, dy, dx):
    t = _gelu_tanh(x)
    a = np.multiply(t, t)
    np.subtract(1.0, a, out=a)
    d_inner = GELU_C * (1.0 + GELU_A3 * x * x)
    np.multiply(a, 0.5 * x * d_inner, out=a)
    np.add(t, 1.0, out=t)
    np.multiply(t, 0.5, out=t)
    np.add(t, a, out=t)
    np.multiply(dy, t, out=a)
    np.add(dx, a, out=dx)


def bias_gelu_forward(h, b):
    """GELU(h + b): cpu_add_forward (backend.py:74-88) then cpu_gelu_forward (backend.py:376-395);
    the sum is what gelu_add_bias_kernel forms per element (metal_ops.metal:3746-3747)"""
    return gelu_forward(np.add(h, b))


def bias_gelu_backward_into(h, b, dy, dh=None, db=None):
    """dh += dy * GELU'(h + b) (cpu_gelu_backward, backend.py:396-414); db += the same terms
    summed over the leading axes (cpu_add_backward's reduction, backend.py:89-105)"""
    term = np.zeros_like(np.asarray(h, dtype=np.float32))
    gelu_backward_into(np.add(h, b), dy, term)
    if dh is not None:
        np.add(dh, term, out=dh)
    if db is not None:
        add_backward_into(term, db)


# --------------------------------------------------------------------------
# ReLU^2  (no reference counterpart: y = max(x,0)^2, dx += 2 max(x,0) dy)
# --------------------------------------------------------------------------
def relu2_forward(x):
    r = np.maximum(x, F32(0))
    return np.multiply(r, r)


def relu2_backward_into(x, dy, dx):
    r = np.maximum(x, F32(0))
    np.multiply(r, F32(2), out=r)
    np.multiply(r, dy, out=r)
    np.add(dx, r, out=dx)


# --------------------------------------------------------------------------
# LayerNorm  (cpu_layernorm_forward / backward, backend.py:416-487)
# --------------------------------------------------------------------------
def _ln_stats(x, eps):
    """returns (inv_std [.., 1], x_hat) computed as backend.py:420-430 does."""
    r = np.mean(x, axis=-1, keepdims=True)
    f = np.subtract(x, r)
    np.multiply(f, f, out=f)
    np.mean(f, axis=-1, keepdims=True, out=r)
    np.add(r, eps, out=r)
    np.sqrt(r, out=r)
    np.reciprocal(r, out=r)
    np.subtract(x, np.mean(x, axis=-1, keepdims=True), out=f)
    np.multiply(f, r, out=f)
    return r, f


def layernorm_forward(x, gamma, beta, eps):
    _, f = _ln_stats(x, eps)
    y = np.multiply(f, gamma)
    np.add(y, beta, out=y)
    return y


def layernorm_backward_into(x, gamma, dy, eps, dx=None, dgamma=None, dbeta=None):
    inv_std, x_hat = _ln_stats(x, eps)
    lead = tuple(range(x.ndim - 1))
    if dgamma is not None:
        f2 = np.multiply(dy, x_hat)
        tmp = np.sum(f2, axis=lead)
        np.add(dgamma, tmp.reshape(dgamma.shape), out=dgamma)
    if dbeta is not None:
        tmp = np.sum(dy, axis=lead)
        np.add(dbeta, tmp.reshape(dbeta.shape), out=dbeta)
    if dx is not None:
        f2 = np.multiply(dy, gamma)
        f3 = np.multiply(f2, inv_std)
        np.add(dx, f3, out=dx)
        r2 = np.mean(f2, axis=-1, keepdims=True)
        np.multiply(r2, inv_std, out=r2)
        np.subtract(dx, r2, out=dx)
        np.multiply(f2, x_hat, out=f2)
        np.mean(f2, axis=-1, keepdims=True, out=r2)
        np.multiply(r2, inv_std, out=r2)
        np.multiply(x_hat, r2, out=f3)
        np.subtract(dx, f3, out=dx)


# --------------------------------------------------------------------------
# RMSNorm  (slices of the fused ops: forward backend.py:1097-1108, 1737-1745;
#           backward backend.py:1228-1251, 1990-2011)
# --------------------------------------------------------------------------
def _rms_inv(x, eps):
    t = np.multiply(x, x)
    inv = np.mean(t, axis=-1, keepdims=True)
    np.add(inv, F32(eps), out=inv)
    np.sqrt(inv, out=inv)
    np.reciprocal(inv, out=inv)
    return inv


def rmsnorm_forward(x, gamma, eps):
    inv = _rms_inv(x, eps)
    z = np.multiply(x, inv)
    if gamma is not None:
        np.multiply(z, gamma, out=z)
    return z


def rmsnorm_backward_into(x, gamma, dz, eps, dx=None, dgamma=None):
    """backend.py:1990-2011 (weighted) / 1228-1251 (gamma optional)."""
    inv = _rms_inv(x, eps)
    x_hat = np.multiply(x, inv)
    lead = tuple(range(x.ndim - 1))
    if dgamma is not None:
        t = np.multiply(dz, x_hat)
        tmp = np.sum(t, axis=lead)
        np.add(dgamma, tmp, out=dgamma)
    if dx is not None:
        d = np.multiply(dz, gamma) if gamma is not None else np.array(dz, copy=True)
        t = np.multiply(d, x_hat)
        m = np.mean(t, axis=-1, keepdims=True)
        np.multiply(x_hat, m, out=t)
        np.subtract(d, t, out=t)
        np.multiply(t, inv, out=t)
        np.add(dx, t, out=dx)


# --------------------------------------------------------------------------
# residual add fused with a norm: cpu_add_forward then the norm; backward is
# the norm backward accumulated onto the gradient already sitting on h, then
# cpu_add_backward hands that gradient to both operands (backend.py:74-105).
# --------------------------------------------------------------------------
def add_norm_forward(kind, x, res, gamma, beta, eps):
    h = add_forward(x, res)
    if kind == "layer":
        return h, layernorm_forward(h, gamma, beta, eps)
    return h, rmsnorm_forward(h, gamma, eps)


# --------------------------------------------------------------------------
# SwiGLU  (forward backend.py:1113-1126; backward backend.py:1180-1217)
# --------------------------------------------------------------------------
def _sigmoid_ref(g):
    s = np.negative(g)
    np.exp(s, out=s)
    np.add(s, 1.0, out=s)
    np.reciprocal(s, out=s)
    return s


def swiglu_forward(gu):
    H = gu.shape[-1] // 2
    g, u = gu[..., :H], gu[..., H:]
    with np.errstate(over="ignore"):
        h = _sigmoid_ref(g)
    np.multiply(g, h, out=h)
    np.multiply(h, u, out=h)
    return h


def swiglu_backward(gu, dh):
    """returns dgu = [dg | du] (the reference overwrites gu with it)."""
    H = gu.shape[-1] // 2
    g, u = gu[..., :H], gu[..., H:]
    with np.errstate(over="ignore"):
        s = _sigmoid_ref(g)
    dgu = np.empty_like(gu)
    dg, du = dgu[..., :H], dgu[..., H:]
    np.subtract(1.0, s, out=dg)
    np.multiply(dg, g, out=dg)
    np.add(dg, 1.0, out=dg)
    np.multiply(dg, s, out=dg)
    np.multiply(dg, u, out=dg)
    np.multiply(dg, dh, out=dg)
    np.multiply(g, s, out=du)
    np.multiply(du, dh, out=du)
    return dgu


# --------------------------------------------------------------------------
# RoPE
# --------------------------------------------------------------------------
def rope_tables(T, D, theta):
    """module.py:247-255: fp32 tables cos/sin[T, D/2]."""
    pos = np.arange(T, dtype=np.float32)[:, None]
    ch = np.arange(0, D, 2, dtype=np.float32)[None, :]
    inv = np.float32(theta) ** (-ch / np.float32(D))
    f = pos * inv
    return np.cos(f).astype(np.float32), np.sin(f).astype(np.float32)


def rope_nanochat(q, k, cos, sin, backward=False):
    """apply_rope_np / apply_rope_backward_np (backend.py:1382-1417); q, k are
    [B, T, H, D] and are rotated in place."""
    d2 = q.shape[-1] // 2
    c = cos[None, :, None, :]
    s = sin[None, :, None, :]
    for a in (q, k):
        if a is None:
            continue
        a1 = a[..., :d2].copy()
        a2 = a[..., d2:].copy()
        if not backward:
            a[..., :d2] = a1 * c + a2 * s
            a[..., d2:] = -a1 * s + a2 * c
        else:
            a[..., :d2] = a1 * c - a2 * s
            a[..., d2:] = a1 * s + a2 * c


def rope_signed(q, k, cos, sin, rope_sign, backward=False):
    """The GQA loops (forward backend.py:1761-1782, backward 1938-1958): per
    (batch, head) slice, in place, with the rope_sign convention (+1 = HF)."""
    half = q.shape[-1] // 2
    T = q.shape[1]
    cos = cos[:T]
    sin = sin[:T]
    plus = (rope_sign == 1) != backward  # True: lo' = p - q, hi' = hi*c + lo*s
    r0 = np.empty((T, half), dtype=np.float32)
    r1 = np.empty((T, half), dtype=np.float32)
    for data in (q, k):
        if data is None:
            continue
        for b in range(data.shape[0]):
            for h in range(data.shape[2]):
                lo = data[b, :, h, :half]
                hi = data[b, :, h, half:]
                np.multiply(lo, cos, out=r0)
                np.multiply(hi, sin, out=r1)
                if plus:
                    np.subtract(r0, r1, out=r0)
                else:
                    np.add(r0, r1, out=r0)
                np.multiply(lo, sin, out=r1)
                np.multiply(hi, cos, out=hi)
                if plus:
                    np.add(hi, r1, out=hi)
                else:
                    np.subtract(hi, r1, out=hi)
                np.copyto(lo, r0)


# --------------------------------------------------------------------------
# Cross-entropy over the last axis  (cpu_crossentropy_forward / backward,
# backend.py:489-524)
# --------------------------------------------------------------------------
def cross_entropy_forward(x, labels):
    """x [..., V] fp32, labels [...] int -> loss [...]"""
    r = np.max(x, axis=-1, keepdims=True)
    f = np.subtract(x, r)
    e = np.exp(f)
    np.sum(e, axis=-1, keepdims=True, out=r)
    np.log(r, out=r)
    np.subtract(f, r, out=f)
    idx = labels.astype(np.int64)
    gathered = np.take_along_axis(f, idx[..., None], axis=-1)[..., 0]
    return np.negative(gathered)


def cross_entropy_backward_into(x, labels, dloss, dx):
    """dx += (softmax(x) - onehot(labels)) * dloss[..., None]"""
    r = np.max(x, axis=-1, keepdims=True)
    f = np.subtract(x, r)
    np.exp(f, out=f)
    np.sum(f, axis=-1, keepdims=True, out=r)
    np.divide(f, r, out=f)
    V = x.shape[-1]
    flat = f.reshape(-1, V)
    flat[np.arange(flat.shape[0]), labels.astype(np.int64).ravel()] -= 1.0
    np.multiply(f, dloss[..., None], out=f)
    np.add(dx, f, out=dx)


def cross_entropy_fused(x, targets, scale, row_scale=None, write_grad=True):
    """The one-kernel form behind the reference's output projection
    (fused_linear_ce_logits_to_dlogits, metal_ops.metal:8808-8996; row-scaled :8997-9152): returns
    (row_loss, lse, dlogits) for logits x [rows, V] and int targets [rows].  A row whose target lies
    outside [0, V) (an ignored position, metal_ops.metal:8919-8926) or that has no finite logit has
    loss 0, lse 0 and a zero gradient row; every other row is the composition of
    cross_entropy_forward and cross_entropy_backward_into with dloss = scale (or row_scale[r])."""
    x = np.asarray(x, np.float32)
    rows, V = x.shape
    t = np.asarray(targets).astype(np.int64)
    ok = (t >= 0) & (t < V) & np.isfinite(np.max(x, axis=-1))
    safe = np.where(ok, t, 0)
    xs = np.where(ok[:, None], x, np.float32(0.0)).astype(np.float32)
    loss = cross_entropy_forward(xs, safe)
    m = np.max(xs, axis=-1)
    lse = (m + np.log(np.sum(np.exp(xs - m[:, None]), axis=-1, dtype=np.float32))).astype(np.float32)
    loss = np.where(ok, loss, np.float32(0.0)).astype(np.float32)
    lse = np.where(ok, lse, np.float32(0.0)).astype(np.float32)
    if not write_grad:
        return loss, lse, None
    dl = (np.full(rows, scale, np.float32) if row_scale is None else np.asarray(row_scale, np.float32))
    dx = np.zeros_like(xs)
    cross_entropy_backward_into(xs, safe, dl, dx)
    dx[~ok] = 0.0
    return loss, lse, dx


# --------------------------------------------------------------------------
# AdamW  (cpu_adamw_step, backend.py:2013-2038; the step size lr_t comes from
# optimizer.py:445)
# --------------------------------------------------------------------------
def adamw_step(p, g, m, v, lr, lr_t, b1, b2, eps, weight_decay):
    """In place on p, m, v (fp32 arrays); g is read.  Python-float scalars meet
    fp32 arrays, so each scalar is rounded to fp32 once and every numpy call
    rounds its result once."""
    tmp = np.empty_like(p)
    if weight_decay > 0.0:
        np.multiply(p, lr * weight_decay, out=tmp)
        np.subtract(p, tmp, out=p)
    np.multiply(m, b1, out=m)
    np.multiply(g, 1.0 - b1, out=tmp)
    np.add(m, tmp, out=m)
    np.multiply(v, b2, out=v)
    np.multiply(g, g, out=tmp)
    np.multiply(tmp, 1.0 - b2, out=tmp)
    np.add(v, tmp, out=v)
    np.sqrt(v, out=tmp)
    np.add(tmp, eps, out=tmp)
    np.divide(m, tmp, out=tmp)
    np.multiply(tmp, lr_t, out=tmp)
    np.subtract(p, tmp, out=p)


def adamw_step_split(p, g, m, v, lr_wd, b1, b2, eps, step_lr, inv_sqrt_bc2, grad_scale, decay_numel=None):
    """The same sequence with the Metal kernel's extra factors (adamw_step,
    metal_ops.metal:10139-10228): the gradient times grad_scale, sqrt(v) times
    inv_sqrt_bc2 before eps, weight decay on the first decay_numel elements."""
    g = np.multiply(g, F32(grad_scale)) if grad_scale != 1.0 else g
    tmp = np.empty_like(p)
    if lr_wd != 0.0:
        n = p.size if decay_numel is None else decay_numel
        flat = p.reshape(-1)
        np.multiply(flat[:n], lr_wd, out=tmp.reshape(-1)[:n])
        np.subtract(flat[:n], tmp.reshape(-1)[:n], out=flat[:n])
    np.multiply(m, b1, out=m)
    np.multiply(g, 1.0 - b1, out=tmp)
    np.add(m, tmp, out=m)
    np.multiply(v, b2, out=v)
    np.multiply(g, g, out=tmp)
    np.multiply(tmp, 1.0 - b2, out=tmp)
    np.add(v, tmp, out=v)
    np.sqrt(v, out=tmp)
    if inv_sqrt_bc2 != 1.0:
        np.multiply(tmp, inv_sqrt_bc2, out=tmp)
    np.add(tmp, eps, out=tmp)
    np.divide(m, tmp, out=tmp)
    np.multiply(tmp, step_lr, out=tmp)
    np.subtract(p, tmp, out=p)


# --------------------------------------------------------------------------
# AdamW with 8-bit moments  (adamw8bit_step, metal_ops.metal:10229-10361; the
# maps of optimizer.py:144-179).  The reference has this path on its GPU only:
# what follows restates that kernel, one numpy call per rounded operation.
# --------------------------------------------------------------------------
def dynamic_map(signed, max_exponent_bits=7, total_bits=8):
    """The 256 sorted code values of bitsandbytes' "dynamic" 8-bit format as the
    reference builds them (optimizer.py:144-179): for each of 7 decades a linear
    run of bin centres whose length doubles per decade, one finer run below the
    last decade, zero, sorted and scaled so that the largest magnitude is 1."""
    non_sign_bits = total_bits - 1 if signed else total_bits
    additional_items = 2 ** (non_sign_bits - max_exponent_bits) - 1
    values = []
    for exponent in range(max_exponent_bits):
        fraction_items = 2 ** (exponent + non_sign_bits - max_exponent_bits) + 1
        boundaries = np.linspace(0.1, 1.0, fraction_items, dtype=F32)
        means = (boundaries[:-1] + boundaries[1:]) * F32(0.5)
        scaled = means * F32(10.0 ** (exponent - (max_exponent_bits - 1)))
        values.extend(scaled.tolist())
        if signed:
            values.extend((-scaled).tolist())
    if additional_items > 0:
        boundaries = np.linspace(0.0, 0.1, additional_items + 1, dtype=F32)
        means = (boundaries[:-1] + boundaries[1:]) * F32(0.5)
        scaled = means * F32(10.0 ** (-(max_exponent_bits - 1)))
        values.extend(scaled.tolist())
        if signed:
            values.extend((-scaled).tolist())
    values.append(0.0)
    while len(values) < (1 << total_bits):      # the signed map has two zero codes
        values.append(0.0)
    if len(values) != (1 << total_bits):
        raise RuntimeError(f"invalid dynamic-map size: {len(values)}")
    qmap = np.asarray(values, dtype=F32)
    qmap.sort()
    qmap /= np.max(np.abs(qmap))
    return np.ascontiguousarray(qmap, dtype=F32)


def nearest_code(qmap, x):
    """metal_ops.metal:10326-10343: the first entry not below x (bisection over the
    sorted map, never past the last entry), then the nearer of it and the entry below;
    a tie takes the lower"""
    upper = np.minimum(np.searchsorted(qmap, x, side="left"), 255)
    lower = np.where(upper > 0, upper - 1, 0)
    take_upper = np.abs(qmap[upper] - x) < np.abs(qmap[lower] - x)
    return np.where(take_upper, upper, lower).astype(np.uint8)


def adamw8bit_step(p, g, qm, qv, absmax_m, absmax_v, qmap_m, qmap_v, decay, lr_bc1, b1, b2, eps,
                   decay_numel, first_step, inv_sqrt_bc2, clip_coef=1.0):
    """In place on p (fp32), qm, qv (uint8), absmax_m, absmax_v (fp32, one per block
    of 256); g (fp32 values) is read.  Scalars are rounded to fp32 first, as kernel
    arguments are."""
    decay, lr_bc1, b1, b2, eps, inv_sqrt_bc2, clip_coef = (F32(x) for x in (decay, lr_bc1, b1, b2, eps, inv_sqrt_bc2, clip_coef))
    n = p.size
    flat_p = p.reshape(-1)
    blk = np.arange(n) // 256
    if first_step:
        m = np.zeros(n, F32)
        v = np.zeros(n, F32)
    else:
        m = np.multiply(absmax_m[blk], qmap_m[qm.reshape(-1)], dtype=F32)
        v = np.multiply(absmax_v[blk], qmap_v[qv.reshape(-1)], dtype=F32)
    gv = np.multiply(np.asarray(g, F32).reshape(-1), clip_coef, dtype=F32)
    factor = np.where(np.arange(n) < decay_numel, decay, F32(1.0)).astype(F32)
    pv = np.multiply(flat_p, factor, dtype=F32)
    dm = np.multiply(np.subtract(gv, m, dtype=F32), F32(1.0) - b1, dtype=F32)
    m = np.add(m, dm, dtype=F32)
    dv = np.multiply(np.subtract(np.multiply(gv, gv, dtype=F32), v, dtype=F32), F32(1.0) - b2, dtype=F32)
    v = np.add(v, dv, dtype=F32)
    denom = np.add(np.multiply(np.sqrt(np.maximum(v, F32(0.0)), dtype=F32), inv_sqrt_bc2, dtype=F32), eps, dtype=F32)
    dp = np.multiply(np.negative(np.divide(m, denom, dtype=F32)), lr_bc1, dtype=F32)
    flat_p[:] = np.add(pv, dp, dtype=F32)
    nblocks = (n + 255) // 256
    top_m = np.zeros(nblocks, F32)
    top_v = np.zeros(nblocks, F32)
    np.maximum.at(top_m, blk, np.abs(m))
    np.maximum.at(top_v, blk, np.maximum(v, F32(0.0)))
    absmax_m[:] = np.maximum(top_m, F32(1.0e-30))
    absmax_v[:] = np.maximum(top_v, F32(1.0e-30))
    mn = np.clip(np.divide(m, absmax_m[blk], dtype=F32), F32(-1.0), F32(1.0))
    vn = np.clip(np.divide(np.maximum(v, F32(0.0)), absmax_v[blk], dtype=F32), F32(0.0), F32(1.0))
    qm.reshape(-1)[:] = nearest_code(qmap_m, mn)
    qv.reshape(-1)[:] = nearest_code(qmap_v, vn)


def grad_norm_partials(g):
    """sum of squares of every 256-element group of g (grad_norm_sq,
    metal_ops.metal:10103-10137), in float64 so that it checks any fp32 order"""
    flat = np.asarray(g, dtype=np.float64).reshape(-1)
    pad = (-flat.size) % 256
    if pad:
        flat = np.concatenate([flat, np.zeros(pad)])
    return (flat * flat).reshape(-1, 256).sum(1)


# --------------------------------------------------------------------------
# Embedding  (cpu_gather_forward / backward, backend.py:525-538)
# --------------------------------------------------------------------------
def gather_forward(ids, W):
    return W[ids.astype(np.int64)]


def gather_backward_into(ids, dY, dW):
    np.add.at(dW, ids.astype(np.int64).ravel(), dY.reshape(-1, dW.shape[-1]))


def embedding_sum_forward(ids, wte, wpe):
    """x0 = tok_emb(ids) + pos_emb(pos_ids), pos_ids = tile(arange(T))
    (check_tiny_gpt2_kernel.py:282,301)."""
    B, T = ids.shape
    pos = np.tile(np.arange(T, dtype=np.int32), (B, 1))
    return add_forward(gather_forward(ids, wte), gather_forward(pos, wpe))


def embedding_sum_backward_into(ids, dY, dwte, dwpe):
    B, T = ids.shape
    pos = np.tile(np.arange(T, dtype=np.int32), (B, 1))
    if dwte is not None:
        gather_backward_into(ids, dY, dwte)
    if dwpe is not None:
        gather_backward_into(pos, dY, dwpe)


# --------------------------------------------------------------------------
# bf16 storage  (bf16_bits, utils.py:20-27; array form backend.py:5090-5113)
# --------------------------------------------------------------------------
def f32_to_bf16_bits(a):
    bits = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    rounded = (bits + np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    special = (bits & np.uint32(0x7F800000)) == np.uint32(0x7F800000)
    nan = special & ((bits & np.uint32(0x007FFFFF)) != np.uint32(0))
    special_bits = (bits >> np.uint32(16)) | np.where(nan, np.uint32(0x0040), np.uint32(0))
    return np.where(special, special_bits, rounded).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def round_bf16(a):
    """fp32 array rounded to the nearest bf16 value, returned as fp32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(a)).reshape(np.shape(a))
