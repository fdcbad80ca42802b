"""Float64 closed forms and numerical derivatives, independent of cpu_ops.

TEST INFRASTRUCTURE ONLY (same rule as cpu_ops.py).  These are the textbook
formulas, written the way the reference's own checkers write them
(verify_model.py:65-77, 127-135; debug/check_qwen_kernel.py:195-211, 258-324,
593-598, 626-629), evaluated in float64.  tests/test_oracle.py holds cpu_ops to
them; the GPU tests use them to report error against the exact value where the
fp32 CPU result itself carries rounding noise (row-summed parameter grads).
"""
from __future__ import annotations

import numpy as np


def f64(a):
    return np.asarray(a, dtype=np.float64)


def gelu(x):
    x = f64(x)
    return 0.5 * x * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x + 0.044715 * x ** 3)))


def gelu_grad(x):
    x = f64(x)
    k = np.sqrt(2.0 / np.pi)
    t = np.tanh(k * (x + 0.044715 * x ** 3))
    return 0.5 * (1.0 + t) + 0.5 * x * (1.0 - t * t) * k * (1.0 + 3 * 0.044715 * x * x)


def relu2(x):
    x = f64(x)
    return np.where(x > 0, x * x, 0.0)


def relu2_grad(x):
    x = f64(x)
    return np.where(x > 0, 2.0 * x, 0.0)


def layernorm(x, gamma, beta, eps):
    x = f64(x)
    mean = x.mean(axis=-1, keepdims=True)
    var = x.var(axis=-1, keepdims=True)
    inv_std = 1.0 / np.sqrt(var + eps)
    x_hat = (x - mean) * inv_std
    return x_hat * f64(gamma) + f64(beta), inv_std, x_hat


def layernorm_grads(x, gamma, dy, eps):
    _, inv_std, x_hat = layernorm(x, gamma, np.zeros_like(f64(gamma)), eps)
    dy = f64(dy)
    lead = tuple(range(dy.ndim - 1))
    dgamma = (dy * x_hat).sum(axis=lead)
    dbeta = dy.sum(axis=lead)
    a = dy * f64(gamma)
    dx = inv_std * (a - a.mean(axis=-1, keepdims=True) - x_hat * (a * x_hat).mean(axis=-1, keepdims=True))
    return dx, dgamma, dbeta


def rmsnorm(x, gamma, eps):
    x = f64(x)
    inv = 1.0 / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)
    x_hat = x * inv
    z = x_hat if gamma is None else x_hat * f64(gamma)
    return z, inv, x_hat


def rmsnorm_grads(x, gamma, dz, eps):
    _, inv, x_hat = rmsnorm(x, gamma, eps)
    dz = f64(dz)
    lead = tuple(range(dz.ndim - 1))
    dgamma = (dz * x_hat).sum(axis=lead)
    d = dz if gamma is None else dz * f64(gamma)
    dx = inv * (d - x_hat * (d * x_hat).mean(axis=-1, keepdims=True))
    return dx, dgamma


def swiglu(gu):
    gu = f64(gu)
    H = gu.shape[-1] // 2
    g, u = gu[..., :H], gu[..., H:]
    s = 1.0 / (1.0 + np.exp(-g))
    return g * s * u


def swiglu_grads(gu, dh):
    gu = f64(gu)
    dh = f64(dh)
    H = gu.shape[-1] // 2
    g, u = gu[..., :H], gu[..., H:]
    s = 1.0 / (1.0 + np.exp(-g))
    dg = dh * u * s * (1.0 + g * (1.0 - s))
    du = dh * g * s
    return np.concatenate((dg, du), axis=-1)


def rope(x, cos, sin, rope_sign, backward=False):
    """x [B,T,H,D]; rotation by +angle for rope_sign=+1 (HF), -angle for -1;
    backward applies the transpose."""
    x = f64(x)
    half = x.shape[-1] // 2
    c = f64(cos)[None, : x.shape[1], None, :]
    s = f64(sin)[None, : x.shape[1], None, :] * (rope_sign if not backward else -rope_sign)
    lo, hi = x[..., :half], x[..., half:]
    return np.concatenate((lo * c - hi * s, hi * c + lo * s), axis=-1)


def gather_backward(ids, dY, V):
    """Row loop in row order, float64 accumulation."""
    dY = f64(dY).reshape(-1, dY.shape[-1])
    dW = np.zeros((V, dY.shape[-1]), dtype=np.float64)
    for n, t in enumerate(np.asarray(ids).ravel()):
        dW[int(t)] += dY[n]
    return dW


def finite_diff(fn, x, idxs, eps=1e-3):
    """Central differences of scalar fn at flat positions idxs of float64 x
    (verify_model.py:65-77)."""
    x = f64(x).copy()
    flat = x.reshape(-1)
    out = np.empty(len(idxs), dtype=np.float64)
    for j, i in enumerate(idxs):
        orig = flat[i]
        flat[i] = orig + eps
        plus = float(fn(x))
        flat[i] = orig - eps
        minus = float(fn(x))
        flat[i] = orig
        out[j] = (plus - minus) / (2.0 * eps)
    return out


def adamw_reference(p0, grads, lr, b1, b2, eps, weight_decay):
    """Textbook AdamW in float64 (Loshchilov & Hutter, with the bias correction
    folded into the step size the way the reference folds it, optimizer.py:445):
    returns the parameters after len(grads) steps and the final moments."""
    p = f64(p0).copy()
    m = np.zeros_like(p)
    v = np.zeros_like(p)
    for t, g in enumerate(grads, start=1):
        g = f64(g)
        p = p * (1.0 - lr * weight_decay)
        m = b1 * m + (1.0 - b1) * g
        v = b2 * v + (1.0 - b2) * g * g
        lr_t = lr * np.sqrt(1.0 - b2 ** t) / (1.0 - b1 ** t)
        p = p - lr_t * m / (np.sqrt(v) + eps)
    return p, m, v


def cross_entropy(x, labels):
    """-log softmax(x)[label] in float64 through scipy's logsumexp"""
    from scipy.special import logsumexp
    x = f64(x)
    picked = np.take_along_axis(x, np.asarray(labels, np.int64)[..., None], axis=-1)[..., 0]
    return logsumexp(x, axis=-1) - picked


def cross_entropy_grad(x, labels, dloss):
    from scipy.special import softmax
    p = softmax(f64(x), axis=-1)
    onehot = np.zeros_like(p)
    np.put_along_axis(onehot, np.asarray(labels, np.int64)[..., None], 1.0, axis=-1)
    return (p - onehot) * f64(dloss)[..., None]
