"""numpy-in / numpy-out wrappers over the typed C-ABI entry points, for tests.

Every function uploads its operands, makes ONE call through the C ABI on the
session context, synchronises, and downloads the results.  bf16 operands are
passed and returned as uint16 bit arrays.
"""
import ctypes as C

import numpy as np

from autograd_amd import capi


def _dt(a):
    return capi.BF16 if np.dtype(a.dtype) == np.dtype(np.uint16) else capi.F32


def _p(d):
    return C.c_void_p(d.ptr) if d is not None else None


def _up(ctx, a):
    return None if a is None else ctx.upload(a)


def _free(*ds):
    for d in ds:
        if d is not None:
            d.free()


def norm_forward(ctx, kind, x, gamma, beta, eps, residual=None, want_h=False):
    rows = int(np.prod(x.shape[:-1]))
    Cw = x.shape[-1]
    dx, dr, dg, db = _up(ctx, x), _up(ctx, residual), _up(ctx, gamma), _up(ctx, beta)
    y = ctx.empty(x.shape, x.dtype)
    h = ctx.empty(x.shape, x.dtype) if want_h else None
    ctx.call("agrad_norm_forward", kind, _dt(x), _p(dx), _p(dr), _p(dg), _p(db), _p(h), _p(y), rows, Cw, eps)
    ctx.synchronize()
    out = y.download(), (h.download() if h is not None else None)
    _free(dx, dr, dg, db, y, h)
    return out


def norm_backward(ctx, kind, x, gamma, dy, eps, dres=None, dx_init=None, want_dx=True, want_dx2=False,
                  dgamma_init=None, dbeta_init=None, want_dgamma=True, want_dbeta=True, flags=0):
    rows = int(np.prod(x.shape[:-1]))
    Cw = x.shape[-1]
    d_x, d_dy, d_g, d_res = _up(ctx, x), _up(ctx, dy), _up(ctx, gamma), _up(ctx, dres)
    d_dx = None
    if want_dx:
        d_dx = ctx.upload(dx_init) if dx_init is not None else ctx.upload(np.full(x.shape, 7, dtype=x.dtype))
    d_dx2 = ctx.upload(np.full(x.shape, 9, dtype=x.dtype)) if want_dx2 else None
    d_dg = d_db = None
    if want_dgamma:
        d_dg = ctx.upload(dgamma_init if dgamma_init is not None else np.full((Cw,), 3, np.float32))
    if want_dbeta:
        d_db = ctx.upload(dbeta_init if dbeta_init is not None else np.full((Cw,), 5, np.float32))
    ws_bytes = ctx.lib.agrad_norm_backward_workspace_bytes(rows, Cw, _dt(x))
    ws = ctx.empty((max(ws_bytes, 1),), np.uint8)
    ctx.call("agrad_norm_backward", kind, _dt(x), _p(d_x), _p(d_dy), _p(d_g), _p(d_res), _p(d_dx), _p(d_dx2),
             _p(d_dg), _p(d_db), _p(ws), ws_bytes, rows, Cw, eps, flags)
    ctx.synchronize()
    out = dict(dx=d_dx.download() if d_dx else None, dx2=d_dx2.download() if d_dx2 else None,
               dgamma=d_dg.download() if d_dg else None, dbeta=d_db.download() if d_db else None)
    _free(d_x, d_dy, d_g, d_res, d_dx, d_dx2, d_dg, d_db, ws)
    return out


def unary(ctx, name, x):
    d_x = ctx.upload(x)
    y = ctx.empty(x.shape, x.dtype)
    ctx.call(name, _dt(x), _p(d_x), _p(y), x.size)
    ctx.synchronize()
    out = y.download()
    _free(d_x, y)
    return out


def unary_backward(ctx, name, x, dy, dx_init=None, flags=0):
    d_x, d_dy = ctx.upload(x), ctx.upload(dy)
    d_dx = ctx.upload(dx_init if dx_init is not None else np.full(x.shape, 7, dtype=x.dtype))
    ctx.call(name, _dt(x), _p(d_x), _p(d_dy), _p(d_dx), x.size, flags)
    ctx.synchronize()
    out = d_dx.download()
    _free(d_x, d_dy, d_dx)
    return out


def swiglu_forward(ctx, gu):
    rows, H2 = int(np.prod(gu.shape[:-1])), gu.shape[-1]
    d_gu = ctx.upload(gu)
    h = ctx.empty(gu.shape[:-1] + (H2 // 2,), gu.dtype)
    ctx.call("agrad_swiglu_forward", _dt(gu), _p(d_gu), _p(h), rows, H2 // 2)
    ctx.synchronize()
    out = h.download()
    _free(d_gu, h)
    return out


def swiglu_backward(ctx, gu, dh, inplace=True, dgu_init=None, flags=0):
    rows, H2 = int(np.prod(gu.shape[:-1])), gu.shape[-1]
    d_gu, d_dh = ctx.upload(gu), ctx.upload(dh)
    if inplace:
        d_out = d_gu
    else:
        d_out = ctx.upload(dgu_init if dgu_init is not None else np.full(gu.shape, 7, dtype=gu.dtype))
    ctx.call("agrad_swiglu_backward", _dt(gu), _p(d_gu), _p(d_dh), _p(d_out), rows, H2 // 2, flags)
    ctx.synchronize()
    out = d_out.download()
    _free(d_gu, d_dh)
    if not inplace:
        _free(d_out)
    return out


def rope(ctx, q, k, cos, sin, sign, backward=False):
    B, T, H, D = q.shape
    HKV = k.shape[2] if k is not None else 0
    d_q, d_k, d_c, d_s = ctx.upload(q), _up(ctx, k), ctx.upload(cos), ctx.upload(sin)
    ctx.call("agrad_rope_qk", _dt(q), _p(d_q), _p(d_k), _p(d_c), _p(d_s), B, T, H, HKV, D, sign, int(backward))
    ctx.synchronize()
    out = d_q.download(), (d_k.download() if d_k is not None else None)
    _free(d_q, d_k, d_c, d_s)
    return out


def gather_forward(ctx, ids, W, wpe=None):
    B, T = ids.shape
    V, Cw = W.shape
    d_i, d_w, d_p = ctx.upload(ids.astype(np.int32)), ctx.upload(W), _up(ctx, wpe)
    out = ctx.upload(np.full((B, T, Cw), 7, dtype=W.dtype))
    ctx.call("agrad_gather_forward", _dt(W), _p(d_i), _p(d_w), _p(d_p), _p(out), B * T, T, Cw, V)
    ctx.synchronize()
    res = out.download()
    _free(d_i, d_w, d_p, out)
    return res


def embedding_backward(ctx, ids, dY, V, dW_init=None, flags=0):
    N = ids.size
    Cw = dY.shape[-1]
    d_i, d_dy = ctx.upload(ids.astype(np.int32)), ctx.upload(dY)
    d_dw = ctx.upload(dW_init) if dW_init is not None else ctx.zeros((V, Cw), dY.dtype)
    ws_bytes = ctx.lib.agrad_embedding_backward_workspace_bytes(N, Cw, V, _dt(dY))
    ws = ctx.empty((max(ws_bytes, 1),), np.uint8)
    ctx.call("agrad_embedding_backward", _dt(dY), _p(d_i), _p(d_dy), _p(d_dw), _p(ws), ws_bytes, N, Cw, V, flags)
    ctx.synchronize()
    res = d_dw.download()
    _free(d_i, d_dy, d_dw, ws)
    return res


def pos_embedding_backward(ctx, dY, dwpe_init=None, flags=0):
    B, T, Cw = dY.shape
    d_dy = ctx.upload(dY)
    d_dp = ctx.upload(dwpe_init if dwpe_init is not None else np.full((T, Cw), 7, dtype=dY.dtype))
    ctx.call("agrad_pos_embedding_backward", _dt(dY), _p(d_dy), _p(d_dp), B, T, Cw, flags)
    ctx.synchronize()
    res = d_dp.download()
    _free(d_dy, d_dp)
    return res
