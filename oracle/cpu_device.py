"""The numpy oracle packaged as a "cpu" device for the host runtime.

TEST INFRASTRUCTURE ONLY.  Registering this device lets one graph script run
once on "cpu" (numpy, oracle/cpu_ops.py) and once on "hip" and compare, which is
how the reference's own harnesses work (run_single_op on "cpu" and "mps",
check_tiny_gpt2_kernel.py:473-490).  The allocator hands out numpy arrays and
byte views of a uint8 arena (CPUAllocator, storage.py:49-64); kernels follow the
CPU calling convention: they read `t.storage.data`, accumulate into
`t.grad.storage.data`, and never store (backend.py:74-105, 376-487, 525-538).
bf16 tensors are stored as uint16 bits and widened around every op.
"""
from __future__ import annotations

from contextlib import ExitStack
from math import prod

import numpy as np

from autograd_amd.backend import Backend
from autograd_amd.device import Device
from autograd_amd.op import (AddLayerNormOp, AddOp, AddRMSNormOp, ContiguousOp, CrossEntropyLossOp, EmbeddingSumOp,
                             BiasGELUOp, ExpOp, GatherOp, GELUOp, LayerNormOp, LogOp, MulOp, PermuteOp, ReLUSquaredOp, ReshapeOp,
                             RMSNormOp, RopeOp, RsqrtOp, SoftmaxOp, SwiGLUOp, TransposeOp, ViewOp)
from autograd_amd.storage import Allocator, Storage
from autograd_amd.utils import is_bf16, storage_dtype

from . import cpu_ops as K


class CPUAllocator(Allocator):
    def __init__(self):
        super().__init__(device="cpu")

    def alloc(self, shape, dtype=np.float32):
        arr = np.empty(shape, dtype=storage_dtype(dtype))
        return Storage(ptr=arr, shape=shape, dtype=arr.dtype, device=self.device, nbytes=arr.nbytes)

    def view(self, storage, offset, shape, dtype):
        dt = storage_dtype(dtype)
        nbytes = prod(shape) * dt.itemsize
        if offset + nbytes > storage.nbytes:
            raise RuntimeError(f"View overflow: {offset}+{nbytes}>{storage.nbytes}")
        flat = storage.data.reshape(-1).view(np.uint8)
        data = flat[offset:offset + nbytes].view(dt).reshape(shape)
        return Storage(ptr=data, shape=shape, dtype=dt, device=self.device, nbytes=nbytes)


def _val(t):
    """fp32 value of a tensor (bf16 storage is widened)"""
    d = t.storage.data
    return K.bf16_bits_to_f32(d).reshape(t.shape) if d.dtype == np.uint16 else d


def _put(t, value):
    d = t.storage.data
    if d.dtype == np.uint16:
        d[...] = K.f32_to_bf16_bits(value).reshape(t.shape)
    else:
        d[...] = value


class _Acc:
    """context: fp32 working copy of a gradient that is written back on exit"""

    def __init__(self, t):
        self.t = t

    def __enter__(self):
        d = self.t.storage.data
        self.work = K.bf16_bits_to_f32(d).reshape(self.t.shape).copy() if d.dtype == np.uint16 else d
        return self.work

    def __exit__(self, *exc):
        if self.t.storage.data.dtype == np.uint16:
            _put(self.t, self.work)


def _param_grad(stack, t):
    """fp32 working view of a parameter's gradient (None if it wants none); a bf16-stored
    gradient is widened here and rounded back once when `stack` closes"""
    if t is None or not t.requires_grad or t.grad is None:
        return None
    return stack.enter_context(_Acc(t.grad))


def cpu_add_forward(inputs, outputs, scratch=None):
    _put(outputs[0], K.add_forward(_val(inputs[0]), _val(inputs[1])))


def cpu_add_backward(inputs, outputs, scratch=None):
    out = outputs[0]
    if out.grad is None:
        return
    g = _val(out.grad)
    for t in inputs[:2]:
        if t.requires_grad and t.grad is not None:
            with _Acc(t.grad) as acc:
                K.add_backward_into(g, acc)


def cpu_mul_forward(inputs, outputs, scratch=None):
    _put(outputs[0], K.mul_forward(_val(inputs[0]), _val(inputs[1])))


def cpu_mul_backward(inputs, outputs, scratch=None):
    x, y, out = inputs[0], inputs[1], outputs[0]
    if out.grad is None:
        return
    g, xv, yv = _val(out.grad), _val(x), _val(y)
    if x.requires_grad and x.grad is not None:
        with _Acc(x.grad) as acc:
            K.mul_backward_into(g, xv, yv, dx=acc)
    if y.requires_grad and y.grad is not None:
        with _Acc(y.grad) as acc:
            K.mul_backward_into(g, xv, yv, dy=acc)


def _cpu_unary(fwd, bwd, saves_output):
    def forward(inputs, outputs, scratch=None):
        _put(outputs[0], fwd(_val(inputs[0])))

    def backward(inputs, outputs, scratch=None):
        x, out = inputs[0], outputs[0]
        if out.grad is None or not x.requires_grad:
            return
        with _Acc(x.grad) as acc:
            bwd(_val(out.grad), _val(out if saves_output else x), acc)
    return forward, backward


cpu_exp_forward, cpu_exp_backward = _cpu_unary(K.exp_forward, K.exp_backward_into, True)
cpu_log_forward, cpu_log_backward = _cpu_unary(K.log_forward, K.log_backward_into, False)
cpu_rsqrt_forward, cpu_rsqrt_backward = _cpu_unary(K.rsqrt_forward, K.rsqrt_backward_into, True)


def cpu_softmax_forward(inputs, outputs, scratch=None):
    x, out = inputs[0], outputs[0]
    _put(out, K.softmax_forward(_val(x), axis=out.op.op.dim))       # the op's own axis (backend.py:356)


def cpu_softmax_backward(inputs, outputs, scratch=None):
    x, out = inputs[0], outputs[0]
    if out.grad is None or not x.requires_grad:
        return
    with _Acc(x.grad) as acc:
        K.softmax_backward_into(_val(out), _val(out.grad), acc, axis=out.op.op.dim)


# views share their input's memory: nothing to do going forward (backend.py:263-313)
def cpu_view_forward(inputs, outputs, scratch=None):
    pass


def cpu_dense_grad_backward(inputs, outputs, scratch=None):
    x, out = inputs[0], outputs[0]
    if out.grad is None or not x.requires_grad or x.grad is None:
        return
    with _Acc(x.grad) as acc:
        K.add_backward_into(_val(out.grad).reshape(x.shape), acc)


def cpu_permute_backward(inputs, outputs, scratch=None):
    x, out = inputs[0], outputs[0]
    if out.grad is None or not x.requires_grad or x.grad is None:
        return
    with _Acc(x.grad) as acc:
        K.permute_backward_into(_val(out.grad), [d % x.ndim for d in out.op.op.dims], acc)


def cpu_transpose_backward(inputs, outputs, scratch=None):
    x, out = inputs[0], outputs[0]
    if out.grad is None or not x.requires_grad or x.grad is None:
        return
    with _Acc(x.grad) as acc:
        K.transpose_backward_into(_val(out.grad), out.op.op.dim0, out.op.op.dim1, acc)


def cpu_contiguous_forward(inputs, outputs, scratch=None):
    x, out = inputs[0], outputs[0]
    out.storage.data[...] = K.contiguous_forward(x.storage.data, x.shape, x.strides, x.offset)


def cpu_gather_forward(inputs, outputs, scratch=None):
    outputs[0].storage.data[...] = K.gather_forward(inputs[0].storage.data, inputs[1].storage.data)


def cpu_gather_backward(inputs, outputs, scratch=None):
    indices, weight, out = inputs[0], inputs[1], outputs[0]
    if out.grad is None or not weight.requires_grad:
        return
    with _Acc(weight.grad) as acc:
        K.gather_backward_into(indices.storage.data, _val(out.grad), acc)


def cpu_embedding_sum_forward(inputs, outputs, scratch=None):
    ids, wte, wpe = inputs
    _put(outputs[0], K.embedding_sum_forward(ids.storage.data, _val(wte), _val(wpe)))


def cpu_embedding_sum_backward(inputs, outputs, scratch=None):
    ids, wte, wpe = inputs
    out = outputs[0]
    if out.grad is None:
        return
    g = _val(out.grad)
    if wte.requires_grad:
        with _Acc(wte.grad) as acc:
            K.embedding_sum_backward_into(ids.storage.data, g, acc, None)
    if wpe.requires_grad:
        with _Acc(wpe.grad) as acc:
            K.embedding_sum_backward_into(ids.storage.data, g, None, acc)


def _unary(fwd, bwd):
    def forward(inputs, outputs, scratch=None):
        _put(outputs[0], fwd(_val(inputs[0])))

    def backward(inputs, outputs, scratch=None):
        x, out = inputs[0], outputs[0]
        if out.grad is None or not x.requires_grad:
            return
        with _Acc(x.grad) as acc:
            bwd(_val(x), _val(out.grad), acc)
    return forward, backward


cpu_gelu_forward, cpu_gelu_backward = _unary(K.gelu_forward, K.gelu_backward_into)
cpu_relu2_forward, cpu_relu2_backward = _unary(K.relu2_forward, K.relu2_backward_into)


def cpu_bias_gelu_forward(inputs, outputs, scratch=None):
    _put(outputs[0], K.bias_gelu_forward(_val(inputs[0]), _val(inputs[1])))


def cpu_bias_gelu_backward(inputs, outputs, scratch=None):
    h, b, out = inputs[0], inputs[1], outputs[0]
    if out.grad is None:
        return
    g, hv, bv = _val(out.grad), _val(h), _val(b)
    if h.requires_grad and h.grad is not None:
        with _Acc(h.grad) as acc:
            K.bias_gelu_backward_into(hv, bv, g, dh=acc)
    if b.requires_grad and b.grad is not None:
        with _Acc(b.grad) as acc:
            K.bias_gelu_backward_into(hv, bv, g, db=acc)


def cpu_swiglu_forward(inputs, outputs, scratch=None):
    _put(outputs[0], K.swiglu_forward(_val(inputs[0])))


def cpu_swiglu_backward(inputs, outputs, scratch=None):
    gu, out = inputs[0], outputs[0]
    if out.grad is None or not gu.requires_grad:
        return
    with _Acc(gu.grad) as acc:
        np.add(acc, K.swiglu_backward(_val(gu), _val(out.grad)), out=acc)


def _norm_backward(kind, x_val, gamma, beta, dy, eps, dx_targets, gamma_t, beta_t):
    C = x_val.shape[-1]
    g = _val(gamma) if gamma is not None else None
    dgamma = gamma_t.grad if gamma_t is not None and gamma_t.requires_grad else None
    dbeta = beta_t.grad if beta_t is not None and beta_t.requires_grad else None
    local = np.zeros_like(x_val) if dx_targets else None
    dg = dgamma.storage.data if dgamma is not None else None
    db = dbeta.storage.data if dbeta is not None else None
    if kind == "layer":
        K.layernorm_backward_into(x_val, g if g is not None else np.ones(C, np.float32), dy, eps, local, dg, db)
    else:
        K.rmsnorm_backward_into(x_val, g, dy, eps, local, dg)
    return local


def cpu_layernorm_forward(inputs, outputs, scratch=None):
    x, gamma, beta = inputs
    _put(outputs[0], K.layernorm_forward(_val(x), _val(gamma), _val(beta), outputs[0].op.op.eps))


def cpu_layernorm_backward(inputs, outputs, scratch=None):
    x, gamma, beta = inputs
    out = outputs[0]
    if out.grad is None:
        return
    eps = out.op.op.eps
    if x.requires_grad and x.grad.storage.data.dtype != np.uint16:
        # fp32: accumulate straight into x.grad in the reference's order (backend.py:469-487)
        with ExitStack() as stack:
            dg, db = _param_grad(stack, gamma), _param_grad(stack, beta)
            K.layernorm_backward_into(_val(x), _val(gamma), _val(out.grad), eps, x.grad.storage.data, dg, db)
        return
    local = _norm_backward("layer", _val(x), gamma, beta, _val(out.grad), eps, x.requires_grad, gamma, beta)
    if x.requires_grad:
        with _Acc(x.grad) as acc:
            np.add(acc, local, out=acc)


def cpu_rmsnorm_forward(inputs, outputs, scratch=None):
    x = inputs[0]
    gamma = _val(inputs[1]) if len(inputs) > 1 else None
    _put(outputs[0], K.rmsnorm_forward(_val(x), gamma, outputs[0].op.op.eps))


def cpu_rmsnorm_backward(inputs, outputs, scratch=None):
    x = inputs[0]
    gamma = inputs[1] if len(inputs) > 1 else None
    out = outputs[0]
    if out.grad is None:
        return
    eps = out.op.op.eps
    if x.requires_grad and x.grad.storage.data.dtype != np.uint16:
        with ExitStack() as stack:
            K.rmsnorm_backward_into(_val(x), _val(gamma) if gamma is not None else None, _val(out.grad), eps,
                                    x.grad.storage.data, _param_grad(stack, gamma))
        return
    local = _norm_backward("rms", _val(x), gamma, None, _val(out.grad), eps, x.requires_grad, gamma, None)
    if x.requires_grad:
        with _Acc(x.grad) as acc:
            np.add(acc, local, out=acc)


def cpu_add_norm_forward(inputs, outputs, scratch=None):
    x, res = inputs[0], inputs[1]
    h, y = outputs
    op = h.op.op
    _put(h, K.add_forward(_val(x), _val(res)))
    hv = _val(h)   # what the norm reads is what was stored (bf16: the rounded sum)
    if isinstance(op, AddLayerNormOp):
        _put(y, K.layernorm_forward(hv, _val(inputs[2]), _val(inputs[3]), op.eps))
    else:
        _put(y, K.rmsnorm_forward(hv, _val(inputs[2]) if len(inputs) > 2 else None, op.eps))


def cpu_add_norm_backward(inputs, outputs, scratch=None):
    """norm backward accumulated onto h.grad, then the add's backward."""
    x, res = inputs[0], inputs[1]
    h, y = outputs
    op = h.op.op
    is_ln = isinstance(op, AddLayerNormOp)
    gamma = inputs[2] if len(inputs) > 2 else None
    beta = inputs[3] if is_ln else None
    total = _val(h.grad).astype(np.float32).copy() if h.grad is not None else np.zeros(h.shape, np.float32)
    if y.grad is not None:
        need_dx = any(t.requires_grad for t in (x, res))
        C = h.shape[-1]
        g = _val(gamma) if gamma is not None else None
        with ExitStack() as stack:
            dg, db = _param_grad(stack, gamma), _param_grad(stack, beta)
            if is_ln:
                K.layernorm_backward_into(_val(h), g, _val(y.grad), op.eps, total if need_dx else None, dg, db)
            else:
                K.rmsnorm_backward_into(_val(h), g, _val(y.grad), op.eps, total if need_dx else None, dg)
    elif h.grad is None:
        return
    for t in (x, res):
        if t.requires_grad and t.grad is not None:
            with _Acc(t.grad) as acc:
                np.add(acc, total, out=acc)


def cpu_cross_entropy_forward(inputs, outputs, scratch=None):
    logits, labels = inputs
    x = _val(logits)
    _put(outputs[0], K.cross_entropy_forward(x, labels.storage.data))
    # the second output (row log-sum-exp) is an aid for the device kernels only
    m = x.max(-1, keepdims=True)
    _put(outputs[1], (m + np.log(np.exp(x - m).sum(-1, keepdims=True)))[..., 0])


def cpu_cross_entropy_backward(inputs, outputs, scratch=None):
    logits, labels = inputs
    loss = outputs[0]
    if loss.grad is None or not logits.requires_grad:
        return
    with _Acc(logits.grad) as acc:
        K.cross_entropy_backward_into(_val(logits), labels.storage.data, _val(loss.grad), acc)


def cpu_rope_forward(inputs, outputs, scratch=None):
    q, k, cos, sin = inputs
    q2, k2 = outputs
    bhtd = q2.op.op.layout == "bhtd"        # the CPU kernels take [B,T,H,D] (backend.py:1383): transpose around them
    qv, kv = _val(q), _val(k)
    qv = np.ascontiguousarray(qv.transpose(0, 2, 1, 3)) if bhtd else qv.copy()
    kv = np.ascontiguousarray(kv.transpose(0, 2, 1, 3)) if bhtd else kv.copy()
    K.rope_signed(qv, kv, cos.storage.data, sin.storage.data, q2.op.op.rope_sign, False)
    _put(q2, np.ascontiguousarray(qv.transpose(0, 2, 1, 3)) if bhtd else qv)
    _put(k2, np.ascontiguousarray(kv.transpose(0, 2, 1, 3)) if bhtd else kv)


def cpu_rope_backward(inputs, outputs, scratch=None):
    q, k, cos, sin = inputs
    q2, k2 = outputs
    sign = q2.op.op.rope_sign
    for src, dst in ((q, q2), (k, k2)):
        if not src.requires_grad or dst.grad is None:
            continue
        bhtd = q2.op.op.layout == "bhtd"
        g = _val(dst.grad)
        g = np.ascontiguousarray(g.transpose(0, 2, 1, 3)) if bhtd else g.copy()
        dummy = np.zeros((g.shape[0], g.shape[1], 1, g.shape[3]), np.float32)
        K.rope_signed(g, dummy, cos.storage.data, sin.storage.data, sign, True)
        if bhtd:
            g = np.ascontiguousarray(g.transpose(0, 2, 1, 3))
        if src.grad.storage.data is dst.grad.storage.data or np.shares_memory(src.grad.storage.data, dst.grad.storage.data):
            _put(src.grad, g)
        else:
            with _Acc(src.grad) as acc:
                np.add(acc, g, out=acc)


class CPUBackend(Backend):
    def __init__(self):
        self.grad_scale = 1.0
        self.accumulate_parameter_grads = False
        self.forward_kernels = {
            AddOp: cpu_add_forward, GatherOp: cpu_gather_forward, EmbeddingSumOp: cpu_embedding_sum_forward,
            GELUOp: cpu_gelu_forward, BiasGELUOp: cpu_bias_gelu_forward, ReLUSquaredOp: cpu_relu2_forward, SwiGLUOp: cpu_swiglu_forward,
            LayerNormOp: cpu_layernorm_forward, RMSNormOp: cpu_rmsnorm_forward,
            AddLayerNormOp: cpu_add_norm_forward, AddRMSNormOp: cpu_add_norm_forward, RopeOp: cpu_rope_forward,
            CrossEntropyLossOp: cpu_cross_entropy_forward,
            MulOp: cpu_mul_forward, ExpOp: cpu_exp_forward, LogOp: cpu_log_forward, RsqrtOp: cpu_rsqrt_forward,
            SoftmaxOp: cpu_softmax_forward,
            ViewOp: cpu_view_forward, ReshapeOp: cpu_view_forward, PermuteOp: cpu_view_forward,
            TransposeOp: cpu_view_forward, ContiguousOp: cpu_contiguous_forward,
        }
        self.backward_kernels = {
            AddOp: cpu_add_backward, GatherOp: cpu_gather_backward, EmbeddingSumOp: cpu_embedding_sum_backward,
            GELUOp: cpu_gelu_backward, BiasGELUOp: cpu_bias_gelu_backward, ReLUSquaredOp: cpu_relu2_backward, SwiGLUOp: cpu_swiglu_backward,
            LayerNormOp: cpu_layernorm_backward, RMSNormOp: cpu_rmsnorm_backward,
            AddLayerNormOp: cpu_add_norm_backward, AddRMSNormOp: cpu_add_norm_backward, RopeOp: cpu_rope_backward,
            CrossEntropyLossOp: cpu_cross_entropy_backward,
            MulOp: cpu_mul_backward, ExpOp: cpu_exp_backward, LogOp: cpu_log_backward, RsqrtOp: cpu_rsqrt_backward,
            SoftmaxOp: cpu_softmax_backward,
            ViewOp: cpu_dense_grad_backward, ReshapeOp: cpu_dense_grad_backward, PermuteOp: cpu_permute_backward,
            TransposeOp: cpu_transpose_backward, ContiguousOp: cpu_dense_grad_backward,
        }

    def get_forward_kernel(self, op):
        return self.forward_kernels.get(type(op))

    def get_backward_kernel(self, op):
        return self.backward_kernels.get(type(op))

    def fill_storage(self, storage, value):
        if storage.data.dtype == np.uint16:
            storage.data[...] = K.f32_to_bf16_bits(np.float32(value))
        else:
            storage.data[...] = value

    fill_storage2 = fill_storage

    def copy_from_host(self, tensor, host_np):
        d = tensor.storage.data
        host = np.asarray(host_np)
        if d.dtype == np.uint16 and host.dtype != np.uint16:
            d[...] = K.f32_to_bf16_bits(np.asarray(host, np.float32)).reshape(tensor.shape)
        else:
            d[...] = host.reshape(tensor.shape)

    def copy_to_host(self, tensor):
        d = tensor.storage.data
        if d.dtype == np.uint16:
            return K.bf16_bits_to_f32(d).reshape(tensor.shape).copy()
        return np.array(d, copy=True)

    def storage_to_host(self, storage):
        return np.array(storage.data, copy=True)

    # CPUBackend.adamw_step (backend.py:2602-2605) with the keyword arguments of
    # the Metal backend's (backend.py:5122-5124) so one optimizer drives both
    def adamw_step(self, p_storage, g_storage, m_storage, v_storage, tmp_storage,
                   lr, lr_t, b1, b2, eps, weight_decay, numel=None, decay_numel=None, grad_scale=1.0,
                   lr_bc1=None, inv_sqrt_bc2=1.0):
        g = g_storage.data
        if g.dtype == np.uint16:
            g = K.bf16_bits_to_f32(g).reshape(g.shape)
        p, m, v = p_storage.data, m_storage.data, v_storage.data
        n = p.size if numel is None else int(numel)
        dn = (n if weight_decay != 0.0 else 0) if decay_numel is None else int(decay_numel)
        if lr_bc1 is None and inv_sqrt_bc2 == 1.0 and grad_scale == 1.0 and dn in (0, n):
            K.adamw_step(p, g, m, v, lr, lr_t, b1, b2, eps, weight_decay if dn else 0.0)
        else:
            K.adamw_step_split(p, g, m, v, lr * weight_decay if weight_decay > 0.0 else 0.0, b1, b2, eps,
                               lr_t if lr_bc1 is None else lr_bc1, inv_sqrt_bc2, grad_scale, dn)

    def storage_from_host(self, storage, host_np):
        storage.data.reshape(-1)[:] = np.asarray(host_np, dtype=storage.data.dtype).reshape(-1)

    # the Metal backend's signature (backend.py:5142-5143) over the numpy restatement of its kernel
    def adamw8bit_step(self, p, g, qm, qv, absmax_m, absmax_v, qmap_m, qmap_v,
                       lr, lr_bc1, inv_sqrt_bc2, b1, b2, eps, weight_decay, numel, decay_numel, first_step, grad_scale=1.0):
        gv = g.data
        if gv.dtype == np.uint16:
            gv = K.bf16_bits_to_f32(gv)
        n = int(numel)
        K.adamw8bit_step(p.data.reshape(-1)[:n], gv.reshape(-1)[:n], qm.data.reshape(-1)[:n], qv.data.reshape(-1)[:n],
                         absmax_m.data.reshape(-1), absmax_v.data.reshape(-1), qmap_m.data, qmap_v.data,
                         np.float32(1.0 - float(lr) * float(weight_decay)), lr_bc1, b1, b2, eps, int(decay_numel),
                         bool(first_step), inv_sqrt_bc2, clip_coef=grad_scale)

    def grad_norm_sq(self, g_storage, partial, numel):
        g = g_storage.data
        if g.dtype == np.uint16:
            g = K.bf16_bits_to_f32(g)
        partial.data.reshape(-1)[:] = K.grad_norm_partials(g.reshape(-1)[:int(numel)]).astype(np.float32)


def register():
    """make "cpu" available to Runtime(device="cpu")"""
    Device.register("cpu", CPUAllocator, CPUBackend)
