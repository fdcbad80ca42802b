"""Backend of the "hip" device: binds each layer op to a gfx950 kernel.

Counterpart of the reference's Backend / MetalBackend (backend.py:22-69,
2611-2955, 4938-5113) for the fused layer-op path.  The contract is the
reference's:

  * a bound kernel is `fn(inputs, outputs, scratch=None)`, looked up by the
    exact type of the op in `forward_kernels` / `backward_kernels`
    (backend.py:4938-4950) and stored on `OpNode.forward / .backward`;
  * op attributes are read through `out.op.op.<attr>` (backend.py:2916);
  * backward kernels return early when `out.grad` is None, read `out.grad` and
    write `x.grad.storage`;
  * every launch is `ctx.dispatch_with_args_3d(name, buffer_ids, offsets,
    uint32 args, gx, gy, gz, tg)` with floats passed as bit patterns
    (backend.py:2911-2920).

Differences, all on the CPU side of the reference's own CPU/Metal split:
backward kernels accumulate into existing gradients like the CPU kernels do
(backend.py:414, 477-487) unless the runtime marked this node as the first
writer of a gradient in the pass, in which case they store; LayerNorm backward
honours the op's eps; launch geometry is chosen by the native library, so the
grid arguments are passed as zeros.

There is no CPU fallback: every kernel here ends in a HIP launch.
"""
from __future__ import annotations

from math import prod

import numpy as np

from .op import (AddLayerNormOp, AddOp, AddRMSNormOp, BiasGELUOp, ContiguousOp, CrossEntropyLossOp, EmbeddingSumOp, ExpOp,
                 GatherOp, GELUOp, LayerNormOp, LogOp, MulOp, PermuteOp, ReLUSquaredOp, ReshapeOp, RMSNormOp, RopeOp,
                 RsqrtOp, SoftmaxOp, SwiGLUOp, TransposeOp, ViewOp)
from .scratch import equal_slots, single_slot
from .utils import (bf16_bits, bf16_bits_to_f32_array, contiguous_strides, f32_array_to_bf16_bits, f32_bits,
                    is_bf16, mul_bcast_kind, storage_dtype, xavier_uniform)

F32, BF16 = 0, 1
ACC_INPUT_GRAD, ACC_PARAM_GRAD, ACC_INPUT_GRAD2, ACC_PARAM_GRAD2, PARAM_GRAD_BF16, DEFER_PARAM_GRAD = 1, 2, 4, 8, 16, 32
UNARY_OPS = {ExpOp: 0, LogOp: 1, RsqrtOp: 2}
MUL_KINDS = {"same": 0, "row": 1, "col": 2, "scalar": 3}


class Backend:
    mixed_precision = False

    def get_forward_kernel(self, op):
        raise NotImplementedError()

    def get_backward_kernel(self, op):
        raise NotImplementedError()

    def fill_storage(self, storage, value):
        raise NotImplementedError()

    def fill_storage2(self, storage, value):
        raise NotImplementedError()

    def fill_scalar(self, tensor, value):
        self.fill_storage(tensor.storage, float(value))

    def fill(self, tensor, value):
        self.fill_scalar(tensor, float(value))

    def init(self, tensor):
        """materialise tensor.init_val: number, ndarray, "xavier" or "zeros" (backend.py:43-59)"""
        v = tensor.init_val
        if v is None:
            return
        try:
            if isinstance(v, (int, float)):
                self.fill_scalar(tensor, float(v))
            elif isinstance(v, np.ndarray):
                self.copy_from_host(tensor, v)
            elif v == "xavier":
                self.copy_from_host(tensor, xavier_uniform(tensor.shape, np.float32))
            elif v == "zeros":
                self.fill_scalar(tensor, 0.0)
            else:
                raise ValueError(f"unknown init_val: {v!r}")
        finally:
            tensor.init_val = None

    def plan_scratch(self, node):
        """(forward layout, backward layout) of scratch this backend's kernels need"""
        return None, None

    def begin_pass(self):
        pass

    def end_pass(self):
        pass

    def synchronize(self):
        pass


def _dt(t):
    """dtype code of a tensor or of a storage (whose bf16 bytes are typed uint16)"""
    if is_bf16(t.dtype) or np.dtype(t.dtype) == np.dtype(np.uint16):
        return BF16
    if np.dtype(t.dtype) == np.dtype(np.float32):
        return F32
    raise RuntimeError(f"hip backend: unsupported dtype {t.dtype}")


def _ids(*tensors_or_storages):
    ids, offs = [], []
    for s in tensors_or_storages:
        if s is None:
            ids.append(0)
            offs.append(0)
            continue
        st = s.storage if hasattr(s, "storage") else s
        ids.append(st.ptr.buffer_id)
        offs.append(st.ptr.offset)
    return ids, offs


def _lo_hi(n):
    return [n & 0xFFFFFFFF, (n >> 32) & 0xFFFFFFFF]


def _mask(*present):
    m = 0
    for i, p in enumerate(present):
        if p is not None:
            m |= 1 << i
    return m


class HipBackend(Backend):
    supports_grad_store = True   # kernels take a store / accumulate flag per gradient
    supports_deferred_param_grads = True    # column sums of a pass can be folded in one launch at its end
    single_pass_execute = True   # Runtime.execute runs zero_grad + forward + backward as ONE pass (one wait)
    supports_row_reset = True    # an embedding table's gradient is cleared by rows (clear_table_grad)

    def __init__(self, ctx=None):
        if ctx is None:
            from .device import hip_context
            ctx = hip_context()
        self.ctx = ctx
        self.grad_scale = 1.0
        self.accumulate_parameter_grads = False
        self.use_fp16_gemm = False
        self._capturing = False
        self.forward_kernels = {
            AddOp: self.hip_add_forward,
            GatherOp: self.hip_gather_forward,
            EmbeddingSumOp: self.hip_embedding_sum_forward,
            GELUOp: self.hip_gelu_forward,
            BiasGELUOp: self.hip_bias_gelu_forward,
            ReLUSquaredOp: self.hip_relu2_forward,
            SwiGLUOp: self.hip_swiglu_forward,
            LayerNormOp: self.hip_layernorm_forward,
            RMSNormOp: self.hip_rmsnorm_forward,
            AddLayerNormOp: self.hip_add_norm_forward,
            AddRMSNormOp: self.hip_add_norm_forward,
            RopeOp: self.hip_rope_forward,
            CrossEntropyLossOp: self.hip_cross_entropy_forward,
            MulOp: self.hip_mul_forward,
            ExpOp: self.hip_unary_forward,
            LogOp: self.hip_unary_forward,
            RsqrtOp: self.hip_unary_forward,
            SoftmaxOp: self.hip_softmax_forward,
            ViewOp: self.hip_view_forward,
            ReshapeOp: self.hip_view_forward,
            PermuteOp: self.hip_view_forward,
            TransposeOp: self.hip_view_forward,
            ContiguousOp: self.hip_contiguous_forward,
        }
        self.backward_kernels = {
            AddOp: self.hip_add_backward,
            GatherOp: self.hip_gather_backward,
            EmbeddingSumOp: self.hip_embedding_sum_backward,
            GELUOp: self.hip_gelu_backward,
            BiasGELUOp: self.hip_bias_gelu_backward,
            ReLUSquaredOp: self.hip_relu2_backward,
            SwiGLUOp: self.hip_swiglu_backward,
            LayerNormOp: self.hip_layernorm_backward,
            RMSNormOp: self.hip_rmsnorm_backward,
            AddLayerNormOp: self.hip_add_norm_backward,
            AddRMSNormOp: self.hip_add_norm_backward,
            RopeOp: self.hip_rope_backward,
            CrossEntropyLossOp: self.hip_cross_entropy_backward,
            MulOp: self.hip_mul_backward,
            ExpOp: self.hip_unary_backward,
            LogOp: self.hip_unary_backward,
            RsqrtOp: self.hip_unary_backward,
            SoftmaxOp: self.hip_softmax_backward,
            ViewOp: self.hip_dense_grad_backward,
            ReshapeOp: self.hip_dense_grad_backward,
            PermuteOp: self.hip_permute_backward,
            TransposeOp: self.hip_permute_backward,
            ContiguousOp: self.hip_dense_grad_backward,
        }

    # -- lookup (backend.py:4938-4950) -------------------------------------------
    def get_forward_kernel(self, op):
        return self.forward_kernels.get(type(op))

    def get_backward_kernel(self, op):
        return self.backward_kernels.get(type(op))

    def bind_add_forward(self, node):
        return self.hip_add_forward

    def bind_add_backward(self, node):
        return self.hip_add_backward

    def _launch(self, name, tensors, args):
        ids, offs = _ids(*tensors)
        self.ctx.dispatch_with_args_3d(name, ids, offs, [int(a) & 0xFFFFFFFF for a in args], 0, 0, 0, 0)

    # -- gradient write mode -------------------------------------------------------
    def _input_flag(self, node, t):
        return 0 if id(t.grad) in node.overwrite_grads else ACC_INPUT_GRAD

    def _param_flag(self, node, *params):
        for p in params:                            # about to be written: no longer known to be all zero
            if p is not None and p.grad is not None:
                p.grad.dirty_rows = None
        if self.accumulate_parameter_grads:
            return ACC_PARAM_GRAD
        live = [p for p in params if p is not None and p.requires_grad and p.grad is not None]
        if live and all(id(p.grad) in node.overwrite_grads for p in live):
            return 0
        return ACC_PARAM_GRAD

    def _grad_flag(self, node, t):
        """flag for a gradient that may belong to a parameter or an activation"""
        if t.op is None:
            return ACC_INPUT_GRAD if self._param_flag(node, t) else 0
        return self._input_flag(node, t)

    # -- column sums folded at the end of the pass ---------------------------------------
    def can_defer_param_grads(self, node):
        """True if this node's backward kernel ends in a column-sum fold whose results
        only parameters receive (nobody reads a parameter gradient before the pass ends)"""
        op = node.op
        if isinstance(op, (LayerNormOp, RMSNormOp, AddLayerNormOp, AddRMSNormOp)):
            first = 2 if isinstance(op, (AddLayerNormOp, AddRMSNormOp)) else 1
            params = [p for p in node.inputs[first:] if p.requires_grad]
            return bool(params) and all(p.op is None for p in params)
        if isinstance(op, BiasGELUOp):
            b = node.inputs[1]
            return b.requires_grad and b.op is None
        if isinstance(op, AddOp):
            out = node.outputs[0]
            small = [t for t in node.inputs[:2] if t.requires_grad and t.shape != out.shape]
            return bool(small) and all(t.op is None for t in small)
        return False

    @staticmethod
    def _defer_flag(node):
        return DEFER_PARAM_GRAD if getattr(node, "defer_param_grads", False) else 0

    def finalize_param_grads(self):
        """fold every column sum the backward kernels of this pass left pending (one launch)"""
        self.ctx.finalize_param_grads()

    # -- scratch -----------------------------------------------------------------
    def _check_gradient_storage(self, node):
        """A leaf may keep its gradient in another type than its values (fp32 values, bf16
        gradient: the reference's bf16 gradient store).  Only the kernels that own a
        parameter gradient can write one: the embedding tables, the norm parameters and the
        broadcast operand of an Add (a bias, a position table)."""
        op = node.op
        for i, t in enumerate(node.inputs):
            if t.op is not None or not t.requires_grad or t.grad is None or t.grad.dtype == t.dtype:
                continue
            if _dt(t.grad) == _dt(t):
                continue
            table = isinstance(op, (GatherOp, EmbeddingSumOp)) and i >= 1
            norm_param = (isinstance(op, (LayerNormOp, RMSNormOp)) and i >= 1) or \
                         (isinstance(op, (AddLayerNormOp, AddRMSNormOp)) and i >= 2)
            bias = (isinstance(op, AddOp) and t.shape != node.outputs[0].shape
                    and self._trailing(t.shape, node.outputs[0].shape)) or (isinstance(op, BiasGELUOp) and i == 1)
            if not (table or norm_param or bias) or _dt(t) != F32 or _dt(t.grad) != BF16:
                raise RuntimeError(f"{op.op_name}: input {i} ({t.name or 'unnamed'}) stores {t.dtype} values and a "
                                   f"{t.grad.dtype} gradient; only embedding tables, norm parameters and biases "
                                   "(fp32 values, bf16 gradient) can keep their gradient in another type")

    def plan_scratch(self, node):
        op = node.op
        self._check_gradient_storage(node)
        if isinstance(op, (LayerNormOp, RMSNormOp, AddLayerNormOp, AddRMSNormOp)):
            first_param = 2 if isinstance(op, (AddLayerNormOp, AddRMSNormOp)) else 1
            if any(p.requires_grad for p in node.inputs[first_param:]):
                x = node.inputs[0]
                rows, C = prod(x.shape[:-1]), x.shape[-1]
                return None, single_slot("workspace", self.ctx.norm_backward_workspace_bytes(rows, C, _dt(x)))
        if isinstance(op, AddOp):
            out = node.outputs[0]
            need = 0
            for t in node.inputs[:2]:
                if t.requires_grad and t.shape != out.shape and t.numel:
                    need = max(need, self.ctx.broadcast_grad_workspace_bytes(out.numel // t.numel, t.numel))
            if need:
                return None, single_slot("workspace", need)
        if isinstance(op, SoftmaxOp):
            x = node.inputs[0]
            if x.ndim and op.axis(x) != x.ndim - 1 and x.numel:
                dt = storage_dtype(x.dtype)
                return (equal_slots(("moved_x", "moved_y"), (x.numel,), dt),
                        equal_slots(("moved_y", "moved_dy", "moved_dx"), (x.numel,), dt) if x.requires_grad else None)
        if isinstance(op, BiasGELUOp):
            h, b = node.inputs
            if b.requires_grad:
                need = self.ctx.gelu_bias_backward_workspace_bytes(prod(h.shape[:-1]), h.shape[-1])
                if need:
                    return None, single_slot("workspace", need)
        if isinstance(op, MulOp):
            x, y = node.inputs
            if y.requires_grad:
                kind, lead, inner = self._mul_geometry(x, y)
                need = self.ctx.mul_backward_workspace_bytes(kind, lead, inner)
                if need:
                    return None, single_slot("workspace", need)
        if isinstance(op, (GatherOp, EmbeddingSumOp)):
            ids, w = node.inputs[0], node.inputs[1]
            if w.requires_grad:
                n = prod(ids.shape)
                if len(node.outputs) > 1:
                    return (single_slot("sort_workspace", self.ctx.embedding_sort_workspace_bytes(n, w.shape[0])),
                            single_slot("workspace", max(256, self.ctx.embedding_backward_sorted_workspace_bytes(n, w.shape[1]))))
                nbytes = self.ctx.embedding_backward_workspace_bytes(n, w.shape[1], w.shape[0], _dt(w))
                return None, single_slot("workspace", nbytes)
        return None, None

    # -- Add (cpu_add_forward / cpu_add_backward, backend.py:74-105) ----------------
    @staticmethod
    def _trailing(small, big):
        """True if `small` (after dropping leading 1s) is the trailing shape of `big`"""
        sh = tuple(small)
        while sh and sh[0] == 1:
            sh = sh[1:]
        return len(sh) <= len(big) and tuple(big[len(big) - len(sh):]) == sh

    def hip_add_forward(self, inputs, outputs, scratch=None):
        x, y, out = inputs[0], inputs[1], outputs[0]
        if x.shape == y.shape:
            self._launch("add_residual_forward", [x, y, out], [_dt(out)] + _lo_hi(out.numel))
            return
        # one operand has the output's shape, the other its trailing shape (a bias,
        # a position table): add_pos_forward / bias add of the reference's Metal backend
        big, small = (x, y) if x.shape == out.shape else (y, x)
        if big.shape != out.shape or not self._trailing(small.shape, out.shape) or _dt(big) != _dt(small):
            raise RuntimeError(f"Unsupported Add shape: x.shape={x.shape}, y.shape={y.shape}")
        inner = small.numel
        self._launch("add_broadcast_forward", [big, small, out],
                     [_dt(out)] + _lo_hi(out.numel // max(inner, 1)) + _lo_hi(inner))

    def hip_add_backward(self, inputs, outputs, scratch=None):
        out = outputs[0]
        if out.grad is None:
            return
        node = out.op
        for t in inputs[:2]:
            if not t.requires_grad or t.grad is None:
                continue
            if t.shape == out.shape:
                if _dt(t.grad) != _dt(out.grad):
                    raise RuntimeError(f"Add backward: gradient of {t.dtype} input stored as {t.grad.dtype}")
                self._launch("add_residual_backward", [out.grad, t.grad],
                             [_dt(out), self._grad_flag(node, t)] + _lo_hi(out.numel))
            elif self._trailing(t.shape, out.shape) and (_dt(t.grad) == _dt(out.grad)
                                                        or (_dt(out.grad) == F32 and _dt(t.grad) == BF16)):
                inner = t.numel
                lead = out.numel // max(inner, 1)
                flag = (ACC_PARAM_GRAD if self._grad_flag(node, t) else 0) | self._defer_flag(node)
                if _dt(t.grad) != _dt(out.grad):
                    flag |= PARAM_GRAD_BF16       # a bf16 bias gradient under fp32 activations
                ws = scratch["workspace"] if scratch and "workspace" in scratch else None
                self._launch("add_broadcast_backward", [out.grad, t.grad, ws],
                             [_dt(out)] + _lo_hi(lead) + _lo_hi(inner) + [flag]
                             + _lo_hi(ws.nbytes if ws is not None else 0) + [_mask(out.grad, t.grad, ws)])
            else:
                raise RuntimeError(f"Unsupported Add backward shape: {t.shape} from {out.shape}")

    # -- Mul, Exp, Log, Rsqrt, Softmax (backend.py:107-146, 320-374) ------------------
    @staticmethod
    def _mul_geometry(x, y):
        """(native kind, lead, inner) of x * y: x is seen as [lead, inner]"""
        kind = mul_bcast_kind(x.shape, y.shape)
        if kind in ("row", "col"):
            inner = x.shape[-1]
        elif kind == "scalar":
            inner = x.shape[-1] if x.ndim else 1      # rows of the full sum's first stage
        else:
            inner = x.numel
        inner = max(inner, 1)
        return MUL_KINDS[kind], x.numel // inner, inner

    def hip_mul_forward(self, inputs, outputs, scratch=None):
        x, y, out = inputs[0], inputs[1], outputs[0]
        kind, lead, inner = self._mul_geometry(x, y)
        self._launch("mul_forward_kernel", [x, y, out], [_dt(out), kind] + _lo_hi(lead) + _lo_hi(inner))

    def hip_mul_backward(self, inputs, outputs, scratch=None):
        x, y, out = inputs[0], inputs[1], outputs[0]
        if out.grad is None:
            return
        node = out.op
        kind, lead, inner = self._mul_geometry(x, y)
        dx = x.grad if x.requires_grad and x.grad is not None else None
        dy = y.grad if y.requires_grad and y.grad is not None else None
        if dx is None and dy is None:
            return
        if x is y:
            # x * x: both products land in the one gradient, the second call adds
            self._launch("mul_backward_kernel", [out.grad, x, y, dx, None, None],
                         [_dt(out), kind] + _lo_hi(lead) + _lo_hi(inner) + [self._grad_flag(node, x)] + _lo_hi(0)
                         + [_mask(out.grad, x, y, dx, None, None)])
            self._launch("mul_backward_kernel", [out.grad, x, y, None, dx, None],
                         [_dt(out), kind] + _lo_hi(lead) + _lo_hi(inner) + [ACC_INPUT_GRAD2] + _lo_hi(0)
                         + [_mask(out.grad, x, y, None, dx, None)])
            return
        flags = (ACC_INPUT_GRAD if dx is not None and self._grad_flag(node, x) else 0) \
            | (ACC_INPUT_GRAD2 if dy is not None and self._grad_flag(node, y) else 0)
        ws = scratch["workspace"] if scratch and "workspace" in scratch else None
        self._launch("mul_backward_kernel", [out.grad, x, y, dx, dy, ws],
                     [_dt(out), kind] + _lo_hi(lead) + _lo_hi(inner) + [flags]
                     + _lo_hi(ws.nbytes if ws is not None else 0) + [_mask(out.grad, x, y, dx, dy, ws)])

    def hip_unary_forward(self, inputs, outputs, scratch=None):
        x, out = inputs[0], outputs[0]
        self._launch("unary_forward", [x, out], [_dt(x), UNARY_OPS[type(out.op.op)]] + _lo_hi(x.numel))

    def hip_unary_backward(self, inputs, outputs, scratch=None):
        x, out = inputs[0], outputs[0]
        if out.grad is None or not x.requires_grad:
            return
        op = out.op.op
        saved = out if op.saves_output else x
        self._launch("unary_backward", [out.grad, saved, x.grad],
                     [_dt(x), UNARY_OPS[type(op)], self._grad_flag(out.op, x)] + _lo_hi(x.numel))

    # Softmax over an inner axis: the axis is moved to the end through a strided copy
    # into scratch, the row kernels run there, and a second strided copy brings the
    # result back (two extra passes; the last axis -- what attention uses -- takes none).
    @staticmethod
    def _axis_last(x, axis):
        """(dims, shape, strides) of x read with `axis` moved to the end"""
        dims = [d for d in range(x.ndim) if d != axis] + [axis]
        dense = contiguous_strides(x.shape)
        return dims, [x.shape[d] for d in dims], [dense[d] for d in dims]

    @staticmethod
    def _axis_back(x, dims, moved_shape):
        """strides with which the moved (dense) tensor is read in x's own index order"""
        dense = contiguous_strides(moved_shape)
        strides = [0] * x.ndim
        for i, d in enumerate(dims):
            strides[d] = dense[i]
        return strides

    def hip_softmax_forward(self, inputs, outputs, scratch=None):
        x, out = inputs[0], outputs[0]
        axis = out.op.op.axis(x)
        if axis == x.ndim - 1:
            V = x.shape[-1]
            self._launch("softmax_forward", [x, out], [_dt(x)] + _lo_hi(x.numel // max(V, 1)) + [V])
            return
        if scratch is None:
            raise RuntimeError("softmax over an inner axis needs its arena scratch (plan_scratch)")
        if x.numel == 0:
            return
        dims, shape, strides = self._axis_last(x, axis)
        moved, result = scratch["moved_x"], scratch["moved_y"]
        V = x.shape[axis]
        self._gather_strided("contiguous_forward_kernel", x, 0, moved, shape, strides, 0)
        self._launch("softmax_forward", [moved, result], [_dt(x)] + _lo_hi(x.numel // V) + [V])
        self._gather_strided("contiguous_forward_kernel", result, 0, out, x.shape, self._axis_back(x, dims, shape), 0)

    def hip_softmax_backward(self, inputs, outputs, scratch=None):
        x, out = inputs[0], outputs[0]
        if out.grad is None or not x.requires_grad:
            return
        axis = out.op.op.axis(x)
        if axis == x.ndim - 1:
            V = x.shape[-1]
            self._launch("softmax_backward", [out, out.grad, x.grad],
                         [_dt(x)] + _lo_hi(x.numel // max(V, 1)) + [V, self._grad_flag(out.op, x)])
            return
        if scratch is None:
            raise RuntimeError("softmax over an inner axis needs its arena scratch (plan_scratch)")
        if x.numel == 0:
            return
        dims, shape, strides = self._axis_last(x, axis)
        y, dy, dx = scratch["moved_y"], scratch["moved_dy"], scratch["moved_dx"]
        V = x.shape[axis]
        self._gather_strided("contiguous_forward_kernel", out, 0, y, shape, strides, 0)
        self._gather_strided("contiguous_forward_kernel", out.grad, 0, dy, shape, strides, 0)
        self._launch("softmax_backward", [y, dy, dx], [_dt(x)] + _lo_hi(x.numel // V) + [V, 0])
        self._gather_strided("strided_add_backward_kernel", dx, 0, x.grad, x.shape, self._axis_back(x, dims, shape),
                             self._grad_flag(out.op, x))

    # -- views and layout changes (backend.py:263-318, 2754-2866) --------------------
    # View / Reshape / Permute / Transpose outputs share their input's memory, so
    # their forward launches nothing; the gradients are dense tensors of their own.
    def hip_view_forward(self, inputs, outputs, scratch=None):
        pass

    def hip_dense_grad_backward(self, inputs, outputs, scratch=None):
        """x.grad (+)= out.grad, element for element (View, Reshape, Contiguous)"""
        x, out = inputs[0], outputs[0]
        if out.grad is None or not x.requires_grad or x.grad is None:
            return
        self._launch("add_residual_backward", [out.grad, x.grad],
                     [_dt(out), self._grad_flag(out.op, x)] + _lo_hi(out.numel))

    def _gather_strided(self, name, src, src_offset_elems, dst, shape, strides, flags):
        st = src.storage if hasattr(src, "storage") else src
        dstst = dst.storage if hasattr(dst, "storage") else dst
        es = np.dtype(st.dtype).itemsize
        if es not in (2, 4) or np.dtype(dstst.dtype).itemsize != es:
            raise RuntimeError(f"strided copy: unsupported element types {st.dtype} -> {dstst.dtype}")
        if any(s < 0 for s in strides):
            raise RuntimeError("strided copy: negative strides")
        self.ctx.dispatch_contiguous(name, st.ptr.buffer_id, st.ptr.offset + int(src_offset_elems) * es,
                                     dstst.ptr.buffer_id, dstst.ptr.offset, [int(d) for d in shape],
                                     [int(s) for s in strides], prod(shape), 1 if es == 2 else 0, flags)

    def hip_permute_backward(self, inputs, outputs, scratch=None):
        """x.grad[c] (+)= out.grad[c permuted]: a strided read of the dense out.grad"""
        x, out = inputs[0], outputs[0]
        if out.grad is None or not x.requires_grad or x.grad is None:
            return
        op = out.op.op
        n = x.ndim
        dims = tuple(d % n for d in op.dims) if isinstance(op, PermuteOp) else None
        if dims is None:
            dims = list(range(n))
            dims[op.dim0 % n], dims[op.dim1 % n] = dims[op.dim1 % n], dims[op.dim0 % n]
        dense = contiguous_strides(out.shape)
        strides = [0] * n
        for i, d in enumerate(dims):
            strides[d] = dense[i]         # x's dimension d is out's dimension i
        self._gather_strided("strided_add_backward_kernel", out.grad, 0, x.grad, x.shape, strides,
                             self._grad_flag(out.op, x))

    def hip_contiguous_forward(self, inputs, outputs, scratch=None):
        x, out = inputs[0], outputs[0]
        self._gather_strided("contiguous_forward_kernel", x, x.offset, out, x.shape, x.strides, 0)

    # -- embedding (backend.py:525-538, 2777-2815) ----------------------------------
    # When the table needs a gradient the op carries an `order` output: the forward
    # kernel then also orders the ids (one launch, beside the gather) and the
    # backward kernel starts at the segmented sum.
    def zero_grad_and_order(self, node, table):
        """table.grad = 0 and the order of the node's ids for its backward kernel, in one launch
        (the ordering workgroups ride at the front of the fill's grid); the node's forward
        kernel is then the plain gather.  False when this node cannot take it."""
        indices = node.inputs[0]
        scratch = getattr(node.forward, "keywords", {}).get("scratch")
        if len(node.outputs) < 2 or indices.op is not None or table.grad is None or scratch is None \
                or "sort_workspace" not in scratch:
            return False
        ws, g = scratch["sort_workspace"], table.grad.storage
        self._launch("embedding_order", [indices, node.outputs[1], ws, g],
                     [prod(indices.shape), table.shape[0]] + _lo_hi(ws.nbytes) + _lo_hi(g.nbytes) + [0b1111])
        table.grad.dirty_rows = []
        node.order_ready = True
        return True

    def _embedding_forward(self, indices, table, wpe, outputs, scratch):
        out = outputs[0]
        V, C = table.shape
        B, T = indices.shape
        if len(outputs) > 1 and not out.op.order_ready:
            if scratch is None:
                raise RuntimeError("embedding forward needs its arena workspace (plan_scratch)")
            ws = scratch["sort_workspace"]
            kept = out.op.kept_ids
            if kept is not None and table.grad is not None and table.grad.dirty_rows \
                    and any(k is kept for k in table.grad.dirty_rows):
                table.grad.dirty_rows = None        # the list of an earlier pass is about to be overwritten
            self._launch("gather_forward_sorted", [indices, table, wpe, out, outputs[1], ws, kept],
                         [_dt(table), B * T, T, C, V] + _lo_hi(ws.nbytes)
                         + [_mask(indices, table, wpe, out, outputs[1], ws, kept)])
            out.op.kept_fresh = kept is not None
        elif wpe is None:
            self._launch("gather_forward_kernel", [indices, table, out], [_dt(table), B * T, C, V])
        else:
            self._launch("embedding_sum_forward", [indices, table, wpe, out], [_dt(table), B * T, T, C, V])

    def _embedding_grad(self, node, indices, weight, outputs, scratch, wpe=None):
        """Token-table gradient; returns True when the position table's gradient (wpe
        given) went into the same launch."""
        if scratch is None:
            raise RuntimeError("embedding backward needs its arena workspace (plan_scratch)")
        out = outputs[0]
        ws = scratch["workspace"]
        V, C = weight.shape
        # one storage type throughout, or bf16 table gradients under fp32 activations
        # (the reference's bf16 gradient store, backend.py:2808-2812)
        grads = [g for g in (weight.grad, wpe.grad if wpe is not None else None) if g is not None]
        narrow = _dt(out.grad) == F32 and all(_dt(g) == BF16 for g in grads)
        if _dt(out.grad) != _dt(weight) or not (narrow or all(_dt(g) == _dt(weight) for g in grads)):
            raise RuntimeError(f"embedding backward: upstream {out.grad.dtype}, table {weight.dtype}, gradients "
                               f"{[str(g.dtype) for g in grads]}: the kernels take one storage type throughout, or "
                               "bf16 table gradients under fp32 activations")
        clean_but = weight.grad.dirty_rows          # (every gradient writer forgets it: _param_flag)
        flag = self._param_flag(node, weight) | (PARAM_GRAD_BF16 if narrow else 0)
        if len(outputs) > 1:
            T = 0
            if wpe is not None:
                T = indices.shape[1]
                if self._param_flag(node, wpe):
                    flag |= ACC_PARAM_GRAD2
            dwpe = wpe.grad if wpe is not None else None
            self._launch("gather_backward_sorted", [outputs[1], out.grad, weight.grad, ws, dwpe],
                         [_dt(weight), prod(indices.shape), C, V, flag] + _lo_hi(ws.nbytes)
                         + [T, _mask(outputs[1], out.grad, weight.grad, ws, dwpe)])
            node.order_ready = False        # the next forward pass orders its own ids unless told otherwise
            # the rows this call stored are the rows of the ids the forward kernel kept -- if it
            # kept them, and this is the first backward pass over that copy
            if clean_but is not None and node.kept_fresh and not any(k is node.kept_ids for k in clean_but):
                weight.grad.dirty_rows = clean_but + [node.kept_ids]
            node.kept_fresh = False
            return wpe is not None
        else:
            self._launch("gather_backward_kernel", [indices, out.grad, weight.grad, ws],
                         [_dt(weight), prod(indices.shape), C, V, flag] + _lo_hi(ws.nbytes))

    def hip_gather_forward(self, inputs, outputs, scratch=None):
        self._embedding_forward(inputs[0], inputs[1], None, outputs, scratch)

    def hip_gather_backward(self, inputs, outputs, scratch=None):
        indices, weight, out = inputs[0], inputs[1], outputs[0]
        if out.grad is None or not weight.requires_grad:
            return
        self._embedding_grad(out.op, indices, weight, outputs, scratch)

    def hip_embedding_sum_forward(self, inputs, outputs, scratch=None):
        self._embedding_forward(inputs[0], inputs[1], inputs[2], outputs, scratch)

    def hip_embedding_sum_backward(self, inputs, outputs, scratch=None):
        indices, wte, wpe = inputs
        out = outputs[0]
        if out.grad is None:
            return
        B, T = indices.shape
        fused = False
        if wte.requires_grad:
            fused = self._embedding_grad(out.op, indices, wte, outputs, scratch,
                                         wpe if wpe.requires_grad and wpe.grad is not None else None)
        if wpe.requires_grad and not fused:
            # rows beyond T of a longer table get no gradient
            self._launch("pos_emb_grad", [out.grad, wpe.grad],
                         [_dt(out), B, T, wpe.shape[1], self._param_flag(out.op, wpe)])

    # -- activations ------------------------------------------------------------------
    def _unary_forward(self, kernel, inputs, outputs):
        x, out = inputs[0], outputs[0]
        self._launch(kernel, [x, out], [_dt(x)] + _lo_hi(x.numel))

    def _unary_backward(self, kernel, inputs, outputs):
        x, out = inputs[0], outputs[0]
        if out.grad is None or not x.requires_grad:
            return
        self._launch(kernel, [out.grad, x, x.grad], [_dt(x), self._grad_flag(out.op, x)] + _lo_hi(x.numel))

    def hip_gelu_forward(self, inputs, outputs, scratch=None):
        self._unary_forward("gelu_forward_kernel", inputs, outputs)

    def hip_gelu_backward(self, inputs, outputs, scratch=None):
        self._unary_backward("gelu_backward_kernel", inputs, outputs)

    # -- GELU(h + b) (gelu_add_bias_kernel / gelu_backward_bias_kernel, metal_ops.metal:3737-3773)
    def hip_bias_gelu_forward(self, inputs, outputs, scratch=None):
        h, b, out = inputs[0], inputs[1], outputs[0]
        self._launch("gelu_add_bias_kernel", [h, b, out], [_dt(h)] + _lo_hi(prod(h.shape[:-1])) + [h.shape[-1]])

    def hip_bias_gelu_backward(self, inputs, outputs, scratch=None):
        h, b, out = inputs[0], inputs[1], outputs[0]
        if out.grad is None:
            return
        node = out.op
        dh = h.grad if h.requires_grad else None
        db = b.grad if b.requires_grad else None
        if dh is None and db is None:
            return
        flags, ws, ws_bytes = 0, None, 0
        if dh is not None:
            flags |= self._grad_flag(node, h)
        if db is not None:
            if scratch is None:
                raise RuntimeError("BiasGELU backward needs its arena workspace (plan_scratch)")
            ws = scratch["workspace"]
            ws_bytes = ws.nbytes
            if self._grad_flag(node, b):
                flags |= ACC_PARAM_GRAD
            flags |= self._defer_flag(node)
            if _dt(db) != _dt(h):
                flags |= PARAM_GRAD_BF16          # planning has checked that this is bf16 under fp32
        self._launch("gelu_backward_bias_kernel", [out.grad, h, b, dh, db, ws],
                     [_dt(h)] + _lo_hi(prod(h.shape[:-1])) + [h.shape[-1], flags] + _lo_hi(ws_bytes)
                     + [_mask(out.grad, h, b, dh, db, ws)])

    def hip_relu2_forward(self, inputs, outputs, scratch=None):
        self._unary_forward("relu2_forward_kernel", inputs, outputs)

    def hip_relu2_backward(self, inputs, outputs, scratch=None):
        self._unary_backward("relu2_backward_kernel", inputs, outputs)

    def hip_swiglu_forward(self, inputs, outputs, scratch=None):
        gu, out = inputs[0], outputs[0]
        H = out.shape[-1]
        self._launch("swiglu_forward_kernel", [gu, out], [_dt(gu), prod(out.shape[:-1]), H])

    def hip_swiglu_backward(self, inputs, outputs, scratch=None):
        gu, out = inputs[0], outputs[0]
        if out.grad is None or not gu.requires_grad:
            return
        H = out.shape[-1]
        self._launch("swiglu_backward_kernel", [gu, out.grad, gu.grad],
                     [_dt(gu), prod(out.shape[:-1]), H, self._grad_flag(out.op, gu)])

    # -- norms ----------------------------------------------------------------------
    def _norm_forward(self, kernel, x, residual, gamma, beta, h, y, eps):
        rows, C = prod(x.shape[:-1]), x.shape[-1]
        self._launch(kernel, [x, residual, gamma, beta, h, y],
                     [_dt(x), rows, C, f32_bits(eps), _mask(x, residual, gamma, beta, h, y)])

    def _norm_backward(self, kernel, node, x_saved, dy, gamma, beta, dres, dx, dx2, eps, flags, scratch):
        rows, C = prod(x_saved.shape[:-1]), x_saved.shape[-1]
        dgamma = gamma.grad if gamma is not None and gamma.requires_grad else None
        dbeta = beta.grad if beta is not None and beta.requires_grad else None
        # fp32 parameter gradients, or both stored as bf16 (the reference's bf16 gradient store)
        kinds = {_dt(g) for g in (dgamma, dbeta) if g is not None}
        if len(kinds) > 1:
            raise RuntimeError("norm backward: the gradients of gamma and beta must share one storage type")
        if kinds == {BF16}:
            flags |= PARAM_GRAD_BF16
        ws = None
        if dgamma is not None or dbeta is not None:
            flags |= self._defer_flag(node)
            if scratch is None:
                raise RuntimeError("norm backward needs its arena workspace (plan_scratch)")
            ws = scratch["workspace"]
        if dx is None and dgamma is None and dbeta is None:
            return
        self._launch(kernel, [x_saved, dy, gamma, dres, dx, dx2, dgamma, dbeta, ws],
                     [_dt(x_saved), rows, C, f32_bits(eps), flags,
                      _mask(x_saved, dy, gamma, dres, dx, dx2, dgamma, dbeta, ws)]
                     + _lo_hi(ws.nbytes if ws is not None else 0))

    def hip_layernorm_forward(self, inputs, outputs, scratch=None):
        x, gamma, beta = inputs
        self._norm_forward("layernorm_forward", x, None, gamma, beta, None, outputs[0], outputs[0].op.op.eps)

    def hip_layernorm_backward(self, inputs, outputs, scratch=None):
        x, gamma, beta = inputs
        out = outputs[0]
        if out.grad is None:
            return
        node = out.op
        dx = x.grad if x.requires_grad else None
        flags = (self._grad_flag(node, x) if dx is not None else 0) | self._param_flag(node, gamma, beta)
        self._norm_backward("layernorm_backward_kernel", node, x, out.grad, gamma, beta, None, dx, None,
                            node.op.eps, flags, scratch)

    def hip_rmsnorm_forward(self, inputs, outputs, scratch=None):
        x = inputs[0]
        gamma = inputs[1] if len(inputs) > 1 else None
        self._norm_forward("rmsnorm_forward", x, None, gamma, None, None, outputs[0], outputs[0].op.op.eps)

    def hip_rmsnorm_backward(self, inputs, outputs, scratch=None):
        x = inputs[0]
        gamma = inputs[1] if len(inputs) > 1 else None
        out = outputs[0]
        if out.grad is None:
            return
        node = out.op
        dx = x.grad if x.requires_grad else None
        flags = (self._grad_flag(node, x) if dx is not None else 0) | self._param_flag(node, gamma)
        self._norm_backward("rmsnorm_backward", node, x, out.grad, gamma, None, None, dx, None,
                            node.op.eps, flags, scratch)

    def hip_add_norm_forward(self, inputs, outputs, scratch=None):
        x, res = inputs[0], inputs[1]
        h, y = outputs
        op = h.op.op
        if isinstance(op, AddLayerNormOp):
            self._norm_forward("layernorm_forward", x, res, inputs[2], inputs[3], h, y, op.eps)
        else:
            gamma = inputs[2] if len(inputs) > 2 else None
            self._norm_forward("rmsnorm_forward", x, res, gamma, None, h, y, op.eps)

    def hip_add_norm_backward(self, inputs, outputs, scratch=None):
        """dh_total = h.grad + norm_backward(y.grad); both operands of the add
        receive dh_total (cpu_add_backward, backend.py:78-105)."""
        x, res = inputs[0], inputs[1]
        h, y = outputs
        node = h.op
        op = node.op
        is_ln = isinstance(op, AddLayerNormOp)
        gamma = inputs[2] if len(inputs) > 2 else None
        beta = inputs[3] if is_ln else None
        kernel = "layernorm_backward_kernel" if is_ln else "rmsnorm_backward"
        if y.grad is None:
            # only the residual stream carries gradient: plain add backward
            if h.grad is not None:
                for t in (x, res):
                    if t.requires_grad and t.grad is not None:
                        self._launch("add_residual_backward", [h.grad, t.grad],
                                     [_dt(h), self._grad_flag(node, t)] + _lo_hi(h.numel))
            return
        targets = [t for t in (x, res) if t.requires_grad and t.grad is not None]
        dres = h.grad                      # may be None when nothing else consumed h
        pflags = self._param_flag(node, gamma, beta)
        if not targets:
            self._norm_backward(kernel, node, h, y.grad, gamma, beta, None, None, None, op.eps, pflags, scratch)
            return
        first, second = targets[0], (targets[1] if len(targets) > 1 else None)
        flags = pflags | self._grad_flag(node, first)
        if second is not None and self._grad_flag(node, second):
            flags |= ACC_INPUT_GRAD2
        self._norm_backward(kernel, node, h, y.grad, gamma, beta, dres, first.grad,
                            second.grad if second is not None else None, op.eps, flags, scratch)

    # -- rotary (backend.py:1382-1417, 1755-1782, 1937-1958) ----------------------------
    def _rope(self, q, k, cos, sin, sign, backward, layout="bthd"):
        """q (and k, if given) rotated in place; shapes are [B,T,heads,D], or [B,heads,T,D] for layout 'bhtd'"""
        if layout == "bhtd":
            B, H, T, D = q.shape
            HKV = k.shape[1] if k is not None else 0
        else:
            B, T, H, D = q.shape
            HKV = k.shape[2] if k is not None else 0
        self._launch("rope_qk_inplace_bhtd" if layout == "bhtd" else "rope_qk_inplace", [q, k, cos, sin],
                     [_dt(q), B, T, H, HKV, D, 1 if sign == 1 else 0, 1 if backward else 0, _mask(q, k)])

    @staticmethod
    def _same_memory(a, b):
        return (a.storage.ptr.buffer_id, a.storage.ptr.offset) == (b.storage.ptr.buffer_id, b.storage.ptr.offset)

    def hip_rope_forward(self, inputs, outputs, scratch=None):
        """The kernel rotates in place.  When the runtime could alias an output
        with its input they are one buffer; otherwise (a leaf input, or one that
        is read elsewhere) the input is copied first."""
        q, k, cos, sin = inputs
        q2, k2 = outputs
        for a, b in ((q, q2), (k, k2)):
            if not self._same_memory(a, b):
                self._launch("copy_kernel", [a, b], _lo_hi(b.storage.nbytes))
        self._rope(q2, k2, cos, sin, q2.op.op.rope_sign, False, q2.op.op.layout)

    def hip_rope_backward(self, inputs, outputs, scratch=None):
        q, k, cos, sin = inputs
        q2, k2 = outputs
        gq = q2.grad if q.requires_grad else None
        gk = k2.grad if k.requires_grad else None
        if gq is None and gk is None:
            return
        sign, layout = q2.op.op.rope_sign, q2.op.op.layout
        if gq is not None:
            self._rope(gq, gk, cos, sin, sign, True, layout)
        else:
            self._rope(gk, None, cos, sin, sign, True, layout)      # k alone takes q's slot
        node = q2.op
        for src, g in ((q, gq), (k, gk)):
            if g is not None and src.grad is not None and not self._same_memory(src.grad, g):
                self._launch("add_residual_backward", [g, src.grad],
                             [_dt(src), self._grad_flag(node, src)] + _lo_hi(src.numel))

    # -- cross-entropy (backend.py:489-524) -----------------------------------------------
    def hip_cross_entropy_forward(self, inputs, outputs, scratch=None):
        logits, labels = inputs
        loss, lse = outputs
        rows, V = prod(logits.shape[:-1]), logits.shape[-1]
        self._launch("cross_entropy_forward", [logits, labels, loss, lse],
                     [_dt(logits)] + _lo_hi(rows) + [V, _mask(logits, labels, loss, lse)])

    def hip_cross_entropy_backward(self, inputs, outputs, scratch=None):
        logits, labels = inputs
        loss, lse = outputs
        if loss.grad is None or not logits.requires_grad or logits.grad is None:
            return
        rows, V = prod(logits.shape[:-1]), logits.shape[-1]
        self._launch("cross_entropy_backward", [logits, labels, loss.grad, lse, logits.grad],
                     [_dt(logits)] + _lo_hi(rows) + [V, self._grad_flag(loss.op, logits),
                                                    _mask(logits, labels, loss.grad, lse, logits.grad)])

    # -- fills and copies (backend.py:5069-5113) ---------------------------------------
    def fill_storage(self, storage, value):
        dt = np.dtype(storage.dtype)
        n = prod(storage.shape)
        if dt == np.dtype(np.float32):
            self.ctx.fill_scalar("fill_scalar_kernel", [storage.ptr.buffer_id], [storage.ptr.offset], float(value), n)
        else:
            self.fill_storage2(storage, value)

    def fill_storage2(self, storage, value):
        dt = np.dtype(storage.dtype)
        if dt == np.dtype(np.uint16):
            bits = bf16_bits(value)
        elif dt == np.dtype(np.float32):
            bits = f32_bits(value)
        elif dt.kind in "iu":
            bits = int(value) & (0xFFFFFFFF >> (8 * (4 - dt.itemsize))) if dt.itemsize <= 4 else None
        else:
            bits = None
        if bits is None or dt.itemsize not in (1, 2, 4):
            raise RuntimeError(f"fill: unsupported dtype {dt}")
        self.ctx.fill_scalar2("fill_scalar_kernel2", [storage.ptr.buffer_id], [storage.ptr.offset],
                              bits, dt.itemsize, prod(storage.shape))

    def fill(self, tensor, value):
        super().fill(tensor, value)
        tensor.dirty_rows = [] if float(value) == 0.0 else None

    def clear_table_grad(self, table):
        """table.grad = 0.  When all that is not zero in it are the rows of id lists the forward
        kernels kept (the backward passes since the last clear were embedding nodes' only), those
        rows are cleared -- N*C items a list where the fill writes V*C; otherwise the fill."""
        g = table.grad
        lists = g.dirty_rows
        if lists is None or len(table.shape) != 2:
            self.fill(g, 0)
            return
        V, C = table.shape
        for kept in lists:
            self._launch("embedding_grad_reset", [kept, g], [_dt(g), prod(kept.shape), C, V])
        g.dirty_rows = []

    def copy_from_host(self, tensor, host_np):
        tensor.dirty_rows = None
        st = tensor.storage
        dt = np.dtype(st.dtype)
        host = np.asarray(host_np)
        if dt == np.dtype(np.uint16) and host.dtype != np.dtype(np.uint16):
            host = f32_array_to_bf16_bits(np.asarray(host, dtype=np.float32))
        else:
            host = np.ascontiguousarray(host, dtype=dt)
        if host.size != prod(tensor.shape):
            raise ValueError(f"copy_from_host: {host.shape} does not fill {tensor.shape}")
        self.ctx.copy_from_host(st.ptr.buffer_id, st.ptr.offset, host.reshape(-1))

    def copy_to_host(self, tensor):
        """fp32 array for fp32 and bf16 tensors (bf16 is widened), raw otherwise"""
        if not tensor.is_contiguous:
            raise RuntimeError("copy_to_host of a permuted view: call contiguous() in the graph first")
        st = tensor.storage
        dt = np.dtype(st.dtype)
        raw = self.ctx.copy_to_host(st.ptr.buffer_id, st.ptr.offset, list(tensor.shape), dt.name)
        if dt == np.dtype(np.uint16):
            return bf16_bits_to_f32_array(raw).reshape(tensor.shape)
        return raw

    def storage_to_host(self, storage):
        """raw host copy of a storage (no dtype widening)"""
        return self.ctx.copy_to_host(storage.ptr.buffer_id, storage.ptr.offset, list(storage.shape),
                                     np.dtype(storage.dtype).name)

    def storage_from_host(self, storage, host_np):
        """raw host copy into a storage (the array already has the storage's dtype and size)"""
        host = np.ascontiguousarray(host_np, dtype=np.dtype(storage.dtype))
        if host.size != prod(storage.shape):
            raise ValueError(f"storage_from_host: {host.shape} does not fill {storage.shape}")
        self.ctx.copy_from_host(storage.ptr.buffer_id, storage.ptr.offset, host.reshape(-1))

    # -- optimizer (backend.py:5115-5140) ------------------------------------------------
    def grad_norm_sq(self, g_storage, partial, numel):
        """partial[i] = sum of squares of 256-element group i of the gradient"""
        self._launch("grad_norm_sq", [g_storage, partial], _lo_hi(int(numel)) + [_dt(g_storage)])

    def adamw8bit_step(self, p, g, qm, qv, absmax_m, absmax_v, qmap_m, qmap_v,
                       lr, lr_bc1, inv_sqrt_bc2, b1, b2, eps, weight_decay, numel, decay_numel, first_step, grad_scale=1.0):
        """One AdamW step with 8-bit moments on one parameter; the signature and the
        argument list of the launch are the Metal backend's (backend.py:5142-5151)."""
        g_bf16 = np.dtype(g.dtype) == np.dtype(np.uint16)
        if not g_bf16 and np.dtype(g.dtype) != np.dtype(np.float32):
            raise RuntimeError(f"adamw8bit: gradient dtype {g.dtype}")
        if int(numel) > 0xFFFFFFFF:
            raise RuntimeError("adamw8bit: one launch takes at most 2^32 - 1 elements")
        self._launch("adamw8bit_step", [p, g, qm, qv, absmax_m, absmax_v, qmap_m, qmap_v],
                     [f32_bits(1.0 - float(lr) * float(weight_decay)), f32_bits(lr_bc1), f32_bits(b1), f32_bits(b2),
                      f32_bits(eps), int(numel), int(decay_numel), int(bool(first_step)), f32_bits(inv_sqrt_bc2),
                      int(g_bf16), f32_bits(grad_scale)])

    def adamw_step(self, p_storage, g_storage, m_storage, v_storage, tmp_storage,
                   lr, lr_t, b1, b2, eps, weight_decay, numel=None, decay_numel=None, grad_scale=1.0,
                   lr_bc1=None, inv_sqrt_bc2=1.0):
        """One AdamW step on a flat slab.  Scalars are rounded to fp32 the way
        numpy rounds the Python floats of cpu_adamw_step (backend.py:2013-2038):
        lr*weight_decay, 1.0-b1 and 1.0-b2 are formed in double first."""
        if numel is None:
            numel = prod(p_storage.shape)
        if decay_numel is None:
            decay_numel = numel if weight_decay != 0.0 else 0
        lr_wd = float(lr) * float(weight_decay) if weight_decay > 0.0 else 0.0
        step_lr = lr_t if lr_bc1 is None else lr_bc1
        floats = [lr_wd, b1, 1.0 - b1, b2, 1.0 - b2, eps, step_lr, inv_sqrt_bc2, grad_scale]
        self._launch("adamw_step", [p_storage, g_storage, m_storage, v_storage],
                     [f32_bits(x) for x in floats] + _lo_hi(int(numel)) + _lo_hi(int(decay_numel))
                     + [_dt(g_storage)])

    def begin_pass(self):
        if not self._capturing:
            self.ctx.begin_pass()

    def end_pass(self):
        # a pass boundary waits for the GPU, which a recording cannot contain
        if not self._capturing:
            self.ctx.end_pass()

    # -- graphs -----------------------------------------------------------------------
    def capture_begin(self):
        """record every launch until capture_end instead of running it"""
        self.ctx.graph_begin()
        self._capturing = True

    def capture_end(self):
        self._capturing = False
        return self.ctx.graph_end()

    def graph_launch(self, graph_id):
        self.ctx.graph_launch(graph_id)

    def graph_destroy(self, graph_id):
        self.ctx.graph_destroy(graph_id)

    def synchronize(self):
        self.ctx.synchronize()
