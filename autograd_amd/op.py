"""Graph operators of the fused layer-op path.

Same contract as the reference's op.py: an Op instance is called on input
Tensors, infers the output shape, and records an OpNode on every output
(`out.op`); the runtime later binds `node.forward` / `node.backward` to backend
kernels looked up by the exact type of the op (op.py:13-50, runtime.py:241-243).

AddOp, GatherOp, GELUOp and LayerNormOp keep the reference's names, arguments
and shape checks (op.py:52-59, 219-267).  RMSNorm, SwiGLU, rotary and the
residual-fused norms exist in the reference only inside fused GEMM ops
(op.py:395-507); here they are ops of their own.  ReLU^2 and EmbeddingSum are
new.
"""
from __future__ import annotations

from abc import ABC, abstractmethod

import numpy as np

from .tensor import Tensor
from .utils import broadcast_shape, mul_bcast_kind


class OpNode:
    __slots__ = ("op", "inputs", "outputs", "forward", "backward", "scratch_fwd_layout",
                 "scratch_bwd_layout", "name", "overwrite_grads", "defer_param_grads", "order_ready", "kept_ids", "kept_fresh")

    def __init__(self, op, inputs, outputs, name=""):
        self.op = op
        self.inputs = tuple(inputs)
        self.outputs = tuple(outputs)
        self.forward = None
        self.backward = None
        self.scratch_fwd_layout = None
        self.scratch_bwd_layout = None
        self.name = name
        # ids of gradient tensors this node is the first to write in a backward
        # pass: its kernel may store instead of accumulate (set by the runtime)
        self.overwrite_grads = frozenset()
        # the backward kernel leaves its parameter-gradient column sums (dgamma / dbeta, a bias
        # gradient) unfolded and the runtime folds all of a pass's sums in one launch at the
        # end of the pass (set by the runtime; the node's backward scratch then lives that long)
        self.defer_param_grads = False
        # an embedding node whose ids have already been ordered for this step's gradient (the
        # ordering rode with the zero fill of the table's gradient): its forward kernel is then
        # the plain gather.  Set by Runtime.execute, cleared by the node's backward kernel.
        self.order_ready = False
        # an embedding node whose table has a gradient: a buffer outside the arena in which the
        # forward kernel leaves a copy of the ids it read (set by the runtime), and whether that
        # copy is of the forward pass the next backward pass belongs to.  The table's gradient is
        # then cleared row by row (those ids' rows) instead of as a whole.
        self.kept_ids = None
        self.kept_fresh = False


class Op(ABC):
    op_name = "Op"
    recompute_output = False
    # One store-or-accumulate choice covers all of this op's parameter gradients (gamma and beta of a
    # norm share a flag bit of the kernel).  False where every parameter has a flag of its own.
    shared_param_grad_flag = True
    # indices of outputs that may be written before the forward pass starts (the id order of
    # an embedding, written together with the gradient's zero fill): they hold their arena
    # bytes from the first step on
    early_outputs = ()
    # indices (output i aliases input j): the kernel works in place, the
    # runtime gives output and input (and their grads) the same memory
    inplace_aliases: dict = {}
    # index of the input that output 0 is a view of (same memory, other shape or
    # strides); such an output gets no memory of its own
    view_of_input = None
    # only ops that read through strides take a permuted / transposed view
    accepts_strided = False

    def require_contiguous(self, inputs):
        if self.accepts_strided:
            return
        for t in inputs:
            if not t.is_contiguous:
                raise RuntimeError(f"{self.op_name} requires contiguous inputs (got strides {t.strides} for shape "
                                   f"{t.shape}); call contiguous() first")

    def __call__(self, *inputs):
        self.require_contiguous(inputs)
        shape = self.infer_shape(*inputs)
        out = Tensor(shape=shape, dtype=self.infer_dtype(*inputs), device=inputs[0].device,
                     requires_grad=any(t.requires_grad for t in inputs))
        out.op = OpNode(op=self, inputs=inputs, outputs=(out,))
        return out

    @abstractmethod
    def infer_shape(self, *inputs):
        ...

    def infer_dtype(self, *inputs):
        return inputs[0].dtype

    def save_for_backward(self, inputs, outputs):
        return list(inputs) + list(outputs)

    def is_recompute_output(self):
        return self.recompute_output

    def fully_written_inputs(self, inputs, outputs):
        """indices of inputs whose whole gradient tensor this op's backward writes
        (so a first writer may store instead of accumulating onto zeros)"""
        return []

    def __repr__(self):
        return self.op_name


class AddOp(Op):
    op_name = "Add"

    def infer_shape(self, x, y):
        return broadcast_shape(x.shape, y.shape)

    def save_for_backward(self, inputs, outputs):
        return []

    def fully_written_inputs(self, inputs, outputs):
        return [0, 1]


class MulOp(Op):
    """out = x * y; y has x's shape, its trailing [C], one factor per row ([..., 1]) or
    one element (op.py:61-69; the broadcast kinds of utils.py:134-143)"""
    op_name = "Mul"

    def infer_shape(self, x, y):
        shape = broadcast_shape(x.shape, y.shape)
        if tuple(shape) != tuple(x.shape):
            raise RuntimeError(f"Mul: the second operand is the broadcast one, got x={x.shape} y={y.shape}")
        mul_bcast_kind(x.shape, y.shape)      # raises on a kind the kernels do not have
        return shape

    def save_for_backward(self, inputs, outputs):
        return list(inputs)

    def fully_written_inputs(self, inputs, outputs):
        return [0, 1]


class _UnaryOp(Op):
    saves_output = True      # backward reads y (exp, rsqrt) rather than x (log)

    def infer_shape(self, x):
        return x.shape

    def save_for_backward(self, inputs, outputs):
        return list(outputs) if self.saves_output else list(inputs)

    def fully_written_inputs(self, inputs, outputs):
        return [0]


class ExpOp(_UnaryOp):
    op_name = "Exp"


class LogOp(_UnaryOp):
    op_name = "Log"
    saves_output = False


class RsqrtOp(_UnaryOp):
    op_name = "Rsqrt"


class SoftmaxOp(_UnaryOp):
    """softmax over `dim` (op.py:205-218; any axis, as cpu_softmax_forward takes it,
    backend.py:354-362).  The kernels work along the last axis; another axis is moved
    there and back through scratch copies."""
    op_name = "Softmax"

    def __init__(self, dim=-1):
        self.dim = dim

    def infer_shape(self, x):
        if x.ndim == 0 or not -x.ndim <= self.dim < x.ndim:
            raise ValueError(f"Softmax: dim={self.dim} for a tensor of {x.ndim} axes")
        return x.shape

    def axis(self, x):
        return self.dim % x.ndim


# -- views and layout changes (op.py:89-185) --------------------------------------
def resolve_reshape_shape(numel, target_shape):
    """target shape with its single -1 filled in (utils.py:85-100)"""
    shape = list(target_shape)
    holes = [i for i, d in enumerate(shape) if d == -1]
    if len(holes) > 1:
        raise ValueError(f"reshape: at most one -1, got {tuple(target_shape)}")
    known = 1
    for d in shape:
        if d != -1:
            known *= d
    if known == 0:
        raise ValueError(f"reshape: invalid target_shape {tuple(target_shape)}")
    if holes:
        if numel % known != 0:
            raise ValueError(f"reshape: numel {numel} not divisible by {known},target={tuple(target_shape)}")
        shape[holes[0]] = numel // known
    elif known != numel:
        raise ValueError(f"reshape: numel mismatch: {numel} -> {tuple(shape)}")
    return tuple(shape)


class _LayoutOp(Op):
    """output 0 shares input 0's memory; forward launches nothing"""
    view_of_input = 0
    accepts_strided = True

    def _make(self, x, shape, strides, is_contiguous):
        out = Tensor(shape=shape, dtype=x.dtype, strides=strides, offset=x.offset, is_contiguous=is_contiguous,
                     requires_grad=x.requires_grad, device=x.device)
        out.op = OpNode(op=self, inputs=(x,), outputs=(out,))
        return out

    def save_for_backward(self, inputs, outputs):
        return []       # the gradient kernels read gradients only

    def fully_written_inputs(self, inputs, outputs):
        return [0]


class ReshapeOp(_LayoutOp):
    """same elements under another shape; the input must be contiguous (utils.py:102-109)"""
    op_name = "Reshape"

    def __init__(self, shape):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = shape[0]
        self.shape = tuple(shape)

    def infer_shape(self, x):
        return resolve_reshape_shape(x.numel, self.shape)

    def __call__(self, x):
        shape = self.infer_shape(x)
        if not x.is_contiguous:
            raise RuntimeError("reshape view requires contiguous input")
        return self._make(x, shape, None, True)


class ViewOp(ReshapeOp):
    op_name = "View"

    def __call__(self, x):
        if not x.is_contiguous:
            raise RuntimeError("view requires contiguous")
        return super().__call__(x)


class PermuteOp(_LayoutOp):
    """out.shape[i] = x.shape[dims[i]]; a view with permuted strides"""
    op_name = "Permute"

    def __init__(self, dims):
        if len(dims) == 1 and isinstance(dims[0], (tuple, list)):
            dims = dims[0]
        self.dims = tuple(int(d) for d in dims)

    def infer_shape(self, x):
        if sorted(d % x.ndim for d in self.dims) != list(range(x.ndim)):
            raise ValueError(f"permute: {self.dims} is not a permutation of {x.ndim} dimensions")
        return tuple(x.shape[d] for d in self.dims)

    def __call__(self, x):
        shape = self.infer_shape(x)
        return self._make(x, shape, tuple(x.strides[d] for d in self.dims), False)


class TransposeOp(_LayoutOp):
    op_name = "Transpose"

    def __init__(self, dim0, dim1):
        self.dim0 = dim0
        self.dim1 = dim1

    def infer_shape(self, x):
        shape = list(x.shape)
        shape[self.dim0], shape[self.dim1] = shape[self.dim1], shape[self.dim0]
        return tuple(shape)

    def __call__(self, x):
        shape = self.infer_shape(x)
        strides = list(x.strides)
        strides[self.dim0], strides[self.dim1] = strides[self.dim1], strides[self.dim0]
        return self._make(x, shape, tuple(strides), False)


class ContiguousOp(Op):
    """a dense copy of a (possibly permuted) view"""
    op_name = "Contiguous"
    accepts_strided = True

    def infer_shape(self, x):
        return x.shape

    def save_for_backward(self, inputs, outputs):
        return []

    def fully_written_inputs(self, inputs, outputs):
        return [0]


def _order_output(indices, table):
    """When the table needs a gradient, the embedding ops carry a second,
    gradient-free output of 6N + 128 uint32: the rows ordered so that each token's rows are
    adjacent and ascending, what every row is told about its token's run, and the
    gradient kernel's arrival counters.  A
    device may fill it in its forward kernel (where ordering the ids is free) and
    start its backward kernel from it; a device that has no use for it leaves it
    alone.  `__call__` still returns the embedding only."""
    if not table.requires_grad:
        return ()
    n = 1
    for d in indices.shape:
        n *= d
    return (Tensor(shape=(6 * n + 128,), dtype=np.uint32, requires_grad=False, device=table.device),)


class GatherOp(Op):
    """out[b, t, :] = weight[indices[b, t], :]"""
    op_name = "Gather"
    early_outputs = (1,)

    def infer_shape(self, indices, weight):
        if indices.ndim != 2:
            raise ValueError("Gather indices must be 2D (B, T)")
        if weight.ndim != 2:
            raise ValueError("Gather weight must be 2D (V, C)")
        return indices.shape + (weight.shape[1],)

    def __call__(self, indices, weight):
        self.require_contiguous((indices, weight))
        out = Tensor(shape=self.infer_shape(indices, weight), dtype=weight.dtype,
                     requires_grad=weight.requires_grad, device=weight.device)
        outputs = (out,) + _order_output(indices, weight)
        node = OpNode(op=self, inputs=(indices, weight), outputs=outputs)
        for t in outputs:
            t.op = node
        return out

    def save_for_backward(self, inputs, outputs):
        return list(inputs) + list(outputs[1:])


class EmbeddingSumOp(Op):
    """out[b, t, :] = wte[indices[b, t], :] + wpe[t, :] -- the GPT-2 input
    embedding tok_emb(ids) + pos_emb(arange(T)) as one op
    (check_tiny_gpt2_kernel.py:282,301)."""
    op_name = "EmbeddingSum"
    early_outputs = (1,)
    shared_param_grad_flag = False      # the token table and the position table have a flag each

    def infer_shape(self, indices, wte, wpe):
        if indices.ndim != 2 or wte.ndim != 2 or wpe.ndim != 2:
            raise ValueError("EmbeddingSum takes indices (B, T), wte (V, C), wpe (T_max, C)")
        if wte.shape[1] != wpe.shape[1]:
            raise ValueError("EmbeddingSum C mismatch")
        if wpe.shape[0] < indices.shape[1]:
            raise ValueError("EmbeddingSum: position table shorter than the sequence")
        return indices.shape + (wte.shape[1],)

    def __call__(self, indices, wte, wpe):
        self.require_contiguous((indices, wte, wpe))
        out = Tensor(shape=self.infer_shape(indices, wte, wpe), dtype=wte.dtype, device=wte.device,
                     requires_grad=wte.requires_grad or wpe.requires_grad)
        outputs = (out,) + _order_output(indices, wte)
        node = OpNode(op=self, inputs=(indices, wte, wpe), outputs=outputs)
        for t in outputs:
            t.op = node
        return out

    def save_for_backward(self, inputs, outputs):
        return [inputs[0]] + list(outputs[1:])

    def fully_written_inputs(self, inputs, outputs):
        return [2] if inputs[2].shape[0] == inputs[0].shape[1] else []


class GELUOp(Op):
    op_name = "GELU"

    def infer_shape(self, x):
        return x.shape

    def save_for_backward(self, inputs, outputs):
        return list(inputs)

    def fully_written_inputs(self, inputs, outputs):
        return [0]


class BiasGELUOp(Op):
    """y = GELU(h + b) with b the trailing [C] of h: the bias add of a linear layer folded
    into its activation (gelu_add_bias_kernel / gelu_backward_bias_kernel,
    metal_ops.metal:3737-3773; as a graph the reference writes Add then GELU, op.py:47-59, 241-245)"""
    op_name = "BiasGELU"

    def infer_shape(self, h, b):
        trailing = tuple(b.shape)
        while len(trailing) > 1 and trailing[0] == 1:
            trailing = trailing[1:]
        if len(h.shape) < 1 or trailing != (h.shape[-1],):
            raise RuntimeError(f"BiasGELU: the bias must be the trailing [C] of h, got h={h.shape} b={b.shape}")
        return h.shape

    def save_for_backward(self, inputs, outputs):
        return list(inputs)

    def fully_written_inputs(self, inputs, outputs):
        return [0, 1]


class ReLUSquaredOp(Op):
    op_name = "ReLUSquared"

    def infer_shape(self, x):
        return x.shape

    def save_for_backward(self, inputs, outputs):
        return list(inputs)

    def fully_written_inputs(self, inputs, outputs):
        return [0]


class SwiGLUOp(Op):
    """gu[..., 2H] -> silu(gu[..., :H]) * gu[..., H:]"""
    op_name = "SwiGLU"

    def infer_shape(self, gu):
        if gu.shape[-1] % 2 != 0:
            raise ValueError("SwiGLU last dimension must be even (gate | up)")
        return gu.shape[:-1] + (gu.shape[-1] // 2,)

    def save_for_backward(self, inputs, outputs):
        return list(inputs)

    def fully_written_inputs(self, inputs, outputs):
        return [0]


class LayerNormOp(Op):
    op_name = "LayerNorm"

    def __init__(self, normalized_dim=-1, eps=1e-6):
        if normalized_dim != -1:
            raise ValueError("LayerNorm normalises the last dimension")
        self.normalized_dim = normalized_dim
        self.eps = eps

    def infer_shape(self, x, gamma, beta):
        if gamma.shape != beta.shape:
            raise ValueError("gamma/beta shape mismatch")
        if x.shape[self.normalized_dim] != gamma.shape[0]:
            raise ValueError("LayerNorm C mismatch")
        return x.shape

    def save_for_backward(self, inputs, outputs):
        return list(inputs)

    def fully_written_inputs(self, inputs, outputs):
        return [0, 1, 2]


class RMSNormOp(Op):
    """z = x / sqrt(mean(x^2) + eps) [* gamma]; inputs (x,) or (x, gamma)."""
    op_name = "RMSNorm"

    def __init__(self, eps=1e-6):
        self.eps = eps

    def infer_shape(self, x, gamma=None):
        if gamma is not None and gamma.shape != (x.shape[-1],):
            raise ValueError(f"norm_weight shape must be ({x.shape[-1]},), got {gamma.shape}")
        return x.shape

    def save_for_backward(self, inputs, outputs):
        return list(inputs)

    def fully_written_inputs(self, inputs, outputs):
        return list(range(len(inputs)))


class CrossEntropyLossOp(Op):
    """loss[b, t] = -log softmax(logits[b, t, :])[labels[b, t]]  (op.py:269-284).

    The node has a second, gradient-free output: the row's log-sum-exp, which
    the backward kernel uses instead of reducing the row again.  `__call__`
    returns the loss only, like the reference's op.  loss is fp32 whatever the
    logits' type."""
    op_name = "CrossEntropyLoss"

    def __init__(self, dim=-1):
        if dim != -1:
            raise ValueError("CrossEntropyLoss reduces the last axis")
        self.dim = dim

    def infer_shape(self, logits, labels):
        if logits.shape[:-1] != labels.shape:
            raise ValueError("CE shape mismatch")
        return labels.shape

    def __call__(self, logits, labels):
        self.require_contiguous((logits, labels))
        shape = self.infer_shape(logits, labels)
        loss = Tensor(shape=shape, dtype=np.float32, requires_grad=logits.requires_grad, device=logits.device)
        lse = Tensor(shape=shape, dtype=np.float32, requires_grad=False, device=logits.device)
        node = OpNode(op=self, inputs=(logits, labels), outputs=(loss, lse))
        loss.op = node
        lse.op = node
        return loss

    def save_for_backward(self, inputs, outputs):
        return list(inputs) + [outputs[1]]

    def fully_written_inputs(self, inputs, outputs):
        return [0]


class _AddNormOp(Op):
    """(h, y) = (x + residual, norm(x + residual)).  Two outputs: h continues
    the residual stream, y feeds the next block."""
    n_norm_params = 0

    def __call__(self, *inputs):
        self.require_contiguous(inputs)
        x, res = inputs[0], inputs[1]
        if x.shape != res.shape:
            raise ValueError("fused residual add needs operands of one shape")
        self.infer_shape(*inputs)
        req = any(t.requires_grad for t in inputs)
        h = Tensor(shape=x.shape, dtype=x.dtype, device=x.device, requires_grad=req)
        y = Tensor(shape=x.shape, dtype=x.dtype, device=x.device, requires_grad=req)
        node = OpNode(op=self, inputs=inputs, outputs=(h, y))
        h.op = node
        y.op = node
        return h, y

    def save_for_backward(self, inputs, outputs):
        return [outputs[0]] + list(inputs[2:])

    def fully_written_inputs(self, inputs, outputs):
        return list(range(len(inputs)))


class AddLayerNormOp(_AddNormOp):
    op_name = "AddLayerNorm"

    def __init__(self, eps=1e-5):
        self.eps = eps
        self.normalized_dim = -1

    def infer_shape(self, x, res, gamma, beta):
        if gamma.shape != beta.shape or gamma.shape != (x.shape[-1],):
            raise ValueError("AddLayerNorm gamma/beta shape mismatch")
        return x.shape


class AddRMSNormOp(_AddNormOp):
    op_name = "AddRMSNorm"

    def __init__(self, eps=1e-6):
        self.eps = eps

    def infer_shape(self, x, res, gamma=None):
        if gamma is not None and gamma.shape != (x.shape[-1],):
            raise ValueError("AddRMSNorm gamma shape mismatch")
        return x.shape


class RopeOp(Op):
    """Split-half rotary embedding of q [B,T,H,D] and k [B,T,HKV,D] with tables
    cos/sin [T_max, D/2].  rope_sign=+1 is the HF convention, -1 the nanochat
    one (FusedRMSNormGQAOp.rope_sign, op.py:486-491).  Works in place: the
    outputs take over the inputs' memory."""
    op_name = "Rope"
    inplace_aliases = {0: 0, 1: 1}

    def __init__(self, rope_sign=1, layout="bthd"):
        if rope_sign not in (1, -1):
            raise ValueError("rope_sign must be +1 or -1")
        if layout not in ("bthd", "bhtd"):
            raise ValueError("layout must be 'bthd' (the CPU kernels', backend.py:1383) or 'bhtd' (attention's)")
        self.rope_sign = rope_sign
        self.layout = layout

    def infer_shape(self, q, k, cos, sin):
        t_axis, h_axis = (1, 2) if self.layout == "bthd" else (2, 1)
        if (q.ndim != 4 or k.ndim != 4 or q.shape[0] != k.shape[0] or q.shape[t_axis] != k.shape[t_axis]
                or q.shape[3] != k.shape[3]):
            raise ValueError("Rope takes q (B,T,H,D) and k (B,T,HKV,D), or (B,H,T,D) and (B,HKV,T,D) with layout='bhtd'")
        D = q.shape[3]
        if D % 2 or cos.shape != sin.shape or cos.ndim != 2 or cos.shape[1] != D // 2 or cos.shape[0] < q.shape[t_axis]:
            raise ValueError("Rope tables must be (T_max >= T, D/2)")
        return q.shape, k.shape

    def __call__(self, q, k, cos, sin):
        self.require_contiguous((q, k, cos, sin))
        qs, ks = self.infer_shape(q, k, cos, sin)
        q2 = Tensor(shape=qs, dtype=q.dtype, device=q.device, requires_grad=q.requires_grad)
        k2 = Tensor(shape=ks, dtype=k.dtype, device=k.device, requires_grad=k.requires_grad)
        node = OpNode(op=self, inputs=(q, k, cos, sin), outputs=(q2, k2))
        q2.op = node
        k2.op = node
        return q2, k2

    def save_for_backward(self, inputs, outputs):
        return [inputs[2], inputs[3]]


INT_DTYPES = (np.dtype(np.int32),)
