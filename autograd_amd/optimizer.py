"""AdamW over the runtime's parameter slabs, and the gradient-norm clip
(counterpart of the reference's optimizer.py:11-20, 54-140, 443-600).

Only the fp32-state optimizer is provided (`state_mode="fp32"`); the reference's
8-bit and "mini" state modes are outside this package.

On a device whose backend owns a native context, parameters that the runtime
packed into one slab (matrices first, then vectors) are updated by ONE kernel
launch per slab, with the matrix-shaped prefix receiving weight decay
(optimizer.py:97-140).  On other devices every parameter is updated on its own
(optimizer.py:488-498).

`bias_correction` chooses between the reference's two equivalent ways of
applying the Adam bias correction:
  "folded"  step = lr * sqrt(1 - b2^t) / (1 - b1^t), denominator sqrt(v) + eps
            -- the reference's CPU path (optimizer.py:445, backend.py:2034-2038);
            the default, so that results match the CPU implementation bit for bit;
  "split"   step = lr / (1 - b1^t), denominator sqrt(v) / sqrt(1 - b2^t) + eps
            -- the reference's Metal path (optimizer.py:480-486).
"""
from __future__ import annotations

import math
from math import prod

import numpy as np

from .storage import Storage
from .utils import itemsize

VALID_MODE = {"fp32", "8bit", "mini"}


def get_lr_cosine_schedule(step, max_steps, warmup_steps, max_lr, min_lr):
    """linear warm-up, then half a cosine from max_lr down to min_lr (optimizer.py:11-20)"""
    if step < warmup_steps:
        return max_lr * (step + 1) / warmup_steps
    if step > max_steps:
        return min_lr
    ratio = (step - warmup_steps) / (max_steps - warmup_steps)
    return min_lr + 0.5 * (1.0 + math.cos(math.pi * ratio)) * (max_lr - min_lr)


def _span(storage, numel, dtype):
    ptr = type(storage.ptr)(storage.ptr.buffer_id, storage.ptr.offset)
    return Storage(ptr, (numel,), dtype, storage.device, numel * itemsize(dtype))


class AdamW:
    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, state_mode="fp32",
                 runtime=None, bias_correction="folded"):
        if state_mode not in VALID_MODE:
            raise ValueError(f"invalid state_mode={state_mode!r}, expected one of {VALID_MODE}")
        if state_mode != "fp32":
            raise NotImplementedError(f"state_mode={state_mode!r}: only fp32 optimizer state is provided")
        if bias_correction not in ("folded", "split"):
            raise ValueError(f"bias_correction={bias_correction!r}: expected 'folded' or 'split'")
        self.params = [p for p in params if p.requires_grad]
        self.lr, self.betas, self.eps, self.weight_decay = lr, betas, eps, weight_decay
        self.state_mode, self.bias_correction = state_mode, bias_correction
        self.t = 0
        self.m, self.v = [], []
        self.dispatches = ()
        self._state = []
        if runtime is None:
            from .runtime import Runtime
            runtime = Runtime.get_default()
        self.runtime = runtime
        self.backend = runtime.backend
        self.allocator = runtime.allocator
        if not self.params:
            return
        for p in self.params:
            if p.storage is None or p.grad is None or p.grad.storage is None:
                raise RuntimeError(f"parameter {getattr(p, 'name', '?')} has no storage yet: bind the graph first")
            if np.dtype(p.dtype) != np.dtype(np.float32):
                raise RuntimeError("AdamW keeps fp32 master parameters; got " + str(p.dtype))
        if hasattr(self.backend, "ctx"):
            self._prepare_merged()
        else:
            self._prepare_per_parameter()

    # one (p, g, m, v, numel, decay_numel) per launch -------------------------------------
    def _prepare_per_parameter(self):
        out = []
        for p in self.params:
            m = self.allocator.zeros(p.shape, np.float32)
            v = self.allocator.zeros(p.shape, np.float32)
            self._state += [m, v]
            self.m.append(m)
            self.v.append(v)
            n = prod(p.shape)
            out.append((p.storage, p.grad.storage, m, v, n, n if p.ndim > 1 else 0))
        self.dispatches = tuple(out)

    def _prepare_merged(self):
        groups = {}
        for i, p in enumerate(self.params):
            groups.setdefault(p.storage.ptr.buffer_id, []).append(i)
        self.m = [None] * len(self.params)
        self.v = [None] * len(self.params)
        out = []
        view = self.allocator.view
        for indices in groups.values():
            indices.sort(key=lambda i: self.params[i].storage.ptr.offset)
            first = self.params[indices[0]]
            start = first.storage.ptr.offset
            end = max(self.params[i].storage.ptr.offset + self.params[i].storage.nbytes for i in indices)
            numel = (end - start) // 4
            m_all = self.allocator.zeros((numel,), np.float32)
            v_all = self.allocator.zeros((numel,), np.float32)
            self._state += [m_all, v_all]
            merge, decay_numel, saw_vector = True, numel, False
            g_dtype = first.grad.storage.dtype
            for i in indices:
                p = self.params[i]
                off = p.storage.ptr.offset - start
                self.m[i] = view(m_all, off, p.shape, np.float32)
                self.v[i] = view(v_all, off, p.shape, np.float32)
                g = p.grad.storage
                # one launch needs the gradients laid out like the parameters
                if (g.dtype != g_dtype or g.ptr.buffer_id != first.grad.storage.ptr.buffer_id
                        or (g.ptr.offset - first.grad.storage.ptr.offset) * 4 != off * itemsize(g.dtype)):
                    merge = False
                if p.ndim <= 1:
                    if not saw_vector:
                        decay_numel, saw_vector = off // 4, True
                elif saw_vector:
                    merge = False
            if merge:
                # the span from the first parameter to the end of the last one: wider
                # than any one parameter's storage, so it is described directly
                # (every launch is still bounds-checked against the real allocation)
                p_all = _span(first.storage, numel, np.float32)
                g_all = _span(first.grad.storage, numel, g_dtype)
                out.append((p_all, g_all, m_all, v_all, numel, decay_numel))
            else:
                for i in indices:
                    p = self.params[i]
                    n = prod(p.shape)
                    out.append((p.storage, p.grad.storage, self.m[i], self.v[i], n, n if p.ndim > 1 else 0))
        self.dispatches = tuple(out)

    # ------------------------------------------------------------------------------------
    def step(self, grad_scale=1.0):
        """one update of every parameter (optimizer.py:443-500)"""
        self.t += 1
        b1, b2 = self.betas
        lr_t = self.lr * math.sqrt(1.0 - b2 ** self.t) / (1.0 - b1 ** self.t)
        lr_bc1 = inv_sqrt_bc2 = None
        if self.bias_correction == "split":
            lr_bc1 = self.lr / (1.0 - b1 ** self.t)
            inv_sqrt_bc2 = 1.0 / math.sqrt(1.0 - b2 ** self.t)
        self.backend.begin_pass()
        for p, g, m, v, numel, decay_numel in self.dispatches:
            self.backend.adamw_step(p, g, m, v, None, self.lr, lr_t, b1, b2, self.eps, self.weight_decay,
                                    numel=numel, decay_numel=decay_numel, grad_scale=grad_scale,
                                    lr_bc1=lr_bc1, inv_sqrt_bc2=1.0 if inv_sqrt_bc2 is None else inv_sqrt_bc2)
        self.backend.end_pass()

    def zero_grad(self):
        for p in self.params:
            if p.grad is not None:
                self.backend.fill_storage2(p.grad.storage, 0.0)

    def build_grad_clip(self):
        """-> clip_grad_norm(max_norm, eps=1e-6) -> (grad_norm, clip_coef); the
        coefficient is handed to step(grad_scale=...) rather than applied to the
        gradients (optimizer.py:505-600)."""
        items = [(g, int(n)) for _, g, _, _, n, _ in self.dispatches]
        partials = [self.allocator.empty(((n + 255) // 256,), np.float32) for _, n in items]
        self._state += partials

        def clip_grad_norm(max_norm, eps=1e-6):
            self.backend.begin_pass()
            for (g, n), part in zip(items, partials):
                self.backend.grad_norm_sq(g, part, n)
            self.backend.end_pass()
            norm_sq = 0.0
            for part in partials:
                norm_sq += float(np.sum(self.backend.storage_to_host(part), dtype=np.float64))
            grad_norm = math.sqrt(norm_sq)
            if not math.isfinite(grad_norm):
                return grad_norm, 0.0
            return grad_norm, min(1.0, float(max_norm) / (grad_norm + eps))

        return clip_grad_norm

    def release(self):
        rel = getattr(self.allocator, "release", None)
        if rel is not None:
            for s in self._state:
                rel(s)
        self._state = []
