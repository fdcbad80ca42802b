"""AdamW over the runtime's parameter slabs, and the gradient-norm clip
(counterpart of the reference's optimizer.py:11-20, 54-140, 443-600).

`state_mode="fp32"` keeps both moments in fp32; `state_mode="8bit"` keeps them as
one byte per element plus one fp32 scale per block of 256 (optimizer.py:143-232,
469-479) for every parameter of at least 4096 elements, fp32 below that.  The
reference's "mini" mode is outside this package.

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


def build_dynamic_map(signed, max_exponent_bits=7, total_bits=8):
    """The sorted 256-entry code book of the 8-bit moments (optimizer.py:144-179):
    per decade 10^-6 .. 10^0 the centres of 2^k equal bins of [0.1, 1] (k grows by one
    per decade; the unsigned map starts one power higher and has one more value below
    the last decade), mirrored when signed, zero-padded to 256, sorted, and scaled so
    that the largest magnitude is exactly 1."""
    f32 = np.float32
    magnitude_bits = total_bits - 1 if signed else total_bits
    runs = []
    for decade in range(max_exponent_bits):
        edges = np.linspace(0.1, 1.0, 2 ** (decade + magnitude_bits - max_exponent_bits) + 1, dtype=f32)
        runs.append((edges[:-1] + edges[1:]) * f32(0.5) * f32(10.0 ** (decade - (max_exponent_bits - 1))))
    below = 2 ** (magnitude_bits - max_exponent_bits) - 1
    if below > 0:
        edges = np.linspace(0.0, 0.1, below + 1, dtype=f32)
        runs.append((edges[:-1] + edges[1:]) * f32(0.5) * f32(10.0 ** (-(max_exponent_bits - 1))))
    # the reference collects the values as Python floats before rounding them back to fp32
    positive = np.concatenate(runs).astype(np.float64)
    values = np.concatenate([positive, -positive]) if signed else positive
    size = 1 << total_bits
    if values.size >= size:
        raise RuntimeError(f"invalid dynamic-map size: {values.size}")
    qmap = np.zeros(size, f32)
    qmap[:values.size] = values.astype(f32)
    qmap.sort()
    qmap /= np.max(np.abs(qmap))
    return np.ascontiguousarray(qmap, dtype=f32)


def _span(storage, numel, dtype):
    ptr = type(storage.ptr)(storage.ptr.buffer_id, storage.ptr.offset)
    return Storage(ptr, (numel,), dtype, storage.device, numel * itemsize(dtype))


class AdamW:
    BLOCK_SIZE = 256          # elements per scale of the 8-bit moments (optimizer.py:50)

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, state_mode="fp32",
                 runtime=None, bias_correction="folded"):
        if state_mode not in VALID_MODE:
            raise ValueError(f"invalid state_mode={state_mode!r}, expected one of {VALID_MODE}")
        if state_mode == "mini":
            raise NotImplementedError("state_mode='mini': only fp32 and 8-bit optimizer state are provided")
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
        self.qmap_m = self.qmap_v = None
        if state_mode == "8bit":
            self._prepare_8bit()
        elif hasattr(self.backend, "ctx"):
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

    # ("fp32", p, g, m, v, numel, decays) or ("q8", p, g, qm, qv, absmax_m, absmax_v, numel, decays)
    # per parameter (optimizer.py:143-232) ------------------------------------------------
    def _prepare_8bit(self, min_8bit_size=4096):
        if not hasattr(self.backend, "adamw8bit_step"):
            raise NotImplementedError("this device's backend has no 8-bit AdamW step")
        self.qmap_m = self.allocator.empty((256,), np.float32)
        self.qmap_v = self.allocator.empty((256,), np.float32)
        self.backend.storage_from_host(self.qmap_m, build_dynamic_map(signed=True))
        self.backend.storage_from_host(self.qmap_v, build_dynamic_map(signed=False))
        self._state += [self.qmap_m, self.qmap_v]
        out = []
        for p in self.params:
            n = prod(p.shape)
            if n < min_8bit_size:                  # small state is not worth quantising
                m = self.allocator.zeros(p.shape, np.float32)
                v = self.allocator.zeros(p.shape, np.float32)
                self._state += [m, v]
                out.append(("fp32", p.storage, p.grad.storage, m, v, n, p.ndim > 1))
            else:
                blocks = (n + self.BLOCK_SIZE - 1) // self.BLOCK_SIZE
                m = self.allocator.zeros((n,), np.uint8)
                v = self.allocator.zeros((n,), np.uint8)
                absmax_m = self.allocator.zeros((blocks,), np.float32)
                absmax_v = self.allocator.zeros((blocks,), np.float32)
                self._state += [m, v, absmax_m, absmax_v]
                out.append(("q8", p.storage, p.grad.storage, m, v, absmax_m, absmax_v, n, p.ndim > 1))
            self.m.append(m)
            self.v.append(v)
        self.dispatches = tuple(out)

    def _step_8bit(self, grad_scale):
        b1, b2 = self.betas
        lr_t = self.lr * math.sqrt(1.0 - b2 ** self.t) / (1.0 - b1 ** self.t)
        lr_bc1 = self.lr / (1.0 - b1 ** self.t)
        inv_sqrt_bc2 = 1.0 / math.sqrt(1.0 - b2 ** self.t)
        for item in self.dispatches:
            if item[0] == "fp32":
                _, p, g, m, v, n, decays = item
                self.backend.adamw_step(p, g, m, v, None, self.lr, lr_t, b1, b2, self.eps,
                                        self.weight_decay if decays else 0.0, numel=n, decay_numel=n if decays else 0,
                                        grad_scale=grad_scale, lr_bc1=lr_bc1, inv_sqrt_bc2=inv_sqrt_bc2)
            else:
                _, p, g, qm, qv, absmax_m, absmax_v, n, decays = item
                self.backend.adamw8bit_step(p, g, qm, qv, absmax_m, absmax_v, self.qmap_m, self.qmap_v, self.lr, lr_bc1,
                                            inv_sqrt_bc2, b1, b2, self.eps, self.weight_decay if decays else 0.0, n,
                                            n if decays else 0, first_step=(self.t == 1), grad_scale=grad_scale)

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
        if self.state_mode == "8bit":
            self._step_8bit(grad_scale)
            self.backend.end_pass()
            return
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
        if self.state_mode == "8bit":
            items = [(item[2], int(item[-2])) for item in self.dispatches]
        else:
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
