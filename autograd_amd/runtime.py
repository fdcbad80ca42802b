"""Graph compiler and executor for the layer-op path.

Counterpart of the reference's runtime.py for what this path needs:
topological order and gradient tensors (runtime.py:123-152), parameter slabs
(runtime.py:154-206), kernel binding (runtime.py:241-246), lifetime analysis and
the first-fit training arena (runtime.py:20-59, 272-513), and the execute /
zero_grad / forward / backward_graph loops (runtime.py:802-854).

The arena is ONE device allocation; every activation, activation gradient and
scratch block is a `(buffer_id, byte offset)` view into it, 256-byte aligned.

Gradient zeroing.  The reference's CPU path zero-fills a gradient right before
the first backward kernel that adds into it (runtime.py:844-854).  Here that
first writer is told to store instead (OpNode.overwrite_grads) whenever its
kernel writes the whole tensor, which removes one full write and one full read
of every activation gradient; the numbers are the same as accumulating onto
zeros.  `fuse_grad_zeroing=False` restores fill-then-accumulate.
"""
from __future__ import annotations

import functools
from math import prod

import numpy as np

from .device import Device
from .scratch import ScratchViews
from .tensor import Tensor
from .utils import align_up, is_bf16, itemsize

ARENA_ALIGN = 256


class MemoryPlanner:
    """First-fit placement of byte ranges with explicit alloc / free
    (runtime.py:20-59): a block goes to the lowest offset where it fits between
    the live blocks."""

    def __init__(self, align=ARENA_ALIGN):
        self.align = align
        self.live = {}      # key -> (offset, size)
        self.offsets = {}   # key -> offset, kept after free
        self.peak = 0

    def alloc(self, key, nbytes):
        if key in self.offsets:
            return self.offsets[key]
        size = align_up(max(int(nbytes), 1), self.align)
        cursor = 0
        for off, sz in sorted(self.live.values()):
            if cursor + size <= off:
                break
            cursor = max(cursor, off + sz)
        self.live[key] = (cursor, size)
        self.offsets[key] = cursor
        self.peak = max(self.peak, cursor + size)
        return cursor

    def free(self, key):
        self.live.pop(key, None)

    def get_offset(self, key):
        return self.offsets.get(key)


class _Scratch:
    """stand-in for a per-node scratch block in the lifetime table"""
    __slots__ = ("nbytes", "node", "phase")

    def __init__(self, nbytes, node, phase):
        self.nbytes, self.node, self.phase = nbytes, node, phase


class CapturedGraph:
    """a recorded sequence of launches; see Runtime.capture"""

    def __init__(self, backend, graph_id):
        self.backend, self.graph_id = backend, graph_id

    def launch(self):
        if self.graph_id is None:
            raise RuntimeError("graph was destroyed")
        self.backend.graph_launch(self.graph_id)

    def destroy(self):
        if self.graph_id is not None:
            self.backend.graph_destroy(self.graph_id)
            self.graph_id = None


class Runtime:
    _default_runtime = None

    @classmethod
    def get_default(cls):
        if cls._default_runtime is None:
            cls._default_runtime = Runtime()
        return cls._default_runtime

    def __init__(self, device="hip", forward_only=False, owns_params=True, use_fp16_gemm=False,
                 fuse_grad_zeroing=True, defer_param_grad_sums=True, row_reset=True):
        self.loss = None
        self.topo = []
        self.forward_only = forward_only
        self.owns_params = owns_params
        self.is_compiled = False
        self.unified_arena = None
        self.allocator = Device.get_allocator(device)
        self.backend = Device.get_backend(device)
        self.node_to_clear_grads = {}
        self.grad_scale = 1.0
        self.accumulate_parameter_grads = False
        self.use_fp16_gemm = use_fp16_gemm
        self.backend.use_fp16_gemm = use_fp16_gemm
        # only a backend whose kernels honour OpNode.overwrite_grads can skip the fills
        self.fuse_grad_zeroing = bool(fuse_grad_zeroing and getattr(self.backend, "supports_grad_store", False))
        # The column sums of parameter gradients (dgamma / dbeta of every norm, bias gradients)
        # end in a second, tiny launch that costs its launch floor -- a fifth of a norm backward
        # at 16384 x 384 -- and nothing reads a parameter gradient before the pass ends: with this
        # on, the backward kernels leave their partial rows in their scratch and ONE launch at
        # the end of backward_graph folds them all (same bits as folding each on its own).
        self.defer_param_grad_sums = bool(defer_param_grad_sums
                                          and getattr(self.backend, "supports_deferred_param_grads", False))
        # The gradient of an embedding table is zero outside the rows of the last pass's ids:
        # zero_grad clears those rows (N*C items) instead of filling the table (V*C items; 1 GB
        # at V = 151936, C = 1536 fp32, where the rows are 100 MB).  The forward kernel keeps the
        # copy of the ids that names them.
        self.row_reset = bool(row_reset and getattr(self.backend, "supports_row_reset", False))
        self.arena_bytes = 0
        self._owns_arena = False       # release() frees only an arena this runtime allocated
        self.memory_plan = None        # key -> arena offset, set by plan_memory()
        self._keyobj = {}
        self.leaves = []
        self.consumers = {}
        self._alias_of = {}            # output tensor -> input tensor it shares memory and gradient with
        self._view_of = {}             # output tensor -> input tensor whose memory it re-reads (layout ops)
        self._stored_leaf_grads = set()   # ids of leaf grads whose first writer stores the whole tensor
        self._slabs = []

    # -- entry points (runtime.py:89-121) ------------------------------------------
    def backward(self, loss, grad_scale=1.0, accumulate_parameter_grads=False):
        self.loss = loss
        self.grad_scale = float(grad_scale)
        self.accumulate_parameter_grads = bool(accumulate_parameter_grads)
        self.backend.accumulate_parameter_grads = self.accumulate_parameter_grads
        self.backend.grad_scale = self.grad_scale
        if not self.is_compiled:
            self.build_topo(loss)
            self.bind_memory()
            self.is_compiled = True
        self.execute()

    def run_forward(self, output, feeds=None, return_value=True):
        if not self.is_compiled:
            self.loss = output
            self.build_topo(output)
            self.bind_memory()
            self.is_compiled = True
        for tensor, host_value in (feeds or {}).items():
            self.backend.copy_from_host(tensor, host_value)
        self.forward()
        if not return_value:
            return None
        self.backend.synchronize()
        return self.backend.copy_to_host(output)

    # -- graph -------------------------------------------------------------------
    def build_topo(self, loss):
        self.loss = loss
        seen_nodes, seen_tensors = set(), set()
        self.topo, self.leaves = [], []

        def visit(tensor):
            node = tensor.op
            if node is None or id(node) in seen_nodes:
                return
            seen_nodes.add(id(node))
            for src in node.inputs:
                visit(src)
            for t in node.inputs + node.outputs:
                if id(t) in seen_tensors:
                    continue
                seen_tensors.add(id(t))
                if t.op is None:
                    self.leaves.append(t)
                if not self.forward_only and t.requires_grad and t.grad is None:
                    gdt = t.grad_dtype if t.op is None else t.dtype
                    t.grad = Tensor(shape=t.shape, dtype=gdt, requires_grad=False, device=t.device)
            self.topo.append(node)

        visit(loss)

        self.consumers = {}
        for node in self.topo:
            for t in node.inputs:
                self.consumers.setdefault(id(t), []).append(node)
        # an output nobody reads never receives a gradient
        for node in self.topo:
            for t in node.outputs:
                if t is not loss and id(t) not in self.consumers:
                    t.grad = None

        self._place_leaves()

        for node in self.topo:
            node.forward = self.backend.get_forward_kernel(node.op)
            node.backward = self.backend.get_backward_kernel(node.op)
            if node.forward is None or (node.backward is None and not self.forward_only):
                raise RuntimeError(f"device {self.allocator.device!r} has no kernel for {type(node.op).__name__}")
            fwd, bwd = self.backend.plan_scratch(node)
            node.scratch_fwd_layout, node.scratch_bwd_layout = fwd, (None if self.forward_only else bwd)
            node.defer_param_grads = bool(self.defer_param_grad_sums and node.scratch_bwd_layout is not None
                                          and self.backend.can_defer_param_grads(node))
            # an embedding whose table takes a gradient keeps a copy of each pass's ids outside
            # the arena: the rows to clear in that gradient before the next pass
            if self.row_reset and not self.forward_only and node.op.early_outputs and len(node.outputs) > 1 \
                    and node.inputs[1].grad is not None and node.kept_ids is None:
                node.kept_ids = self.allocator.alloc((prod(node.inputs[0].shape),), np.int32)
                self._slabs.append(node.kept_ids)

        self._resolve_aliases()

    def _place_leaves(self):
        """Parameters that need gradients are packed into one slab, their
        gradients into another (runtime.py:154-206); other leaves get their own
        allocation."""
        params = [t for t in self.leaves
                  if self.owns_params and not self.forward_only and t.requires_grad and t.grad is not None
                  and t.storage is None and hasattr(self.allocator, "ctx")]
        if params:
            order = [t for t in params if t.ndim > 1] + [t for t in params if t.ndim <= 1]
            poff, goff, pcur, gcur = {}, {}, 0, 0
            for t in order:
                pcur = align_up(pcur, ARENA_ALIGN)
                poff[id(t)] = pcur
                pcur += prod(t.shape) * itemsize(t.dtype)
                gcur = align_up(gcur, ARENA_ALIGN)
                goff[id(t)] = gcur
                gcur += prod(t.shape) * itemsize(t.grad.dtype)
            pslab = self.allocator.empty((align_up(pcur, ARENA_ALIGN),), np.uint8)
            gslab = self.allocator.empty((align_up(gcur, ARENA_ALIGN),), np.uint8)
            self.backend.fill_storage2(pslab, 0)
            self.backend.fill_storage2(gslab, 0)
            self._slabs += [pslab, gslab]
            for t in order:
                t.storage = self.allocator.view(pslab, poff[id(t)], t.shape, t.dtype)
                t.grad.storage = self.allocator.view(gslab, goff[id(t)], t.shape, t.grad.dtype)
                self.backend.init(t)
        for t in self.leaves:
            if t.requires_grad and not self.owns_params:
                if t.storage is None or (not self.forward_only and t.grad.storage is None):
                    raise RuntimeError(f"shared parameter {t.name} has no storage")
                continue
            if t.storage is None:
                t.storage = self.allocator.alloc(t.shape, t.dtype)
                self.backend.init(t)
            if not self.forward_only and t.grad is not None and t.grad.storage is None:
                t.grad.storage = self.allocator.alloc(t.grad.shape, t.grad.dtype)
                self.backend.fill_storage2(t.grad.storage, 0)

    def _resolve_aliases(self):
        """In-place ops: an output shares its input's memory when the input is
        an activation nobody else reads; otherwise the backend copies first."""
        self._alias_of = {}
        self._view_of = {}
        for node in self.topo:
            if node.op.view_of_input is not None:
                self._view_of[id(node.outputs[0])] = node.inputs[node.op.view_of_input]
        for node in self.topo:
            for out_i, in_i in node.op.inplace_aliases.items():
                src, dst = node.inputs[in_i], node.outputs[out_i]
                # a view's memory belongs to its base, which others may still read
                if src.op is None or len(self.consumers.get(id(src), [])) != 1 or src is self.loss \
                        or id(src) in self._view_of:
                    continue
                # The only other reader a single-consumer activation can have is its own
                # producer's backward kernel (Exp, Rsqrt and Softmax keep their OUTPUT):
                # overwriting it in place would feed that kernel the rotated values.
                made_by = src.op
                if not self.forward_only and any(t is src for t in
                                                 made_by.op.save_for_backward(made_by.inputs, made_by.outputs)):
                    continue
                self._alias_of[id(dst)] = src

    def _root(self, t):
        """the tensor whose memory `t` lives in (views: same memory, own gradient)"""
        while True:
            if id(t) in self._alias_of:
                t = self._alias_of[id(t)]
            elif id(t) in self._view_of:
                t = self._view_of[id(t)]
            else:
                return t

    def _grad_root(self, t):
        """the tensor whose gradient memory `t`'s gradient lives in"""
        while id(t) in self._alias_of:
            t = self._alias_of[id(t)]
        return t

    # -- memory ------------------------------------------------------------------
    def bind_memory(self):
        """plan the arena, allocate it and bind every view (runtime.py:272-513)"""
        self.plan_memory(force=True)
        if self.arena_bytes == 0:
            self.unified_arena = None
            return
        print(f"Training arena need {self.arena_bytes}")
        self.unified_arena = self.allocator.empty((self.arena_bytes,), np.uint8)
        self._owns_arena = True
        print(f"[ARENA-TRAIN-ALLOC] bytes={self.arena_bytes} "
              f"buffer_id={getattr(self.unified_arena.ptr, 'buffer_id', None)}", flush=True)
        self._bind_views()

    def plan_memory(self, force=False):
        """lifetimes -> first-fit offsets in one arena; allocates nothing
        (runtime.py:515-716).  Sets arena_bytes and returns {key: offset}."""
        if self.memory_plan is not None and not force:
            return self.memory_plan
        n = len(self.topo)
        steps = [(0, node) for node in self.topo]
        if not self.forward_only:
            steps += [(1, node) for node in reversed(self.topo)]

        # who zero-fills / first-writes which gradient (runtime.py:272-284)
        self.node_to_clear_grads = {id(node): [] for node in self.topo}
        self._stored_leaf_grads = set()
        if not self.forward_only:
            touched = set()
            for node in reversed(self.topo):
                overwrite = set()
                full = {node.inputs[i] for i in node.op.fully_written_inputs(node.inputs, node.outputs)}
                aliased_inputs = {id(self._alias_of[id(o)]) for o in node.outputs
                                  if id(o) in self._alias_of and o.grad is not None}
                for x in node.inputs:
                    if not x.requires_grad or x.grad is None or id(x) in touched:
                        continue
                    touched.add(id(x))
                    if id(x) in aliased_inputs:
                        continue          # its gradient is the output's gradient, rotated in place
                    storable = (self.fuse_grad_zeroing and any(x is f for f in full)
                                and sum(1 for t in node.inputs if t is x) == 1)
                    if storable:
                        overwrite.add(id(x.grad))
                        if x.op is None:
                            self._stored_leaf_grads.add(id(x.grad))
                    elif x.op is not None:
                        self.node_to_clear_grads[id(node)].append(x)
                # Most kernels have ONE store-or-accumulate choice for their parameter gradients
                # (gamma and beta of a norm share a flag bit; Op.shared_param_grad_flag).  If only some of this node's
                # leaf gradients are first written here -- a gamma tied to a later node, a
                # beta of its own -- none of them may skip the zero fill, or the kernel
                # would accumulate onto memory nobody cleared.
                leaf_grads = {id(x.grad) for x in node.inputs
                              if x.op is None and x.requires_grad and x.grad is not None}
                if node.op.shared_param_grad_flag and leaf_grads - overwrite:
                    overwrite -= leaf_grads
                    self._stored_leaf_grads -= leaf_grads
                node.overwrite_grads = frozenset(overwrite)

        life = {}       # key object -> [first step, last step]
        keyobj = {}

        def touch(obj, step):
            k = id(obj)
            keyobj[k] = obj
            if k in life:
                life[k][0] = min(life[k][0], step)
                life[k][1] = max(life[k][1], step)
            else:
                life[k] = [step, step]

        for step, (phase, node) in enumerate(steps):
            if phase == 0:
                for t in node.inputs + node.outputs:
                    if self._root(t).op is not None:     # leaves (and views of leaves) live outside the arena
                        touch(self._root(t), step)
                if node.scratch_fwd_layout is not None:
                    touch(_Scratch(node.scratch_fwd_layout.nbytes, node, 0), step)
                for i in node.op.early_outputs:
                    if i < len(node.outputs):
                        touch(self._root(node.outputs[i]), 0)      # may be written before the first node runs
            else:
                for t in node.op.save_for_backward(node.inputs, node.outputs):
                    if self._root(t).op is not None:
                        touch(self._root(t), step)
                for t in node.inputs + node.outputs:
                    if t.grad is not None and t.op is not None:
                        g = self._grad_root(t).grad
                        touch(g if g is not None else t.grad, step)
                if node.scratch_bwd_layout is not None:
                    block = _Scratch(node.scratch_bwd_layout.nbytes, node, 1)
                    touch(block, step)
                    if node.defer_param_grads:
                        touch(block, len(steps) - 1)     # its partial rows wait for the fold that ends the pass
        if self.loss is not None and self.loss.op is not None:
            touch(self._root(self.loss), len(steps))
            if self.loss.grad is not None:
                # written by fill() between the forward and the backward loops
                touch(self._grad_root(self.loss).grad or self.loss.grad, n - 1 if n else 0)

        planner = MemoryPlanner()
        order = sorted(life.items(), key=lambda kv: kv[1][0])
        by_start, by_end = {}, {}
        for k, (a, b) in order:
            by_start.setdefault(a, []).append(k)
            by_end.setdefault(b, []).append(k)
        last = max((b for _, (_, b) in order), default=-1)
        for step in range(last + 1):
            for k in by_end.get(step - 1, []):
                planner.free(k)
            for k in by_start.get(step, []):
                obj = keyobj[k]
                nbytes = obj.nbytes if isinstance(obj, _Scratch) else prod(obj.shape) * itemsize(obj.dtype)
                planner.alloc(k, nbytes)

        self.arena_bytes = planner.peak
        self.memory_plan = {k: planner.get_offset(k) for k in life}
        self._keyobj = keyobj
        return self.memory_plan

    def bind_memory_new(self, arena=None):
        """bind every planned view into `arena` (allocated here when None): several
        runtimes -- a training plan and an inference plan over the same parameters --
        can live in one arena sized for the largest (runtime.py:718-732)"""
        self.plan_memory()
        self._owns_arena = False
        if arena is None and self.arena_bytes:
            arena = self.allocator.empty((self.arena_bytes,), np.uint8)
            self._owns_arena = True
            print(f"[ARENA-ALLOC] bytes={arena.nbytes} buffer_id={getattr(arena.ptr, 'buffer_id', None)}", flush=True)
        if self.arena_bytes and arena.nbytes < self.arena_bytes:
            raise RuntimeError(f"arena too small: need={self.arena_bytes}, have={arena.nbytes}")
        self.unified_arena = arena
        self._bind_views()

    def _bind_views(self):
        arena = self.unified_arena
        for k, obj in self._keyobj.items():
            off = self.memory_plan[k]
            if isinstance(obj, _Scratch):
                node = obj.node
                layout = node.scratch_fwd_layout if obj.phase == 0 else node.scratch_bwd_layout
                block = self.allocator.view(arena, off, (obj.nbytes,), np.uint8)
                views = ScratchViews({name: self.allocator.view(block, o, shape, dt)
                                      for name, (o, shape, dt) in layout.slots.items()})
                if obj.phase == 0:
                    base = getattr(node.forward, "func", node.forward)
                    node.forward = functools.partial(base, scratch=views)
                else:
                    base = getattr(node.backward, "func", node.backward)
                    node.backward = functools.partial(base, scratch=views)
            else:
                obj.storage = self.allocator.view(arena, off, obj.shape, obj.dtype)
        # in topological order, so that chains resolve: in-place outputs (and their
        # gradients) share their input's views; layout ops re-view their input's memory
        for node in self.topo:
            for t in node.outputs:
                if id(t) in self._alias_of:
                    src = self._alias_of[id(t)]
                    t.storage = src.storage
                    if t.grad is not None and src.grad is not None:
                        t.grad.storage = src.grad.storage
                    elif t.grad is not None and src.grad is None:
                        raise RuntimeError("aliased output needs a gradient but its input has none")
                elif id(t) in self._view_of:
                    base = self._view_of[id(t)]
                    t.storage = self.allocator.view(base.storage, 0, t.shape, t.dtype)
        for node in self.topo:
            for t in node.outputs:
                if t.init_val is not None:
                    self.backend.init(t)

    # -- execution (runtime.py:802-854) ---------------------------------------------
    def execute(self, wait=True):
        """zero_grad + forward + backward.  wait=False (backends that run a step as one pass)
        returns once the step is queued: the stream is in order, so the next step, an optimizer
        step or a read-back (which waits by itself) may follow at once, and an index error of this
        step is raised at the next call that waits.  A step's wait leaves the GPU idle while the
        host queues the first kernels of the next: a tenth of a 0.2 ms step."""
        if self.forward_only:
            self.forward()
            return
        if getattr(self.backend, "single_pass_execute", False):
            # one pass, one wait at its end, as the reference runs its GPU device
            # (runtime.py:818-826): a pass boundary drains the GPU, and two of them per
            # step (forward, then backward) are a tenth of a small step
            self._require_bound()
            self._sync_backend()
            self.backend.begin_pass()
            if not self.accumulate_parameter_grads:
                self.zero_grad()
            self._forward_nodes()
            self.backend.fill(self.loss.grad, self.grad_scale)
            self._backward_nodes()
            if wait:
                self.backend.end_pass()
            return
        if not self.accumulate_parameter_grads:
            self.zero_grad()
        self.forward()
        self.backend.fill(self.loss.grad, self.grad_scale)
        self.backward_graph()

    def _sync_backend(self):
        """the backend is one object per device, shared by every Runtime: before this
        runtime launches anything it puts its own settings there"""
        self.backend.accumulate_parameter_grads = self.accumulate_parameter_grads
        self.backend.grad_scale = self.grad_scale
        self.backend.use_fp16_gemm = self.use_fp16_gemm

    def zero_grad(self, order_ids=False):
        """zero the parameter gradients, except those whose first backward kernel
        stores the whole tensor anyway.  order_ids: the zero fill of an embedding table's
        gradient also orders that embedding's ids for the backward pass, in the same launch,
        and the node's next forward kernel is the plain gather -- the caller vouches that the
        ids are already what that forward pass will read.  Off by default, because it does not
        pay on this GPU: the fill runs best with few waves on a CU, and with the 512-thread ordering
        workgroups in its grid it takes 3 us (a 50 MB table) to 25 us (1 GB) longer, where they cost
        the forward gather, whose grid they ride in otherwise, 1 to 3 us."""
        self._sync_backend()
        seen = set()
        for node in self.topo:
            for t in node.inputs + node.outputs:
                if id(t) in seen:
                    continue
                seen.add(id(t))
                if t.grad is not None and t.op is None:
                    if id(t.grad) in self._stored_leaf_grads and not self.accumulate_parameter_grads:
                        continue
                    if order_ids and node.op.early_outputs and len(node.inputs) > 1 and node.inputs[1] is t \
                            and hasattr(self.backend, "zero_grad_and_order") and self.backend.zero_grad_and_order(node, t):
                        continue
                    if self.row_reset and t.grad.dirty_rows is not None:
                        self.backend.clear_table_grad(t)
                    else:
                        self.backend.fill(t.grad, 0)

    def _require_bound(self):
        if self.memory_plan is not None and self.arena_bytes and self.unified_arena is None:
            raise RuntimeError("this runtime's memory is planned but not bound: call bind_memory_new / bind_to first")

    def _forward_nodes(self):
        for node in self.topo:
            node.forward(node.inputs, node.outputs)

    def _backward_nodes(self):
        for node in reversed(self.topo):
            for t in self.node_to_clear_grads.get(id(node), ()):
                if t.grad is not None:
                    self.backend.fill(t.grad, 0)
            node.backward(node.inputs, node.outputs)
        if self.defer_param_grad_sums:
            self.backend.finalize_param_grads()

    def forward(self):
        self._require_bound()
        self._sync_backend()
        self.backend.begin_pass()
        self._forward_nodes()
        self.backend.end_pass()

    def backward_graph(self):
        self._require_bound()
        self._sync_backend()
        self.backend.begin_pass()
        self._backward_nodes()
        self.backend.end_pass()

    def capture(self, fn):
        """Record everything `fn()` launches (for example `rt.execute`) into a device
        graph and return a CapturedGraph; `graph.launch()` replays it as one
        submission, which removes the per-launch cost that dominates chains of small
        ops.  `fn` must already have run once eagerly (kernels load on first use), may
        not read results back, and the replay uses the tensors as they are bound now.
        Choices the host made while recording are part of the recording: a recorded
        zero_grad that cleared an embedding table's gradient by rows (row_reset) clears
        the rows of the ids of the pass before it on every replay, which is right as
        long as the replays and nothing else write that gradient between them -- write
        it from the host or from another runtime and the next step must run eagerly
        (or be recorded again).
        Requires a backend with capture_begin / capture_end (the "hip" device)."""
        if not hasattr(self.backend, "capture_begin"):
            raise RuntimeError(f"device {self.allocator.device!r} cannot record graphs")
        self.backend.capture_begin()
        try:
            fn()
        except BaseException:
            try:
                self.backend.capture_end()
            except Exception:
                pass
            raise
        return CapturedGraph(self.backend, self.backend.capture_end())

    def release(self):
        """return the arena and the parameter slabs to the device"""
        rel = getattr(self.allocator, "release", None)
        if rel is None:
            return
        self.backend.synchronize()
        if self.unified_arena is not None and self._owns_arena:
            rel(self.unified_arena)
        self.unified_arena = None
        self._owns_arena = False
        for slab in self._slabs:
            rel(slab)
        self._slabs = []
        # the kept-id buffers were among the slabs: nothing may name them any more
        for node in self.topo:
            if node.kept_ids is not None:
                node.kept_ids = None
                node.kept_fresh = False
                if len(node.inputs) > 1 and node.inputs[1].grad is not None:
                    node.inputs[1].grad.dirty_rows = None


# -- execution plans (runtime.py:857-947) -------------------------------------------
class ExecutionPlan:
    """A compiled graph with named feed tensors.  Several plans -- a training step
    and forward-only plans at other sequence lengths -- are prepared separately,
    then bound into ONE arena sized for the largest (`bind_plans`), the way the
    reference's engine shares its training arena with the decode plans
    (engine.py:133-170).  Method names are the reference's."""

    def __init__(self, runtime, input_ids, output, target_ids=None, row_scale=None, seq_len=0, mode="train"):
        self.runtime = runtime
        self.input_ids = input_ids
        self.target_ids = target_ids
        self.row_scale = row_scale
        self.output = output
        self.seq_len = seq_len
        self.mode = mode

    def prepare(self):
        rt = self.runtime
        rt.loss = self.output
        rt.build_topo(self.output)
        rt.plan_memory(force=True)
        rt.is_compiled = True
        return self

    def bind_to(self, arena):
        self.runtime.bind_memory_new(arena)

    def _feed(self, tensor, values, what):
        if tensor is None:
            raise ValueError(f"this plan has no {what}")
        self.runtime.backend.copy_from_host(tensor, values)

    def set_inputs(self, values):
        self._feed(self.input_ids, values, "input tensor")

    def set_targets(self, values):
        self._feed(self.target_ids, values, "target tensor")

    def set_row_scale(self, values):
        self._feed(self.row_scale, values, "row scale tensor")

    def forward(self, feeds=None, return_value=True):
        return self.runtime.run_forward(self.output, feeds=feeds, return_value=return_value)

    def backward(self, grad_scale=1.0, accumulate_parameter_grads=False):
        if self.runtime.forward_only:
            raise ValueError("inference plan cannot use backward()")
        self.runtime.backward(self.output, grad_scale=grad_scale,
                              accumulate_parameter_grads=accumulate_parameter_grads)


def bind_plans(plans, arena=None):
    """bind prepared plans into one arena (allocated with the first plan's allocator
    when None) big enough for the largest; returns the arena.  The plans then
    overwrite each other's activations: run one at a time."""
    plans = list(plans)
    need = max((p.runtime.arena_bytes for p in plans), default=0)
    if arena is None and need:
        arena = plans[0].runtime.allocator.empty((need,), np.uint8)
    if need and arena.nbytes < need:
        raise RuntimeError(f"arena too small: need={need}, have={arena.nbytes}")
    for p in plans:
        p.bind_to(arena)
    return arena
