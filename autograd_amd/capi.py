"""ctypes binding of the C ABI in include/autograd_hip.h.

The Python host layer (backend.py) reaches the library through the pybind11
module `hip_ext`, the way the reference reaches Metal through `metal_ext`.  This
module binds the same shared library with ctypes instead: it is what a caller
without pybind11 would write, and what the tests and the benchmark use to drive
the typed entry points with raw device addresses.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import numpy as np

LIB_PATH = Path(__file__).resolve().parent / "libautograd_hip.so"

F32, BF16 = 0, 1
NORM_LAYER, NORM_RMS = 0, 1
ACC_INPUT_GRAD, ACC_PARAM_GRAD, ACC_INPUT_GRAD2, ACC_PARAM_GRAD2, PARAM_GRAD_BF16, DEFER_PARAM_GRAD = 1, 2, 4, 8, 16, 32
UNARY_EXP, UNARY_LOG, UNARY_RSQRT = 0, 1, 2
MUL_SAME, MUL_ROW, MUL_COL, MUL_SCALAR = 0, 1, 2, 3
OK, EINVAL, EHIP, ENOKERNEL, EINDEX, EWORKSPACE = 0, -1, -2, -3, -4, -5
NOALLOC_SCRATCH_BYTES = 32 << 20

class ColsumJob(C.Structure):
    """agrad_colsum_job: one column sum that is still to be folded"""
    _fields_ = [("partial_a", C.c_void_p), ("partial_b", C.c_void_p), ("out_a", C.c_void_p), ("out_b", C.c_void_p),
                ("partial_rows", C.c_uint32), ("C", C.c_uint32), ("flags", C.c_uint32), ("reserved", C.c_uint32)]


_ctx = C.c_void_p
_ptr = C.c_void_p
_u64 = C.c_uint64
_u32 = C.c_uint32
_int = C.c_int
_f32 = C.c_float

# name -> (restype, argtypes); one entry per declaration in the header
SIGNATURES = {
    "agrad_last_error": (C.c_char_p, []),
    "agrad_device_count": (_int, [C.POINTER(_int)]),
    "agrad_ctx_create": (_int, [_int, C.POINTER(_ctx)]),
    "agrad_ctx_destroy": (_int, [_ctx]),
    "agrad_max_buffer_length": (_int, [_ctx, C.POINTER(_u64)]),
    "agrad_alloc": (_int, [_ctx, _u64, C.POINTER(_u64)]),
    "agrad_free": (_int, [_ctx, _u64]),
    "agrad_begin_pass": (_int, [_ctx]),
    "agrad_end_pass": (_int, [_ctx]),
    "agrad_synchronize": (_int, [_ctx]),
    "agrad_copy_from_host": (_int, [_ctx, _u64, _u64, _ptr, _u64]),
    "agrad_copy_to_host": (_int, [_ctx, _u64, _u64, _ptr, _u64]),
    "agrad_fill": (_int, [_ctx, _u64, _u64, _u32, _int, _u64]),
    "agrad_stream": (_int, [_ctx, C.POINTER(_ptr)]),
    "agrad_timer_start": (_int, [_ctx]),
    "agrad_timer_stop": (_int, [_ctx, C.POINTER(_f32)]),
    "agrad_dispatch": (_int, [_ctx, C.c_char_p, C.POINTER(_u64), C.POINTER(_u64), _int,
                              C.POINTER(_u32), _int, _u64, _u64, _u64, _u64]),
    "agrad_kernel_count": (_int, []),
    "agrad_kernel_name": (C.c_char_p, [_int]),
    "agrad_kernel_signature": (C.c_char_p, [C.c_char_p]),
    "agrad_add_forward": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _u64]),
    "agrad_grad_accumulate": (_int, [_ctx, _int, _ptr, _ptr, _u64, _u32]),
    "agrad_cast_f32_to_bf16": (_int, [_ctx, _ptr, _ptr, _u64, _int]),
    "agrad_cast_bf16_to_f32": (_int, [_ctx, _ptr, _ptr, _u64]),
    "agrad_copy": (_int, [_ctx, _ptr, _ptr, _u64]),
    "agrad_norm_forward": (_int, [_ctx, _int, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _u64, _u32, _f32]),
    "agrad_norm_backward_workspace_bytes": (_u64, [_u64, _u32, _int]),
    "agrad_norm_backward": (_int, [_ctx, _int, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr,
                                   _ptr, _u64, _u64, _u32, _f32, _u32]),
    "agrad_norm_backward_noalloc": (_int, [_ctx, _int, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr,
                                           _u64, _u32, _f32, _u32]),
    "agrad_pending_param_grads": (_int, [_ctx, C.POINTER(_u32)]),
    "agrad_finalize_param_grads": (_int, [_ctx]),
    "agrad_colsum_finalize_many": (_int, [_ctx, _ptr, _u32]),
    "agrad_norm_backward_partial": (_int, [_ctx, _int, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr,
                                           _ptr, _u64, _u64, _u32, _f32, _u32, _ptr]),
    "agrad_gelu_forward": (_int, [_ctx, _int, _ptr, _ptr, _u64]),
    "agrad_gelu_backward": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _u64, _u32]),
    "agrad_gelu_bias_forward": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _u64, _u32]),
    "agrad_gelu_bias_backward_workspace_bytes": (_u64, [_u64, _u32]),
    "agrad_gelu_bias_backward": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _u64, _u64, _u32, _u32]),
    "agrad_relu2_forward": (_int, [_ctx, _int, _ptr, _ptr, _u64]),
    "agrad_relu2_backward": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _u64, _u32]),
    "agrad_swiglu_forward": (_int, [_ctx, _int, _ptr, _ptr, _u64, _u32]),
    "agrad_swiglu_forward_tile": (_int, [_ctx, _int, _ptr, _ptr, _u64, _u32, _u32, _u32]),
    "agrad_swiglu_backward": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _u64, _u32, _u32]),
    "agrad_rope_qk": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _u32, _int, _int]),
    "agrad_rope_qk_bhtd": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _u32, _int, _int]),
    "agrad_gather_forward": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _ptr, _u64, _u32, _u32, _u32]),
    "agrad_embedding_backward_workspace_bytes": (_u64, [_u64, _u32, _u32, _int]),
    "agrad_embedding_backward": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _ptr, _u64, _u64, _u32, _u32, _u32]),
    "agrad_embedding_sort_workspace_bytes": (_u64, [_u64, _u32]),
    "agrad_gather_forward_sorted": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _ptr, _u64, _u32, _u32, _u32, _ptr, _ptr, _u64]),
    "agrad_gather_forward_sorted_kept": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _ptr, _u64, _u32, _u32, _u32, _ptr, _ptr, _u64, _ptr]),
    "agrad_set_team_wait_polls": (_int, [_ctx, _u32]),
    "agrad_embedding_order": (_int, [_ctx, _ptr, _u64, _u32, _ptr, _ptr, _u64, _ptr, _u64]),
    "agrad_embedding_grad_reset": (_int, [_ctx, _int, _ptr, _u64, _ptr, _u32, _u32]),
    "agrad_unary_forward": (_int, [_ctx, _int, _int, _ptr, _ptr, _u64]),
    "agrad_unary_backward": (_int, [_ctx, _int, _int, _ptr, _ptr, _ptr, _u64, _u32]),
    "agrad_mul_forward": (_int, [_ctx, _int, _int, _ptr, _ptr, _ptr, _u64, _u64]),
    "agrad_mul_backward_workspace_bytes": (_u64, [_int, _u64, _u64]),
    "agrad_mul_backward": (_int, [_ctx, _int, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _u64, _u64, _u64, _u32]),
    "agrad_softmax_forward": (_int, [_ctx, _int, _ptr, _ptr, _u64, _u32]),
    "agrad_softmax_backward": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _u64, _u32, _u32]),
    "agrad_strided_copy": (_int, [_ctx, _int, _ptr, _ptr, _int, _ptr, _ptr, _u32]),
    "agrad_embedding_backward_sorted_workspace_bytes": (_u64, [_u64, _u32]),
    "agrad_embedding_backward_sorted": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _u64, _u64, _u32, _u32, _u32, _u32]),
    "agrad_pos_embedding_backward": (_int, [_ctx, _int, _ptr, _ptr, _u32, _u32, _u32, _u32]),
    "agrad_graph_begin": (_int, [_ctx]),
    "agrad_graph_end": (_int, [_ctx, C.POINTER(_u64)]),
    "agrad_graph_launch": (_int, [_ctx, _u64]),
    "agrad_graph_destroy": (_int, [_ctx, _u64]),
    "agrad_broadcast_add_forward": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _u64, _u64]),
    "agrad_broadcast_grad_workspace_bytes": (_u64, [_u64, _u64]),
    "agrad_broadcast_add_backward": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _u64, _u64, _u64, _u32]),
    "agrad_cross_entropy_forward": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _ptr, _u64, _u32]),
    "agrad_cross_entropy_backward": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _u64, _u32, _u32]),
    "agrad_cross_entropy_fused": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _u64, _u32, _u64, _f32, _u32]),
    "agrad_adamw8bit_step": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _u64, _u64,
                                    _f32, _f32, _f32, _f32, _f32, _f32, _f32, _int]),
    "agrad_adamw_step": (_int, [_ctx, _int, _ptr, _ptr, _ptr, _ptr, _u64, _u64] + [_f32] * 9),
    "agrad_grad_norm_groups": (_u64, [_u64]),
    "agrad_grad_norm_sq": (_int, [_ctx, _int, _ptr, _ptr, _u64]),
}


class AgradError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(message)
        self.code = code


def load_library(path: Path | str = LIB_PATH) -> C.CDLL:
    path = Path(path)
    if not path.exists():
        raise RuntimeError(f"{path} is missing: build it with `python -m autograd_amd.build`")
    lib = C.CDLL(str(path))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


class Context:
    """Owns an agrad_ctx; `call(name, *args)` raises on a non-zero status."""

    def __init__(self, device: int = 0, lib: C.CDLL | None = None):
        self.lib = lib or load_library()
        handle = _ctx()
        self._check(self.lib.agrad_ctx_create(device, C.byref(handle)))
        self.handle = handle

    def _check(self, rc: int) -> None:
        if rc != OK:
            msg = self.lib.agrad_last_error().decode()
            if rc == EINDEX:
                raise IndexError(msg)
            raise AgradError(rc, msg)

    def call(self, name: str, *args):
        self._check(getattr(self.lib, name)(self.handle, *args))

    def close(self) -> None:
        if self.handle:
            self.lib.agrad_ctx_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- memory ---------------------------------------------------------------
    def alloc(self, nbytes: int) -> int:
        out = _u64()
        self.call("agrad_alloc", int(nbytes), C.byref(out))
        return out.value

    def free(self, buffer_id: int) -> None:
        self.call("agrad_free", buffer_id)

    def upload(self, array: np.ndarray) -> "DeviceArray":
        a = np.ascontiguousarray(array)
        d = DeviceArray(self, a.shape, a.dtype)
        if a.nbytes:
            self.call("agrad_copy_from_host", d.buffer_id, 0, a.ctypes.data_as(_ptr), a.nbytes)
        return d

    def empty(self, shape, dtype) -> "DeviceArray":
        return DeviceArray(self, shape, dtype)

    def zeros(self, shape, dtype) -> "DeviceArray":
        d = DeviceArray(self, shape, dtype)
        if d.nbytes:
            self.call("agrad_fill", d.buffer_id, 0, 0, 1, d.nbytes)
        return d

    def synchronize(self) -> None:
        self.call("agrad_synchronize")

    def timer_start(self) -> None:
        self.call("agrad_timer_start")

    def timer_stop(self) -> float:
        ms = _f32()
        self.call("agrad_timer_stop", C.byref(ms))
        return ms.value


class DeviceArray:
    """A typed view of one device allocation (bf16 travels as uint16)."""

    def __init__(self, ctx: Context, shape, dtype):
        self.ctx = ctx
        self.shape = tuple(int(s) for s in np.atleast_1d(shape)) if not isinstance(shape, tuple) else shape
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        self.buffer_id = ctx.alloc(max(self.nbytes, 1))

    @property
    def ptr(self) -> int:
        return self.buffer_id

    def at(self, byte_offset: int) -> int:
        return self.buffer_id + int(byte_offset)

    def download(self) -> np.ndarray:
        out = np.empty(self.shape, dtype=self.dtype)
        if self.nbytes:
            self.ctx.call("agrad_copy_to_host", self.buffer_id, 0, out.ctypes.data_as(_ptr), self.nbytes)
        return out

    def free(self) -> None:
        if self.buffer_id:
            self.ctx.free(self.buffer_id)
            self.buffer_id = 0
