"""Small host-side helpers shared by the graph IR, the runtime and the backend.

Counterpart of the reference's utils.py for the parts the layer-op path uses:
strides and broadcasting (utils.py:29-66), float bit patterns and the bf16
rounding rule (utils.py:14-27), Xavier init (utils.py:68-71).
"""
from __future__ import annotations

import struct
from math import prod

import numpy as np

BF16 = "bf16"   # dtype tag of bfloat16 tensors; their storage is np.uint16 bits


def is_bf16(dtype) -> bool:
    return isinstance(dtype, str) and dtype.lower() in ("bf16", "bfloat16")


def storage_dtype(dtype) -> np.dtype:
    """numpy dtype of the bytes that back a tensor of `dtype`."""
    return np.dtype(np.uint16) if is_bf16(dtype) else np.dtype(dtype)


def itemsize(dtype) -> int:
    return storage_dtype(dtype).itemsize


def nbytes_of(shape, dtype) -> int:
    return prod(shape) * itemsize(dtype)


def contiguous_strides(shape):
    strides, acc = [], 1
    for extent in reversed(tuple(shape)):
        strides.append(acc)
        acc *= extent
    return tuple(reversed(strides))


def broadcast_shape(a, b):
    out = []
    for i in range(1, max(len(a), len(b)) + 1):
        da = a[-i] if i <= len(a) else 1
        db = b[-i] if i <= len(b) else 1
        if da != db and 1 not in (da, db):
            raise RuntimeError(f"broadcast mismatch: {a} {b}")
        out.append(max(da, db) if 0 not in (da, db) else 0)
    return tuple(reversed(out))


def mul_bcast_kind(x_shape, y_shape) -> str:
    """how y is broadcast against x in x * y: 'scalar', 'row' ([C] against [..., C]),
    'col' ([..., 1] against [..., C]) or 'same' (utils.py:134-143)"""
    x_shape, y_shape = tuple(x_shape), tuple(y_shape)
    if len(y_shape) == 0 or prod(y_shape) == 1:
        return "scalar"
    if len(y_shape) == 1 and x_shape[-1] == y_shape[0]:
        return "row"
    if len(y_shape) == len(x_shape) and y_shape[:-1] == x_shape[:-1] and y_shape[-1] == 1:
        return "col"
    if y_shape == x_shape:
        return "same"
    raise RuntimeError(f"Mul backward: unsupported broadcast x={x_shape} y={y_shape}")


def f32_bits(x) -> int:
    return struct.unpack("<I", struct.pack("<f", float(x)))[0]


def bf16_bits(x) -> int:
    """fp32 -> bf16 bits: round to nearest even, Inf kept, NaN quieted."""
    bits = f32_bits(x)
    if bits & 0x7F800000 == 0x7F800000:
        return ((bits >> 16) | (0x0040 if bits & 0x007FFFFF else 0)) & 0xFFFF
    return ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) & 0xFFFF


def f32_array_to_bf16_bits(a) -> np.ndarray:
    bits = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    rounded = (bits + np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    special = (bits & np.uint32(0x7F800000)) == np.uint32(0x7F800000)
    quiet = np.where((bits & np.uint32(0x007FFFFF)) != 0, np.uint32(0x0040), np.uint32(0))
    return np.where(special, (bits >> np.uint32(16)) | quiet, rounded).astype(np.uint16)


def bf16_bits_to_f32_array(b) -> np.ndarray:
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def xavier_uniform(shape, dtype):
    fan_in, fan_out = shape[-2], shape[-1]
    std = np.sqrt(2.0 / (fan_in + fan_out))
    return np.random.normal(0, std, shape).astype(dtype)


def align_up(value: int, align: int) -> int:
    return (value + align - 1) // align * align
