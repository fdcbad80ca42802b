"""Strided gather into a dense tensor (agrad_strided_copy) against the CPU
restatement, through the C ABI: Contiguous forward of permuted / transposed views
and the Permute / Transpose gradients (backend.py:286-313).  A layout change moves
bits, so every comparison is bit-exact; the accumulating mode is one fp32 add per
element (rounded once for bf16 storage) and is bit-exact as well.

The cases cover both kernels and both widths of each: rows (source contiguous
along the innermost dimension) with 16-byte vectors and element-wise, tiles (a
true transpose through LDS) with 16-byte vectors and element-wise, ragged tile
edges, merged and extent-1 dimensions, broadcast (stride 0), and a source without
any unit-stride dimension.
"""
import ctypes as C

import numpy as np
import pytest

from autograd_amd import capi
from autograd_amd.utils import contiguous_strides
from oracle import cpu_ops as ref
from tests.helpers import from_bf16_bits, to_bf16_bits

pytestmark = pytest.mark.gpu
SEED = 1333


def _run(ctx, flat, shape, strides, dtype, flags=0, init=None):
    dt = capi.BF16 if dtype == "bf16" else capi.F32
    n = int(np.prod(shape)) if len(shape) else 1
    src = ctx.upload(flat)
    dst = ctx.upload(init) if init is not None else ctx.upload(np.full(max(n, 1), 0x7B, flat.dtype))
    sh = (C.c_uint32 * max(len(shape), 1))(*shape)
    st = (C.c_uint64 * max(len(strides), 1))(*strides)
    ctx.call("agrad_strided_copy", dt, C.c_void_p(src.ptr), C.c_void_p(dst.ptr), len(shape), sh, st, flags)
    ctx.synchronize()
    got = dst.download()
    src.free()
    dst.free()
    return got.reshape(-1)[:n].reshape(shape)


def _permuted(shape, dims):
    """(view shape, view strides) of a dense tensor of `shape` under permute(dims)"""
    base = contiguous_strides(shape)
    return tuple(shape[d] for d in dims), tuple(base[d] for d in dims)


PERMS = [
    # dense shape, permutation
    ((4, 16, 6, 64), (0, 2, 1, 3)),       # BTHD -> BHTD: rows, vectors
    ((2, 5, 3, 10), (0, 2, 1, 3)),        # rows, element-wise (10 is no whole number of vectors)
    ((3, 7, 12), (1, 0, 2)),
    ((64, 64), (1, 0)),                   # one full tile
    ((128, 192), (1, 0)),                 # several tiles, vectors
    ((100, 36), (1, 0)),                  # ragged tiles, vectors of 4 (fp32) / element-wise (bf16: 36 % 8)
    ((33, 17), (1, 0)),                   # ragged, element-wise
    ((3, 70, 130), (0, 2, 1)),            # batched transpose, element-wise edges
    ((2, 72, 5, 136), (3, 2, 0, 1)),      # source-contiguous dimension moved outward with a batch in between
    ((4, 8, 16, 32), (3, 2, 1, 0)),       # full reversal
    ((2, 3, 4, 5, 6, 7), (5, 3, 1, 0, 2, 4)),
    ((1, 40, 1, 24), (3, 2, 1, 0)),       # extent-1 dimensions drop out
    ((6, 1), (1, 0)),
    ((1,), (0,)),
    ((2, 2, 2, 2, 2, 2, 2, 8), (6, 5, 4, 3, 2, 1, 0, 7)),   # eight dimensions, innermost kept
]


@pytest.mark.parametrize("shape,dims", PERMS)
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_permuted_view_made_contiguous(ctx, shape, dims, dtype):
    rng = np.random.default_rng(SEED + len(shape) + sum(shape))
    x = rng.standard_normal(shape).astype(np.float32)
    flat = (to_bf16_bits(x) if dtype == "bf16" else x).reshape(-1)
    vshape, vstrides = _permuted(shape, dims)
    want = ref.contiguous_forward(flat, vshape, vstrides)
    np.testing.assert_array_equal(want, np.transpose(flat.reshape(shape), dims))
    got = _run(ctx, flat, vshape, vstrides, dtype)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("shape,dims", PERMS)
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_permute_gradient_accumulates(ctx, shape, dims, dtype):
    """x.grad += out.grad with the permutation undone (cpu_permute_backward,
    backend.py:289-298): out.grad is dense in the permuted shape, x.grad dense in x's"""
    rng = np.random.default_rng(SEED + 7 + sum(shape))
    oshape = tuple(shape[d] for d in dims)
    g = rng.standard_normal(oshape).astype(np.float32)
    base = rng.standard_normal(shape).astype(np.float32)
    if dtype == "bf16":
        gs, bs = to_bf16_bits(g), to_bf16_bits(base)
        g, base = from_bf16_bits(gs), from_bf16_bits(bs)
    else:
        gs, bs = g, base
    dense = contiguous_strides(oshape)
    strides = [0] * len(shape)
    for i, d in enumerate(dims):
        strides[d] = dense[i]
    want = base.copy()
    ref.permute_backward_into(g, list(dims), want)
    got = _run(ctx, gs.reshape(-1), shape, strides, dtype, flags=capi.ACC_INPUT_GRAD, init=bs.reshape(-1))
    if dtype == "bf16":
        np.testing.assert_array_equal(got, to_bf16_bits(want))
    else:
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_broadcast_sliced_and_offset_views(ctx, dtype):
    rng = np.random.default_rng(SEED + 99)
    x = rng.standard_normal(4096).astype(np.float32)
    flat = to_bf16_bits(x) if dtype == "bf16" else x
    cases = [
        ((5, 64), (0, 1)),              # a row repeated (stride 0)
        ((8, 16), (32, 2)),             # every other element: no unit stride anywhere
        ((3, 4, 8), (512, 8, 1)),       # a sliced block: rows, vectors, gaps between rows
        ((16, 24), (1, 64)),            # transpose of a sliced block
        ((7,), (3,)),
        ((), ()),                       # a scalar
        ((0, 5), (5, 1)),               # nothing to move
    ]
    for shape, strides in cases:
        want = ref.contiguous_forward(flat, shape, strides) if len(shape) else flat[:1].reshape(())
        got = _run(ctx, flat, shape, strides, dtype)
        np.testing.assert_array_equal(got, want, err_msg=f"{shape} {strides}")
    # the view may start anywhere in the buffer: the caller passes the address of its first element
    off = 37
    want = ref.contiguous_forward(flat, (6, 10), (20, 2), offset=off)
    got = _run(ctx, flat[off:].copy(), (6, 10), (20, 2), dtype)
    np.testing.assert_array_equal(got, want)


def test_attention_layout_round_trip_at_full_size(ctx):
    """config-4 q, [8, 2048, 12, 128] fp32: BTHD -> BHTD -> BTHD returns the input bits"""
    B, T, H, D = 8, 2048, 12, 128
    rng = np.random.default_rng(SEED + 4)
    x = rng.standard_normal((B, T, H, D)).astype(np.float32)
    vshape, vstrides = _permuted((B, T, H, D), (0, 2, 1, 3))
    y = _run(ctx, x.reshape(-1), vshape, vstrides, "f32")
    np.testing.assert_array_equal(y, np.transpose(x, (0, 2, 1, 3)))
    bshape, bstrides = _permuted((B, H, T, D), (0, 2, 1, 3))
    z = _run(ctx, y.reshape(-1), bshape, bstrides, "f32")
    np.testing.assert_array_equal(z, x)


def test_rejects_bad_arguments(ctx):
    buf = ctx.upload(np.zeros(64, np.float32))
    sh = (C.c_uint32 * 9)(*([2] * 9))
    st = (C.c_uint64 * 9)(*([1] * 9))
    with pytest.raises(capi.AgradError):
        ctx.call("agrad_strided_copy", capi.F32, C.c_void_p(buf.ptr), C.c_void_p(buf.ptr), 9, sh, st, 0)
    with pytest.raises(capi.AgradError):
        ctx.call("agrad_strided_copy", capi.F32, None, C.c_void_p(buf.ptr), 1, sh, st, 0)
    with pytest.raises(capi.AgradError):
        ctx.call("agrad_strided_copy", 7, C.c_void_p(buf.ptr), C.c_void_p(buf.ptr), 1, sh, st, 0)
    buf.free()
