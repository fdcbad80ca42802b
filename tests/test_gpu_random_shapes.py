"""Seeded random shapes through every kernel family against the CPU restatement.

The hand-picked shape lists of the other GPU tests name each launch geometry
once; this file draws shapes the lists do not contain (odd widths, widths just
around the geometry switch points, one-row and one-column problems, ragged row
counts) from a fixed seed, so a shape-dependent indexing mistake has many more
chances to show.  fp32, the tolerances of tests/helpers.py; gather, rotary, ReLU^2
and the layout copies are compared bit for bit.
"""
import numpy as np
import pytest

from autograd_amd import capi
from oracle import closed_form as cf
from oracle import cpu_ops as ref
from tests import gpu_ops as G
from tests.helpers import assert_fp32_close, assert_fp32_parity

pytestmark = pytest.mark.gpu
SEED = 1333
N_DRAWS = 24

# widths around the points where the norm kernels change lanes per row / vectors per lane
_WIDTH_POOL = [1, 2, 3, 4, 5, 7, 8, 12, 60, 63, 64, 65, 68, 124, 128, 132, 252, 256, 260, 380, 384, 388, 508, 512, 516,
               764, 768, 772, 1020, 1024, 1028, 1532, 1536, 1540, 2044, 2048, 2052, 3068, 3072, 4092, 4096, 4100,
               6140, 6144, 6148, 8188, 8192, 8196, 12288, 16384, 16388, 24576, 24580]


def _draws(k):
    rng = np.random.default_rng(SEED + 1000 + k)
    return [(int(rng.integers(1, 70)), int(rng.choice(_WIDTH_POOL)), int(rng.integers(0, 1 << 30))) for _ in range(N_DRAWS)]


@pytest.mark.parametrize("rows,C,seed", _draws(1))
def test_norms_at_random_shapes(ctx, rows, C, seed):
    rng = np.random.default_rng(seed)
    kind = ("layer", "rms")[seed & 1]
    with_res = bool(seed & 2)
    eps = (1e-5, 1e-6)[(seed >> 2) & 1]
    x = rng.standard_normal((rows, C)).astype(np.float32)
    res = rng.standard_normal((rows, C)).astype(np.float32) if with_res else None
    dy = rng.standard_normal((rows, C)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(C)).astype(np.float32)
    beta = (0.1 * rng.standard_normal(C)).astype(np.float32) if kind == "layer" else None
    K = capi.NORM_LAYER if kind == "layer" else capi.NORM_RMS
    h = ref.add_forward(x, res) if with_res else x
    want = ref.layernorm_forward(h, gamma, beta, eps) if kind == "layer" else ref.rmsnorm_forward(h, gamma, eps)
    y, h_got = G.norm_forward(ctx, K, x, gamma, beta, eps, residual=res, want_h=with_res)
    y64 = (cf.layernorm(h, gamma, beta, eps) if kind == "layer" else cf.rmsnorm(h, gamma, eps))[0]
    assert_fp32_parity(y, want, y64, f"{kind} y rows={rows} C={C}")
    if with_res:
        np.testing.assert_array_equal(h_got, h)
    dx, dg, db = np.zeros_like(h), np.zeros_like(gamma), np.zeros_like(gamma)
    if kind == "layer":
        ref.layernorm_backward_into(h, gamma, dy, eps, dx, dg, db)
    else:
        ref.rmsnorm_backward_into(h, gamma, dy, eps, dx, dg)
    out = G.norm_backward(ctx, K, h, gamma, dy, eps, want_dbeta=kind == "layer")
    g64 = cf.layernorm_grads(h, gamma, dy, eps) if kind == "layer" else cf.rmsnorm_grads(h, gamma, dy, eps)
    assert_fp32_parity(out["dx"], dx, g64[0], f"{kind} dx rows={rows} C={C}")
    assert_fp32_parity(out["dgamma"], dg, g64[1], f"{kind} dgamma")
    if kind == "layer":
        assert_fp32_parity(out["dbeta"], db, g64[2], f"{kind} dbeta")


@pytest.mark.parametrize("rows,C,seed", _draws(2))
def test_activations_at_random_shapes(ctx, rows, C, seed):
    rng = np.random.default_rng(seed)
    x = (2.0 * rng.standard_normal((rows, C))).astype(np.float32)
    dy = rng.standard_normal((rows, C)).astype(np.float32)
    assert_fp32_close(G.unary(ctx, "agrad_gelu_forward", x), ref.gelu_forward(x), "gelu")
    d = np.zeros_like(x)
    ref.gelu_backward_into(x, dy, d)
    # where tanh saturates the CPU forms 1 - t*t from a rounded t; the float64 derivative is the arbiter there
    got = G.unary_backward(ctx, "agrad_gelu_backward", x, dy)
    assert_fp32_parity(got, d, dy.astype(np.float64) * cf.gelu_grad(x.astype(np.float64)), "gelu dx")
    np.testing.assert_array_equal(G.unary(ctx, "agrad_relu2_forward", x), ref.relu2_forward(x))
    d = np.zeros_like(x)
    ref.relu2_backward_into(x, dy, d)
    np.testing.assert_array_equal(G.unary_backward(ctx, "agrad_relu2_backward", x, dy), d)
    if C % 2 == 0:
        dh = rng.standard_normal((rows, C // 2)).astype(np.float32)
        assert_fp32_parity(G.swiglu_forward(ctx, x), ref.swiglu_forward(x), cf.swiglu(x), "swiglu h")
        assert_fp32_parity(G.swiglu_backward(ctx, x, dh), ref.swiglu_backward(x, dh), cf.swiglu_grads(x, dh), "swiglu dgu")


@pytest.mark.parametrize("k", range(N_DRAWS))
def test_rotary_at_random_shapes(ctx, k):
    rng = np.random.default_rng(SEED + 3000 + k)
    B, T = int(rng.integers(1, 4)), int(rng.integers(1, 40))
    D = int(rng.choice([2, 4, 8, 16, 24, 32, 64, 96, 128, 256]))
    HKV = int(rng.integers(1, 5))
    H = HKV * int(rng.integers(1, 5))
    sign = (-1, 1)[k & 1]
    q = rng.standard_normal((B, T, H, D)).astype(np.float32)
    kk = rng.standard_normal((B, T, HKV, D)).astype(np.float32)
    cos, sin = ref.rope_tables(T + int(rng.integers(0, 5)), D, float(rng.choice([1e4, 5e5, 1e6])))
    for backward in (False, True):
        wq, wk = q.copy(), kk.copy()
        ref.rope_signed(wq, wk, cos, sin, sign, backward)
        gq, gk = G.rope(ctx, q, kk, cos, sin, sign, backward)
        np.testing.assert_array_equal(gq, wq)
        np.testing.assert_array_equal(gk, wk)


@pytest.mark.parametrize("k", range(N_DRAWS))
def test_embedding_at_random_shapes(ctx, k):
    rng = np.random.default_rng(SEED + 4000 + k)
    B, T = int(rng.integers(1, 9)), int(rng.integers(1, 600))
    V = int(rng.choice([1, 2, 7, 50, 1000, 40000]))
    C = int(rng.choice([1, 3, 4, 8, 20, 64, 100, 256, 384, 1000]))
    dist = ("uniform", "few", "one")[k % 3]
    if dist == "uniform":
        ids = rng.integers(0, V, (B, T), dtype=np.int32)
    elif dist == "few":
        ids = rng.choice(rng.integers(0, V, min(V, 5)), (B, T)).astype(np.int32)
    else:
        ids = np.full((B, T), int(rng.integers(0, V)), np.int32)
    W = (0.02 * rng.standard_normal((V, C))).astype(np.float32)
    wpe = (0.02 * rng.standard_normal((T, C))).astype(np.float32)
    dY = rng.standard_normal((B, T, C)).astype(np.float32)
    np.testing.assert_array_equal(G.gather_forward(ctx, ids, W), ref.gather_forward(ids, W))
    np.testing.assert_array_equal(G.gather_forward(ctx, ids, W, wpe), ref.embedding_sum_forward(ids, W, wpe))
    dW = np.zeros_like(W)
    ref.gather_backward_into(ids, dY, dW)
    got = G.embedding_backward(ctx, ids, dY, V)
    # one token may collect B*T rows: runs of up to 127 rows are added in np.add.at's own order,
    # longer ones in chunks (another association of the same terms)
    terms = np.zeros(V)
    np.add.at(terms, ids.ravel(), 1)
    if terms.max() <= 127:
        np.testing.assert_array_equal(got, dW)
    assert_fp32_parity(got, dW, cf.gather_backward(ids, dY, V), f"dW B={B} T={T} V={V} C={C} {dist}")
    assert not got[terms == 0].any()
    want_pos = dY[0].copy()
    for b in range(1, B):
        want_pos = want_pos + dY[b]
    np.testing.assert_array_equal(G.pos_embedding_backward(ctx, dY), want_pos)


@pytest.mark.parametrize("k", range(N_DRAWS))
def test_cross_entropy_at_random_shapes(ctx, k):
    import ctypes as Ct
    rng = np.random.default_rng(SEED + 5000 + k)
    rows = int(rng.integers(1, 40))
    V = int(rng.choice([1, 2, 3, 5, 63, 64, 65, 255, 257, 1000, 1023, 1025, 4099, 32768, 50257]))
    x = (3.0 * rng.standard_normal((rows, V))).astype(np.float32)
    labels = rng.integers(0, V, rows, dtype=np.int32)
    dloss = rng.standard_normal(rows).astype(np.float32)
    d_x, d_l, d_g = ctx.upload(x), ctx.upload(labels), ctx.upload(dloss)
    d_loss, d_lse = ctx.empty((rows,), np.float32), ctx.empty((rows,), np.float32)
    d_dx = ctx.upload(np.full(x.shape, 7, np.float32))

    def vp(d):
        return Ct.c_void_p(d.ptr)
    ctx.call("agrad_cross_entropy_forward", capi.F32, vp(d_x), vp(d_l), vp(d_loss), vp(d_lse), rows, V)
    ctx.call("agrad_cross_entropy_backward", capi.F32, vp(d_x), vp(d_l), vp(d_g), vp(d_lse), vp(d_dx), rows, V, 0)
    ctx.synchronize()
    want_dx = np.zeros_like(x)
    ref.cross_entropy_backward_into(x, labels, dloss, want_dx)
    assert_fp32_parity(d_loss.download(), ref.cross_entropy_forward(x, labels), cf.cross_entropy(x, labels), f"loss rows={rows} V={V}")
    assert_fp32_parity(d_dx.download(), want_dx, cf.cross_entropy_grad(x, labels, dloss), f"dlogits rows={rows} V={V}")
    for d in (d_x, d_l, d_g, d_loss, d_lse, d_dx):
        d.free()


@pytest.mark.parametrize("k", range(N_DRAWS))
def test_layout_copies_at_random_shapes(ctx, k):
    import ctypes as Ct
    rng = np.random.default_rng(SEED + 6000 + k)
    ndim = int(rng.integers(1, 6))
    shape = tuple(int(rng.choice([1, 2, 3, 4, 5, 8, 16, 17, 64, 66, 130])) for _ in range(ndim))
    while int(np.prod(shape)) > 1 << 21:
        shape = shape[1:]
    dims = tuple(int(d) for d in rng.permutation(len(shape)))
    x = rng.standard_normal(shape).astype(np.float32)
    base = [int(s) // 4 for s in x.strides]
    vshape = tuple(shape[d] for d in dims)
    vstrides = tuple(base[d] for d in dims)
    src = ctx.upload(x.reshape(-1))
    dst = ctx.upload(np.full(max(x.size, 1), 7, np.float32))
    sh = (Ct.c_uint32 * len(dims))(*vshape)
    st = (Ct.c_uint64 * len(dims))(*vstrides)
    ctx.call("agrad_strided_copy", capi.F32, Ct.c_void_p(src.ptr), Ct.c_void_p(dst.ptr), len(dims), sh, st, 0)
    ctx.synchronize()
    np.testing.assert_array_equal(dst.download()[:x.size].reshape(vshape), np.transpose(x, dims))
    src.free()
    dst.free()


@pytest.mark.parametrize("rows,C,seed", _draws(7))
def test_bf16_norms_and_swiglu_at_random_shapes(ctx, rows, C, seed):
    """bf16 storage (8 elements per 16-byte vector: other geometry switch points than
    fp32): 1e-2 relative to the fp32 restatement fed the same bf16-rounded inputs"""
    from tests.helpers import assert_bf16_close, from_bf16_bits, to_bf16_bits
    rng = np.random.default_rng(seed)
    kind = ("layer", "rms")[seed & 1]
    eps = 1e-5
    xs = to_bf16_bits(rng.standard_normal((rows, C)).astype(np.float32))
    dys = to_bf16_bits(rng.standard_normal((rows, C)).astype(np.float32))
    x, dy = from_bf16_bits(xs), from_bf16_bits(dys)
    gamma = (1 + 0.1 * rng.standard_normal(C)).astype(np.float32)
    beta = (0.1 * rng.standard_normal(C)).astype(np.float32) if kind == "layer" else None
    K = capi.NORM_LAYER if kind == "layer" else capi.NORM_RMS
    want = ref.layernorm_forward(x, gamma, beta, eps) if kind == "layer" else ref.rmsnorm_forward(x, gamma, eps)
    y, _ = G.norm_forward(ctx, K, xs, gamma, beta, eps)
    assert_bf16_close(from_bf16_bits(y), want, f"bf16 {kind} y rows={rows} C={C}")
    dx, dg, db = np.zeros_like(x), np.zeros_like(gamma), np.zeros_like(gamma)
    if kind == "layer":
        ref.layernorm_backward_into(x, gamma, dy, eps, dx, dg, db)
    else:
        ref.rmsnorm_backward_into(x, gamma, dy, eps, dx, dg)
    out = G.norm_backward(ctx, K, xs, gamma, dys, eps, want_dbeta=kind == "layer")
    if C > 1:      # one column: dx is exactly 0 up to rounding, nothing relative to compare
        assert_bf16_close(from_bf16_bits(out["dx"]), dx, f"bf16 {kind} dx rows={rows} C={C}")
    assert_fp32_close(out["dgamma"], dg, "bf16 dgamma (fp32 accumulators)", atol=1e-5 * np.sqrt(rows) + 1e-5, rtol=1e-4)
    if C % 2 == 0:
        dh = from_bf16_bits(to_bf16_bits(rng.standard_normal((rows, C // 2)).astype(np.float32)))
        assert_bf16_close(from_bf16_bits(G.swiglu_forward(ctx, xs)), ref.swiglu_forward(x), "bf16 swiglu h")
        assert_bf16_close(from_bf16_bits(G.swiglu_backward(ctx, xs, to_bf16_bits(dh))), ref.swiglu_backward(x, dh),
                          "bf16 swiglu dgu")
