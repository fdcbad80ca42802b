"""Comparison helpers shared by the parity tests."""
import numpy as np

FP32_RTOL = 1e-5   # fp32 outputs: 1e-5 relative / 1e-6 absolute against the CPU restatement
FP32_ATOL = 1e-6
BF16_REL = 1e-2    # bf16-I/O outputs: 1e-2 relative to the fp32 path on the same rounded inputs


def assert_fp32_close(got, ref, what="", rtol=FP32_RTOL, atol=FP32_ATOL):
    got = np.asarray(got, dtype=np.float32)
    ref = np.asarray(ref, dtype=np.float32)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} != {ref.shape}"
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    bound = atol + rtol * np.abs(ref.astype(np.float64))
    bad = err > bound
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(
            f"{what}: {int(bad.sum())}/{bad.size} outside rtol={rtol} atol={atol}; worst at {i}: "
            f"got {got[i]!r} ref {ref[i]!r} |err| {err[i]:.3e}")


def bf16_rel_error(got, ref):
    """max relative error over elements with |ref| > 1e-3 max|ref|, and max abs error."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    scale = np.abs(ref).max() if ref.size else 0.0
    mask = np.abs(ref) > 1e-3 * scale
    rel = (np.abs(got - ref)[mask] / np.abs(ref)[mask]).max() if mask.any() else 0.0
    return float(rel), float(np.abs(got - ref).max() if ref.size else 0.0), float(scale)


def assert_bf16_close(got, ref, what="", rel=BF16_REL):
    r, a, scale = bf16_rel_error(got, ref)
    assert r <= rel, f"{what}: max relative error {r:.3e} > {rel} (max abs {a:.3e}, scale {scale:.3e})"
    # elements under the relative mask are held to the same budget on the output's scale
    assert a <= rel * scale, f"{what}: max abs error {a:.3e} > {rel} * {scale:.3e}"


def to_bf16_bits(a):
    from oracle import cpu_ops
    return cpu_ops.f32_to_bf16_bits(a).reshape(np.shape(a))


def from_bf16_bits(b):
    from oracle import cpu_ops
    return cpu_ops.bf16_bits_to_f32(b).reshape(np.shape(b))
