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


def assert_fp32_parity(got, cpu, exact, what=""):
    """The fp32 bar with its one documented way out: `got` meets rtol 1e-5 / atol 1e-6
    against the CPU restatement `cpu`, or it is as close to the float64 value `exact` as
    the restatement is (largest error within 1.25 x, root-mean-square error within 1.1 x
    of the restatement's: the sample-to-sample spread of two equally good fp32
    evaluations).  tests/test_gpu_error_budget.py tabulates the three distances."""
    got64, cpu64, exact = (np.asarray(a, dtype=np.float64) for a in (got, cpu, exact))
    assert got64.shape == cpu64.shape == exact.shape, f"{what}: shapes {got64.shape} {cpu64.shape} {exact.shape}"
    if (np.abs(got64 - cpu64) <= FP32_ATOL + FP32_RTOL * np.abs(cpu64)).all():
        return
    e_d, e_c = np.abs(got64 - exact), np.abs(cpu64 - exact)
    rms_d, rms_c = np.sqrt((e_d ** 2).mean()), np.sqrt((e_c ** 2).mean())
    assert e_d.max() <= 1.25 * e_c.max() + 1e-12 and rms_d <= 1.1 * rms_c + 1e-12, (
        f"{what}: misses rtol {FP32_RTOL} / atol {FP32_ATOL} against the CPU restatement (max |diff| "
        f"{np.abs(got64 - cpu64).max():.3e}) and is not as close to float64: max {e_d.max():.3e} vs {e_c.max():.3e}, "
        f"rms {rms_d:.3e} vs {rms_c:.3e}")


def assert_chain_close(got, ref, what, kernels, sum_rows=1):
    """Whole-graph fp32 comparisons.  The kernel tests hold every kernel to rtol 1e-5 / atol 1e-6 of its
    own output; `kernels` of them in a chain (forward and backward kernels between the inputs and the
    compared value both count) compound to at most `kernels` times that at the end of the chain, on the
    scale of the values compared; a gradient summed over `sum_rows` rows (gamma, beta, a bias, a table
    row that many ids hit) adds what the two devices' different summation orders may differ by,
    1e-6 sqrt(sum_rows) of that scale."""
    ref64 = np.asarray(ref, dtype=np.float64)
    scale = max(1.0, float(np.abs(ref64).max()) if ref64.size else 1.0)
    atol = FP32_ATOL * kernels * scale + (FP32_ATOL * float(np.sqrt(sum_rows)) * scale if sum_rows > 1 else 0.0)
    assert_fp32_close(got, ref, what, rtol=FP32_RTOL * kernels, atol=atol)


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
