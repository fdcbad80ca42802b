"""The pieces composed: a small language model that needs no matrix product -- next
token logits are a LayerNorm of the current token's row of a [V, V] table, scaled by a
learned vector -- trained for a few dozen AdamW steps with gradient clipping on the
HIP device and on the oracle device.  Gather forward / backward, LayerNorm forward /
backward, broadcast Mul and its gradients, cross-entropy forward / backward, the
runtime's gradient zeroing and AdamW all have to agree step after step for the two
loss curves to stay together, and the loss has to fall for the gradients to be right.
"""
import numpy as np
import pytest

from autograd_amd.op import CrossEntropyLossOp, GatherOp, LayerNormOp
from autograd_amd.optimizer import AdamW
from autograd_amd.runtime import Runtime
from autograd_amd.tensor import Tensor
from oracle import cpu_device

pytestmark = pytest.mark.gpu
SEED = 1333
cpu_device.register()


def _train(device, steps, V, B, T, batches):
    rng = np.random.default_rng(SEED + 40)          # same initial weights on both devices
    table = Tensor(shape=(V, V), dtype=np.float32, device=device, requires_grad=True,
                   init_val=(0.1 * rng.standard_normal((V, V))).astype(np.float32), name="table")
    gamma = Tensor(shape=(V,), dtype=np.float32, device=device, requires_grad=True,
                   init_val=np.ones(V, np.float32), name="gamma")
    beta = Tensor(shape=(V,), dtype=np.float32, device=device, requires_grad=True,
                  init_val=np.zeros(V, np.float32), name="beta")
    temp = Tensor(shape=(V,), dtype=np.float32, device=device, requires_grad=True,
                  init_val=np.full(V, 0.5, np.float32), name="temp")
    ids = Tensor(shape=(B, T), dtype=np.int32, device=device, requires_grad=False, name="ids")
    targets = Tensor(shape=(B, T), dtype=np.int32, device=device, requires_grad=False, name="targets")
    logits = LayerNormOp(eps=1e-5)(GatherOp()(ids, table), gamma, beta) * temp
    loss = CrossEntropyLossOp()(logits, targets)
    rt = Runtime(device=device)
    rt.loss = loss
    rt.build_topo(loss)
    rt.bind_memory()
    rt.is_compiled = True
    opt = AdamW([table, gamma, beta, temp], lr=3e-2, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.01, runtime=rt)
    clip = opt.build_grad_clip()
    curve, norms = [], []
    for step in range(steps):
        x, y = batches[step]
        rt.backend.copy_from_host(ids, x)
        rt.backend.copy_from_host(targets, y)
        rt.backward(loss, grad_scale=1.0 / (B * T))
        rt.backend.synchronize()
        curve.append(float(rt.backend.copy_to_host(loss).mean()))
        norm, coef = clip(1.0)
        norms.append(norm)
        opt.step(grad_scale=coef)
    final = {p.name: rt.backend.copy_to_host(p).copy() for p in (table, gamma, beta, temp)}
    opt.release()
    rt.release()
    return np.array(curve), np.array(norms), final


def test_a_table_language_model_trains_the_same_on_both_devices():
    V, B, T, steps = 96, 8, 64, 40
    rng = np.random.default_rng(SEED + 41)
    batches = []
    for _ in range(steps):
        x = rng.integers(0, V, (B, T), dtype=np.int32)
        noise = rng.random((B, T)) < 0.1
        y = np.where(noise, rng.integers(0, V, (B, T)), (5 * x + 3) % V).astype(np.int32)   # a noisy bigram rule
        batches.append((x, y))
    cpu_curve, cpu_norms, cpu_final = _train("cpu", steps, V, B, T, batches)
    hip_curve, hip_norms, hip_final = _train("hip", steps, V, B, T, batches)
    # it learns: from ~ln(V) towards the noise floor of the rule
    assert abs(cpu_curve[0] - np.log(V)) < 0.4        # unit-variance logits * 0.5: ln V + 1/8
    assert cpu_curve[-1] < cpu_curve[0] - 1.5 and hip_curve[-1] < hip_curve[0] - 1.5
    # and the two devices walk the same path (AdamW's sqrt / divide amplify last-bit differences a little)
    np.testing.assert_allclose(hip_curve, cpu_curve, rtol=2e-4, atol=2e-4)
    np.testing.assert_allclose(hip_norms, cpu_norms, rtol=2e-3)
    for name in cpu_final:
        np.testing.assert_allclose(hip_final[name], cpu_final[name], rtol=0, atol=5e-3, err_msg=name)
