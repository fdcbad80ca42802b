"""Writes tests/golden/layer_ops_small.npz: seeded inputs and the outputs of the
CPU restatement (oracle/cpu_ops.py) for every op of the path at probe sizes.

The reference ships no stored vectors for this path, only recipes (seeds, shapes
and tolerances: check_tiny_gpt2_kernel.py:47-54, 758-794; verify_model.py:22-26,
298-318; debug/check_qwen_kernel.py:19-21), and it was not imported to make
these: the file freezes what the restatement produced when it was checked
against its closed forms, so that a later change to the restatement or to a
kernel shows up against fixed numbers.

    python tests/golden/make_vectors.py
"""
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
from oracle import cpu_ops as K  # noqa: E402

SEED = 1333   # check_tiny_gpt2_kernel.py:47


def build():
    rng = np.random.default_rng(SEED)
    B, T, C, V, H = 2, 8, 32, 53, 64
    v = {}
    x = rng.standard_normal((B, T, C)).astype(np.float32)
    res = rng.standard_normal((B, T, C)).astype(np.float32)
    dy = rng.standard_normal((B, T, C)).astype(np.float32)
    gamma = (1 + 0.02 * rng.standard_normal(C)).astype(np.float32)
    beta = (0.02 * rng.standard_normal(C)).astype(np.float32)
    v.update(x=x, res=res, dy=dy, gamma=gamma, beta=beta)
    v["ln_y"] = K.layernorm_forward(x, gamma, beta, 1e-5)
    dx, dg, db = np.zeros_like(x), np.zeros_like(gamma), np.zeros_like(beta)
    K.layernorm_backward_into(x, gamma, dy, 1e-5, dx, dg, db)
    v.update(ln_dx=dx, ln_dgamma=dg, ln_dbeta=db)
    v["rms_y"] = K.rmsnorm_forward(x, gamma, 1e-6)
    dx, dg = np.zeros_like(x), np.zeros_like(gamma)
    K.rmsnorm_backward_into(x, gamma, dy, 1e-6, dx, dg)
    v.update(rms_dx=dx, rms_dgamma=dg)
    h, y = K.add_norm_forward("layer", x, res, gamma, beta, 1e-5)
    v.update(addln_h=h, addln_y=y)
    a = rng.standard_normal((B * T, H)).astype(np.float32)
    da = rng.standard_normal((B * T, H)).astype(np.float32)
    v.update(act_x=a, act_dy=da, gelu_y=K.gelu_forward(a), relu2_y=K.relu2_forward(a))
    d = np.zeros_like(a)
    K.gelu_backward_into(a, da, d)
    v["gelu_dx"] = d
    d = np.zeros_like(a)
    K.relu2_backward_into(a, da, d)
    v["relu2_dx"] = d
    gu = rng.standard_normal((B * T, 2 * H)).astype(np.float32)
    v.update(gu=gu, swiglu_h=K.swiglu_forward(gu), swiglu_dgu=K.swiglu_backward(gu, da))
    Hq, Hkv, D = 4, 2, 8
    q = rng.standard_normal((B, T, Hq, D)).astype(np.float32)
    k = rng.standard_normal((B, T, Hkv, D)).astype(np.float32)
    cos, sin = K.rope_tables(T, D, 1e4)
    q2, k2 = q.copy(), k.copy()
    K.rope_signed(q2, k2, cos, sin, 1, False)
    v.update(rope_q=q, rope_k=k, rope_cos=cos, rope_sin=sin, rope_q_out=q2, rope_k_out=k2)
    ids = rng.integers(0, V, (B, T), dtype=np.int32)
    ids[0, :4] = 5                                     # a repeated token
    W = (0.02 * rng.standard_normal((V, C))).astype(np.float32)
    wpe = (0.02 * rng.standard_normal((T, C))).astype(np.float32)
    v.update(ids=ids, W=W, wpe=wpe, gather_out=K.gather_forward(ids, W), embsum_out=K.embedding_sum_forward(ids, W, wpe))
    dW, dwpe = np.zeros_like(W), np.zeros_like(wpe)
    K.embedding_sum_backward_into(ids, dy, dW, dwpe)
    v.update(emb_dW=dW, emb_dwpe=dwpe)
    logits = (3.0 * rng.standard_normal((B, T, V))).astype(np.float32)
    dloss = rng.standard_normal((B, T)).astype(np.float32)
    dlog = np.zeros_like(logits)
    K.cross_entropy_backward_into(logits, ids, dloss, dlog)
    v.update(logits=logits, dloss=dloss, ce_loss=K.cross_entropy_forward(logits, ids), ce_dlogits=dlog)
    p = rng.standard_normal(257).astype(np.float32)
    g = rng.standard_normal(257).astype(np.float32)
    m, vv = np.zeros_like(p), np.zeros_like(p)
    v.update(adam_p0=p.copy(), adam_g=g)
    K.adamw_step(p, g, m, vv, 1e-3, 1e-3 * np.sqrt(1 - 0.999) / (1 - 0.9), 0.9, 0.999, 1e-8, 0.1)
    v.update(adam_p1=p, adam_m1=m, adam_v1=vv)
    return v


if __name__ == "__main__":
    out = Path(__file__).with_name("layer_ops_small.npz")
    np.savez_compressed(out, **build())
    print(f"wrote {out} ({out.stat().st_size} bytes)")
