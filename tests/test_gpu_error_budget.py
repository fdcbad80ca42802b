"""Three-way error budget of every fp32 output: device vs the CPU restatement, device vs
float64, CPU restatement vs float64 -- at each fp32 configuration's width and data recipe,
on a block of rows the numpy restatement finishes in seconds.

The bar for fp32 outputs is rtol 1e-5 / atol 1e-6 against the CPU restatement.  Two fp32
evaluations of one formula that associate their adds differently each sit a few ulp of the
largest intermediate away from the exact value, so on outputs whose intermediates are
larger than the result (dx of the norms, the activations' derivatives, sums over rows)
they can differ from EACH OTHER by more than 1e-6 although neither is wrong.  This test
pins what is acceptable there: an output either meets the bar against the CPU restatement,
or the device is as close to the float64 closed form as the CPU restatement is (largest
error no more than 1.25 x the restatement's largest, root-mean-square error no more than
1.1 x the restatement's: the margins are the sample-to-sample spread of two equally good
evaluations over millions of elements) -- and in every case the device differs from the
restatement by no more than the two distances from float64 together.

The table is also written as error_budget.md into the run's output folder, when that can be written.
"""
import os
from pathlib import Path

import numpy as np
import pytest

from autograd_amd import capi
from autograd_amd.configs import CONFIGS
from oracle import closed_form as cf
from oracle import cpu_ops as K
from tests import gpu_ops as G

pytestmark = pytest.mark.gpu

ROWS = 2048
FP32 = [c for c in CONFIGS if c.dtype == "f32"]
_TABLE = []


def _three_way(cfg, what, dev, cpu, exact):
    dev64, cpu64, exact = (np.asarray(a, dtype=np.float64) for a in (dev, cpu, exact))
    e_dc = np.abs(dev64 - cpu64)
    e_d = np.abs(dev64 - exact)
    e_c = np.abs(cpu64 - exact)
    meets_bar = bool((e_dc <= 1e-6 + 1e-5 * np.abs(cpu64)).all())
    rms_d, rms_c = float(np.sqrt((e_d ** 2).mean())), float(np.sqrt((e_c ** 2).mean()))
    row = dict(cfg=cfg.name, what=what, scale=float(np.abs(exact).max()), dev_cpu=float(e_dc.max()), dev_f64=float(e_d.max()),
               cpu_f64=float(e_c.max()), rms_dev=rms_d, rms_cpu=rms_c, meets_bar=meets_bar)
    _TABLE.append(row)
    assert e_dc.max() <= e_d.max() + e_c.max() + 1e-30, (cfg.name, what)
    if not meets_bar:
        assert rms_d <= rms_c * 1.1 + 1e-12, f"{cfg.name} {what}: device rms error {rms_d:.3e} vs restatement {rms_c:.3e}"
        assert e_d.max() <= 1.25 * e_c.max() + 1e-12, f"{cfg.name} {what}: device max error {e_d.max():.3e} vs restatement {e_c.max():.3e}"
    return row


def _write_table():
    lines = ["| config | output | max abs value | device vs CPU | device vs f64 | CPU vs f64 | rms device | rms CPU | rtol 1e-5 / atol 1e-6 vs CPU |",
             "|---|---|---|---|---|---|---|---|---|"]
    for r in _TABLE:
        lines.append(f"| {r['cfg']} | {r['what']} | {r['scale']:.3g} | {r['dev_cpu']:.2e} | {r['dev_f64']:.2e} | {r['cpu_f64']:.2e} | "
                     f"{r['rms_dev']:.2e} | {r['rms_cpu']:.2e} | {'met' if r['meets_bar'] else 'device as close to f64'} |")
    out = Path(os.environ.get("GRAFT_REPO_ROOT", Path(__file__).resolve().parent.parent)) / "gpurun_out"
    try:
        out.mkdir(exist_ok=True)
        (out / "error_budget.md").write_text("\n".join(lines) + "\n")
    except OSError:
        pass


@pytest.fixture(scope="module", autouse=True)
def _table_at_the_end():
    yield
    _write_table()


@pytest.mark.parametrize("cfg", FP32, ids=[f"cfg{c.index}-{c.name}" for c in FP32])
def test_norm_error_budget(ctx, cfg):
    rng = np.random.default_rng(cfg.seed + 100)
    rows, C = min(ROWS, cfg.N), cfg.C
    x = rng.standard_normal((rows, C), dtype=np.float32)
    res = rng.standard_normal((rows, C), dtype=np.float32) if cfg.norm_residual else None
    gamma = (1 + 0.02 * rng.standard_normal(C)).astype(np.float32) if cfg.norm_affine else np.ones(C, np.float32)
    beta = (0.02 * rng.standard_normal(C)).astype(np.float32) if cfg.norm_affine else np.zeros(C, np.float32)
    dy = rng.standard_normal((rows, C), dtype=np.float32)
    dres = rng.standard_normal((rows, C), dtype=np.float32) if cfg.norm_residual else None
    layer = cfg.norm == "layer"
    kind = capi.NORM_LAYER if layer else capi.NORM_RMS
    y, h = G.norm_forward(ctx, kind, x, gamma, beta if layer else None, cfg.norm_eps, residual=res, want_h=res is not None)
    h_cpu = K.add_forward(x, res) if res is not None else x
    if res is not None:
        np.testing.assert_array_equal(h, h_cpu)                    # one fp32 add: the same bits
    if layer:
        y_cpu = K.layernorm_forward(h_cpu, gamma, beta, cfg.norm_eps)
        y_64 = cf.layernorm(h_cpu, gamma, beta, cfg.norm_eps)[0]
    else:
        y_cpu = K.rmsnorm_forward(h_cpu, gamma, cfg.norm_eps)
        y_64 = cf.rmsnorm(h_cpu, gamma, cfg.norm_eps)[0]
    _three_way(cfg, f"{cfg.norm}norm y", y, y_cpu, y_64)
    out = G.norm_backward(ctx, kind, h_cpu, gamma, dy, cfg.norm_eps, dres=dres, want_dbeta=layer)
    dx_cpu = np.zeros_like(x) if dres is None else dres.copy()
    dg_cpu, db_cpu = np.zeros(C, np.float32), np.zeros(C, np.float32)
    if layer:
        K.layernorm_backward_into(h_cpu, gamma, dy, cfg.norm_eps, dx_cpu, dg_cpu, db_cpu)
        dx_64, dg_64, db_64 = cf.layernorm_grads(h_cpu, gamma, dy, cfg.norm_eps)
    else:
        K.rmsnorm_backward_into(h_cpu, gamma, dy, cfg.norm_eps, dx_cpu, dg_cpu)
        dx_64, dg_64 = cf.rmsnorm_grads(h_cpu, gamma, dy, cfg.norm_eps)
    if dres is not None:
        dx_64 = dx_64 + dres.astype(np.float64)
    _three_way(cfg, f"{cfg.norm}norm dx" + (" (+ residual gradient)" if dres is not None else ""), out["dx"], dx_cpu, dx_64)
    _three_way(cfg, f"{cfg.norm}norm dgamma ({rows} rows)", out["dgamma"], dg_cpu, dg_64)
    if layer:
        _three_way(cfg, f"{cfg.norm}norm dbeta ({rows} rows)", out["dbeta"], db_cpu, db_64)


@pytest.mark.parametrize("cfg", FP32, ids=[f"cfg{c.index}-{c.name}" for c in FP32])
def test_activation_error_budget(ctx, cfg):
    rng = np.random.default_rng(cfg.seed + 200)
    rows, H = min(ROWS, cfg.N), cfg.act_width
    if cfg.act == "swiglu":
        gu = rng.standard_normal((rows, 2 * H), dtype=np.float32)
        dh = rng.standard_normal((rows, H), dtype=np.float32)
        _three_way(cfg, "swiglu h", G.swiglu_forward(ctx, gu), K.swiglu_forward(gu), cf.swiglu(gu))
        _three_way(cfg, "swiglu d[g|u]", G.swiglu_backward(ctx, gu, dh), K.swiglu_backward(gu, dh),
                   cf.swiglu_grads(gu, dh))
        return
    x = rng.standard_normal((rows, H), dtype=np.float32)
    dy = rng.standard_normal((rows, H), dtype=np.float32)
    fwd_cpu = K.gelu_forward(x) if cfg.act == "gelu" else K.relu2_forward(x)
    fwd_64 = cf.gelu(x) if cfg.act == "gelu" else cf.relu2(x)
    _three_way(cfg, f"{cfg.act} y", G.unary(ctx, f"agrad_{cfg.act}_forward", x), fwd_cpu, fwd_64)
    dx_cpu = np.zeros_like(x)
    (K.gelu_backward_into if cfg.act == "gelu" else K.relu2_backward_into)(x, dy, dx_cpu)
    dx_64 = (cf.gelu_grad(x) if cfg.act == "gelu" else cf.relu2_grad(x)) * dy.astype(np.float64)
    _three_way(cfg, f"{cfg.act} dx", G.unary_backward(ctx, f"agrad_{cfg.act}_backward", x, dy),
               dx_cpu, dx_64)


@pytest.mark.parametrize("cfg", [c for c in FP32 if c.rope], ids=[f"cfg{c.index}-{c.name}" for c in FP32 if c.rope])
def test_rope_error_budget(ctx, cfg):
    rng = np.random.default_rng(cfg.seed + 300)
    Hq, Hkv, D, theta, sign = cfg.rope
    B, T = 2, min(cfg.T, 512)
    q = rng.standard_normal((B, T, Hq, D), dtype=np.float32)
    k = rng.standard_normal((B, T, Hkv, D), dtype=np.float32)
    cos, sin = K.rope_tables(T, D, theta)
    for backward in (False, True):
        q_ref, k_ref = q.copy(), k.copy()
        K.rope_signed(q_ref, k_ref, cos, sin, sign, backward)
        q_dev, k_dev = G.rope(ctx, q, k, cos, sin, sign, backward=backward)
        name = "rope " + ("backward" if backward else "forward")
        _three_way(cfg, name + " q", q_dev, q_ref, cf.rope(q, cos, sin, sign, backward))
        _three_way(cfg, name + " k", k_dev, k_ref, cf.rope(k, cos, sin, sign, backward))
        np.testing.assert_array_equal(q_dev, q_ref)
        np.testing.assert_array_equal(k_dev, k_ref)


@pytest.mark.parametrize("cfg", FP32, ids=[f"cfg{c.index}-{c.name}" for c in FP32])
def test_embedding_gradient_error_budget(ctx, cfg):
    rng = np.random.default_rng(cfg.seed + 400)
    B, T = (cfg.B, cfg.T) if cfg.N <= 4096 else (max(1, 4096 // cfg.T), min(cfg.T, 4096))
    V, C = min(cfg.V, 8192), min(cfg.C, 256)          # the float64 row loop is the slow part
    ids = rng.integers(0, V, size=(B, T), dtype=np.int32)
    dY = rng.standard_normal((B, T, C), dtype=np.float32)
    dW_cpu = np.zeros((V, C), np.float32)
    K.gather_backward_into(ids, dY, dW_cpu)
    got = G.embedding_backward(ctx, ids, dY, V)
    _three_way(cfg, f"embedding dW ({B * T} uniform ids over {V})", got, dW_cpu, cf.gather_backward(ids, dY, V))
    np.testing.assert_array_equal(got, dW_cpu)        # runs of up to 127 rows: np.add.at's own order
    if cfg.embed == "gather_sum":
        dwpe_cpu = np.zeros((T, C), np.float32)
        K.embedding_sum_backward_into(ids, dY, None, dwpe_cpu)
        _three_way(cfg, f"position table dwpe (B = {B})", G.pos_embedding_backward(ctx, dY, dwpe_init=np.zeros((T, C), np.float32)),
                   dwpe_cpu, dY.astype(np.float64).sum(axis=0))
