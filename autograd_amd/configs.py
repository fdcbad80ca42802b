"""The five benchmark / parity configurations of the fused layer-op path.

Each config lists the ops it exercises with their shapes.  `e` below is the
element size of the large operands (4 for fp32, 2 for bf16 I/O); parameter
vectors, rotary tables and token ids are fp32 / int32 regardless.

Algorithmic bytes per op (what a perfect kernel must move through HBM):
    gather forward        4N + 2*N*C*e            (+ T*C*e with the position table)
    embedding backward    4N + N*C*e + U*C*e      (U = distinct ids; the zero-fill of
                                                   the V*C*e table is counted separately)
    gather-sum backward   the above + T*C*e       (dY counted once)
    norm forward          2*N*C*e ; with the residual fused 4*N*C*e (read x, r; write h, y)
    norm backward         3*N*C*e + 2*C*4 ; with the residual gradient fused 4*N*C*e + 2*C*4
    GELU / ReLU^2         2*N*H*e forward, 3*N*H*e backward
    SwiGLU                3*N*H*e forward, 5*N*H*e backward (in place on gu)
    RoPE                  2*(numel(q) + numel(k))*e, forward and backward
"""
from __future__ import annotations

from dataclasses import dataclass, field


@dataclass(frozen=True)
class LayerOpConfig:
    index: int            # position in the benchmark's config list
    name: str
    dtype: str            # "f32" or "bf16"
    B: int
    T: int
    C: int
    V: int
    seed: int
    embed: str = ""       # "gather", "gather_sum" or "" ; backward is included
    embed_dist: str = "uniform"     # token id distribution for the backward
    norm: str = ""        # "layer" or "rms"
    norm_eps: float = 1e-5
    norm_residual: bool = False
    norm_affine: bool = True        # False: gamma = 1, beta = 0
    act: str = ""         # "gelu", "relu2", "swiglu"
    act_width: int = 0    # H (for swiglu the input is 2H wide)
    rope: tuple = ()      # (H, HKV, D, theta, rope_sign)

    @property
    def N(self) -> int:
        return self.B * self.T

    @property
    def esize(self) -> int:
        return 2 if self.dtype == "bf16" else 4


SEED = 1333   # base seed of the reference's probes (check_tiny_gpt2_kernel.py:47)

CONFIGS = (
    LayerOpConfig(0, "tiny-gpt2-chain", "f32", B=4, T=128, C=128, V=50257, seed=SEED + 0,
                  embed="gather_sum", norm="layer", norm_eps=1e-5, norm_affine=False,
                  act="gelu", act_width=512),
    LayerOpConfig(1, "nanochat-d6", "f32", B=32, T=512, C=384, V=32768, seed=SEED + 1,
                  embed="gather", norm="layer", norm_eps=1e-5, norm_residual=True,
                  act="relu2", act_width=1536, rope=(6, 6, 64, 1e4, -1)),
    LayerOpConfig(2, "gpt2-small", "f32", B=16, T=1024, C=768, V=50257, seed=SEED + 2,
                  embed="gather_sum", norm="layer", norm_eps=1e-5, norm_residual=True,
                  act="gelu", act_width=3072),
    LayerOpConfig(3, "qwen2.5-1.5b", "f32", B=8, T=2048, C=1536, V=151936, seed=SEED + 3,
                  embed="gather", norm="rms", norm_eps=1e-6,
                  act="swiglu", act_width=8960, rope=(12, 2, 128, 1e6, 1)),
    LayerOpConfig(4, "qwen2.5-1.5b-bf16", "bf16", B=8, T=2048, C=1536, V=151936, seed=SEED + 3,
                  embed="gather", norm="rms", norm_eps=1e-6,
                  act="swiglu", act_width=8960, rope=(12, 2, 128, 1e6, 1)),
    LayerOpConfig(5, "llama3-8b-width-bf16", "bf16", B=16, T=4096, C=4096, V=128256, seed=SEED + 4,
                  embed="gather", embed_dist="zipf1.1", norm="rms", norm_eps=1e-5, norm_residual=True,
                  act="swiglu", act_width=14336, rope=(32, 8, 128, 5e5, 1)),
)


def op_bytes(cfg: LayerOpConfig, distinct_ids: int | None = None) -> dict:
    """algorithmic HBM bytes per op and direction: {op name: (forward, backward)}"""
    N, C, e = cfg.N, cfg.C, cfg.esize
    out = {}
    if cfg.embed:
        U = distinct_ids if distinct_ids is not None else N
        fwd = 4 * N + 2 * N * C * e
        bwd = 4 * N + N * C * e + U * C * e
        if cfg.embed == "gather_sum":
            fwd += cfg.T * C * e
            bwd += cfg.T * C * e
        out[cfg.embed] = (fwd, bwd)
    if cfg.norm:
        fwd = (4 if cfg.norm_residual else 2) * N * C * e
        bwd = (4 if cfg.norm_residual else 3) * N * C * e + 2 * C * 4
        out[("add+" if cfg.norm_residual else "") + cfg.norm + "norm"] = (fwd, bwd)
    if cfg.act:
        H = cfg.act_width
        if cfg.act == "swiglu":
            out["swiglu"] = (3 * N * H * e, 5 * N * H * e)
        else:
            out[cfg.act] = (2 * N * H * e, 3 * N * H * e)
    if cfg.rope:
        Hq, Hkv, D, _, _ = cfg.rope
        b = 2 * (N * Hq * D + N * Hkv * D) * e
        out["rope"] = (b, b)
    return out
