"""Seeded synthetic inputs of the benchmark configurations.

x ~ N(0,1); every weight ~ N(0, 0.02); drawn in fp32 with
numpy.random.Generator(PCG64(seed)) in the order x, W_r, gate, up, down,
shared_gate, shared_up, shared_down.  The skewed configuration biases the
selection (not the weights) through expert_bias, the reference's own hook
(moe.py:139-140): -0.085 * 1.2 * ln(rank) with a seeded rank permutation, the six
highest ranks disabled with -4.
"""

from __future__ import annotations

import numpy as np

CONFIGS = {
    "C1": dict(batch=1, seq=2048, H=512, E=8, K=2, I=1024, Ns=0, dtype="f32"),
    "C2": dict(batch=4, seq=2048, H=1024, E=16, K=2, I=2816, Ns=0, dtype="bf16"),
    "C3": dict(batch=8, seq=2048, H=2048, E=64, K=8, I=1408, Ns=2, dtype="bf16"),
    "C4": dict(batch=8, seq=2048, H=2048, E=128, K=8, I=768, Ns=0, dtype="bf16", skew=True),
    "C5": dict(batch=64, seq=1, H=2048, E=64, K=8, I=1408, Ns=0, dtype="bf16"),
}

DESCRIPTIONS = {
    "C1": "MoE layer fwd fp32: T=2048, d_model=512, 8 experts, top-2, SwiGLU d_ff=1024",
    "C2": "MoE layer fwd bf16: T=8192 (4x2048), d_model=1024, 16 experts, top-2, SwiGLU d_ff=2816",
    "C3": "Fine-grained MoE fwd bf16: T=16384, d_model=2048, 64 experts, top-8, SwiGLU d_ff=1408, 2 shared experts",
    "C4": "Skewed-routing MoE fwd bf16: T=16384, d_model=2048, 128 experts, top-8, d_ff=768, Zipf(1.2) expert bias",
    "C5": "Decode-shaped MoE fwd bf16: T=64, d_model=2048, 64 experts, top-8, d_ff=1408",
}


def zipf_expert_bias(num_experts: int) -> np.ndarray:
    rank = 1 + np.random.Generator(np.random.PCG64(1)).permutation(num_experts)
    bias = (-0.085 * 1.2 * np.log(rank.astype(np.float64))).astype(np.float32)
    bias[rank > num_experts - 6] = np.float32(-4.0)
    return bias


def make_inputs(name: str, seed: int = 0) -> dict:
    cfg = dict(CONFIGS[name])
    rng = np.random.Generator(np.random.PCG64(seed))
    B, S, H, E, K, I, Ns = (cfg[k] for k in ("batch", "seq", "H", "E", "K", "I", "Ns"))
    sd = np.float32(0.02)
    x = rng.standard_normal((B, S, H), dtype=np.float32)
    w_router = rng.standard_normal((H, E), dtype=np.float32) * sd
    gate = rng.standard_normal((E, H, I), dtype=np.float32) * sd
    up = rng.standard_normal((E, H, I), dtype=np.float32) * sd
    down = rng.standard_normal((E, I, H), dtype=np.float32) * sd
    shared = None
    if Ns:
        shared = tuple(rng.standard_normal(s, dtype=np.float32) * sd for s in ((H, I * Ns), (H, I * Ns), (I * Ns, H)))
    bias = zipf_expert_bias(E) if cfg.get("skew") else np.zeros((E,), dtype=np.float32)
    return dict(cfg=cfg, x=x, w_router=w_router, expert_bias=bias, gate=gate, up=up, down=down, shared=shared)
