"""Parity of RMSNorm, the fused combine + post-norm + residual kernel and the block entry point
with the oracle, on the GPU (through the C ABI).

The kernel sums the squares in its own order (lane-strided, then a butterfly over the wave), the
oracle with numpy's pairwise sum, so fp32 statistics can differ in the last bits: results are held
to one unit in the last place of the compute dtype on at most a small fraction of elements, and
to the forward's bar 2e-2 of the tensor maximum everywhere."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from research_amd import ops
from research_amd.errors import ContractError
from test_gpu_parity import BF16_MAX_REL, dev, host, random_problem, report

pytestmark = pytest.mark.gpu


def ulp_mismatch_fraction(got: np.ndarray, want: np.ndarray) -> float:
    """Fraction of bf16 values that differ, after checking that none differs by more than one ulp."""
    gb = O.bf16_bits(got).astype(np.int64)
    wb = O.bf16_bits(want).astype(np.int64)
    # order-preserving map of sign-magnitude patterns
    key = lambda b: np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)
    diff = np.abs(key(gb) - key(wb))
    assert diff.max() <= 1, f"bf16 results differ by up to {diff.max()} ulp"
    return float((diff != 0).mean())


def tail_mismatch_fraction(got: np.ndarray, want: np.ndarray, normed: np.ndarray) -> float:
    """out = residual + normed: a normed value that is one ulp off moves the sum by that ulp, which can be
    many ulps of a sum that cancels; so the error is bounded by one ulp of the normed term plus the
    rounding of the sum, and the fraction of elements that differ at all is returned."""
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    bound = 2.0 ** -7 * np.abs(normed) + 2.0 ** -7 * np.abs(want) + 1e-30
    assert np.all(err <= bound), f"worst excess {float(np.max(err / bound)):.2f} x the one-ulp bound"
    return float((got != want).mean())


@pytest.mark.parametrize("rows,hidden,dtype", [(2, 2, "bf16"), (300, 1024, "bf16"), (64, 2048, "bf16"), (33, 200, "bf16"),
                                               (17, 72, "f32"), (1000, 4096, "bf16")])
def test_rmsnorm_matches_oracle(gpu, rows, hidden, dtype):
    rng = np.random.default_rng(rows + hidden)
    x = (rng.standard_normal((rows, hidden)) * 2.5).astype(np.float32)
    scale = (1.0 + 0.2 * rng.standard_normal(hidden)).astype(np.float32)
    want = O.rmsnorm(x, scale, 1e-6, dtype)
    got = host(ops.rmsnorm(dev(x, gpu, dtype), dev(scale, gpu), 1e-6))
    if dtype == "bf16":
        frac = ulp_mismatch_fraction(got, want)
        print(f"[parity] rmsnorm bf16 rows={rows} H={hidden}: elements one ulp off: {frac:.2e}", flush=True)
        assert frac <= 2e-3
    else:
        np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-6)


def test_rmsnorm_reference_known_answer_and_contract(gpu):
    """tests/jaxtitan/test_kernels.py:192-204 and the wrapper's argument checks (:206-216)."""
    x = np.array([[[1.0, 2.0], [3.0, 4.0]]], np.float32)
    w = np.array([0.5, 1.5], np.float32)
    got = host(ops.rmsnorm(dev(x, gpu, "bf16"), dev(w, gpu), 0.0))
    np.testing.assert_array_equal(got, O.rmsnorm(x, w, 0.0, "bf16"))
    with pytest.raises(ContractError, match="rank"):
        ops.rmsnorm(dev(np.ones(4, np.float32), gpu, "bf16"), dev(np.ones(4, np.float32), gpu))
    with pytest.raises(ContractError, match="shape"):
        ops.rmsnorm(dev(np.ones((2, 4), np.float32), gpu, "bf16"), dev(np.ones(3, np.float32), gpu))
    with pytest.raises(ContractError, match="dtype"):
        ops.rmsnorm(dev(np.ones((2, 4), np.float32), gpu, "bf16"), dev(np.ones(4, np.float32), gpu, "bf16"))


@pytest.mark.parametrize("tokens,hidden,top_k,dtype,with_shared",
                         [(300, 2048, 8, "bf16", True), (129, 1024, 2, "bf16", False), (77, 72, 3, "bf16", True),
                          (50, 40, 2, "f32", True), (64, 4096, 8, "bf16", False), (33, 8192, 2, "bf16", True)])
def test_fused_combine_norm_residual(gpu, tokens, hidden, top_k, dtype, with_shared):
    rng = np.random.default_rng(tokens)
    rows = tokens * top_k
    packed_y = rng.standard_normal((rows, hidden)).astype(np.float32)
    inverse = rng.permutation(rows).astype(np.int32)
    w = rng.random((tokens, top_k)).astype(np.float32)
    shared_y = rng.standard_normal((tokens, hidden)).astype(np.float32) if with_shared else None
    residual = rng.standard_normal((tokens, hidden)).astype(np.float32)
    post = (0.3 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    y = O.combine(packed_y, inverse, w, dtype, shared_y)
    normed = O.rmsnorm(y, post, 1e-6, dtype)
    want = O.cast_compute(O.cast_compute(residual, dtype) + normed, dtype)
    pd, wd, rd = dev(packed_y, gpu, dtype), dev(w, gpu, dtype), dev(residual, gpu, dtype)
    sd = None if shared_y is None else dev(shared_y, gpu, dtype)
    got = ops.combine_norm_residual(pd, dev(inverse, gpu), wd, rd, dev(post, gpu), 1e-6, shared_y=sd)
    # the unfused sequence on the GPU: combine (bit-exact against the oracle) -> rmsnorm -> add
    plain = ops.combine(pd, dev(inverse, gpu), wd, sd)
    assert np.array_equal(host(plain), y)
    if dtype == "bf16":
        frac = tail_mismatch_fraction(host(got), want, normed)
        print(f"[parity] combine+norm+residual T={tokens} H={hidden}: elements that differ: {frac:.2e}", flush=True)
        assert frac <= 2e-3
    else:
        np.testing.assert_allclose(host(got), want, rtol=2e-6, atol=2e-6)


@pytest.mark.parametrize("name,tokens,top_k,dtype", [("C1", 256, 2, "f32"), ("C2", 512, 2, "bf16"), ("C3", 512, 8, "bf16")])
def test_block_forward_matches_oracle(gpu, name, tokens, top_k, dtype):
    inp = O.make_inputs(name, seed=0, tokens=tokens)
    cfg = inp["cfg"]
    T = inp["x"].shape[0] * inp["x"].shape[1]
    H = cfg["H"]
    x2 = inp["x"].reshape(T, H)
    rng = np.random.default_rng(9)
    pre = (1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    post = (0.25 + 0.05 * rng.standard_normal(H)).astype(np.float32)
    shared = None if inp["shared"] is None else tuple(dev(m, gpu, dtype) for m in inp["shared"])
    xd = dev(x2, gpu, dtype)
    got = ops.ffn_block_forward(xd, dev(pre, gpu), dev(post, gpu), 1e-6, dev(inp["w_router"], gpu, dtype),
                                dev(inp["expert_bias"], gpu), dev(inp["gate"], gpu, dtype), dev(inp["up"], gpu, dtype),
                                dev(inp["down"], gpu, dtype), top_k, 1.0, shared=shared)
    # staged, like the layer tests: the block equals its parts run one by one on the GPU ...
    normed = ops.rmsnorm(xd, dev(pre, gpu), 1e-6)
    inner = ops.moe_forward(normed, dev(inp["w_router"], gpu, dtype), dev(inp["expert_bias"], gpu),
                            dev(inp["gate"], gpu, dtype), dev(inp["up"], gpu, dtype), dev(inp["down"], gpu, dtype),
                            top_k, 1.0, shared=shared)
    assert torch.equal(inner.expert_ids, got.expert_ids) and torch.equal(inner.inverse, got.inverse)
    normed_y = O.rmsnorm(host(inner.y), post, 1e-6, dtype)
    tail = O.cast_compute(O.cast_compute(x2, dtype) + normed_y, dtype)
    # ... and the oracle's block on the kernel's own routing
    if dtype == "bf16":
        frac = tail_mismatch_fraction(host(got.y), tail, normed_y)
        print(f"[parity] block {name} T={T}: tail elements that differ: {frac:.2e}", flush=True)
        assert frac <= 2e-3
    else:
        np.testing.assert_allclose(host(got.y), tail, rtol=2e-6, atol=2e-6)
    want, ref_inner = O.ffn_block_forward(inp["x"], pre, post, 1e-6, inp["w_router"], inp["expert_bias"], inp["gate"],
                                          inp["up"], inp["down"], top_k, 1.0, dtype, inp["shared"])
    same_route = np.all(host(got.expert_ids) == ref_inner.route.expert_ids, axis=1)
    print(f"[parity] block {name}: tokens routed as the oracle routes them: {int(same_route.sum())}/{T}", flush=True)
    assert same_route.mean() >= 0.99
    rel = report(f"block {name} {dtype} (rows routed alike)", host(got.y)[same_route], want.reshape(T, H)[same_route])
    assert rel <= (BF16_MAX_REL if dtype == "bf16" else 1e-4)
