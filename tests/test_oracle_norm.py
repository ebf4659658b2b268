"""Pins the oracle's RMSNorm: the reference's known-answer test, a float64 closed form, the
reference kernel boundary's multiplication order, and scale invariance."""

from __future__ import annotations

import numpy as np

from oracle import moe_oracle as O


def test_reference_known_answer():
    """tests/jaxtitan/test_kernels.py:192-204: x = [[1,2],[3,4]], weight = [0.5,1.5], eps = 0, bf16."""
    x = np.array([[[1.0, 2.0], [3.0, 4.0]]], np.float32)
    w = np.array([0.5, 1.5], np.float32)
    got = O.rmsnorm(x, w, 0.0, "bf16")
    rows = []
    for a, b in ((1.0, 2.0), (3.0, 4.0)):  # written out with scalar float64 arithmetic
        inv = 1.0 / np.sqrt((a * a + b * b) / 2.0)
        rows.append([a * inv * 0.5, b * inv * 1.5])
    want = O.bf16_round(np.array([rows], np.float32))
    assert got.shape == x.shape and got.dtype == np.float32
    np.testing.assert_array_equal(got, want)


def test_matches_float64_closed_form_and_the_other_multiplication_order():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((37, 1024)).astype(np.float32) * 3.0
    w = (1.0 + 0.1 * rng.standard_normal(1024)).astype(np.float32)
    eps = 1e-6
    x64 = x.astype(np.float64)
    want64 = x64 / np.sqrt(np.mean(x64 * x64, axis=-1, keepdims=True) + eps) * w
    got32 = O.rmsnorm(x, w, eps, "f32")
    np.testing.assert_allclose(got32, want64, rtol=3e-6, atol=1e-6)
    # bf16: inputs are rounded first, the result is the bf16 rounding of the exact value up to
    # results within an fp32 ulp of a rounding boundary
    xb = O.bf16_round(x).astype(np.float64)
    exact = xb / np.sqrt(np.mean(xb * xb, axis=-1, keepdims=True) + eps) * w
    gotb = O.rmsnorm(x, w, eps, "bf16")
    differs = gotb != O.bf16_round(exact.astype(np.float32))
    assert differs.mean() < 2e-3
    assert np.max(np.abs(gotb - exact)) <= np.max(np.abs(exact)) * 2.0 ** -8
    # rmsnorm_reference's order (kernels/rmsnorm.py:18-21): (x * inv_rms) * weight
    xf = O.bf16_round(x)
    inv = np.float32(1.0) / np.sqrt(np.sum(xf * xf, axis=-1, keepdims=True, dtype=np.float32) / np.float32(1024) + np.float32(eps))
    other = O.bf16_round((xf * inv) * w)
    assert (other != gotb).mean() < 2e-3


def test_scale_invariance_at_zero_eps():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((5, 64)).astype(np.float32)
    w = np.ones(64, np.float32)
    a = O.rmsnorm(x, w, 0.0, "f32")
    b = O.rmsnorm(4.0 * x, w, 0.0, "f32")  # a power of two: exact in floating point
    np.testing.assert_array_equal(a, b)
    np.testing.assert_allclose(np.mean(a.astype(np.float64) ** 2, axis=-1), 1.0, rtol=1e-6)


def test_block_forward_composes_norms_layer_and_residual():
    inp = O.make_inputs("C1", seed=3, tokens=16)
    H = inp["cfg"]["H"]
    rng = np.random.default_rng(2)
    pre = (1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    post = (0.5 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    out, inner = O.ffn_block_forward(inp["x"], pre, post, 1e-6, inp["w_router"], inp["expert_bias"], inp["gate"],
                                     inp["up"], inp["down"], 2, 1.0, "f32")
    normed = O.rmsnorm(inp["x"], pre, 1e-6, "f32")
    direct = O.moe_forward(normed, inp["w_router"], inp["expert_bias"], inp["gate"], inp["up"], inp["down"], 2, 1.0, "f32")
    np.testing.assert_array_equal(inner.y, direct.y)
    np.testing.assert_allclose(out, inp["x"] + O.rmsnorm(direct.y, post, 1e-6, "f32"), rtol=1e-6, atol=1e-6)
    # zero post scale: the block is the identity on x
    ident, _ = O.ffn_block_forward(inp["x"], pre, np.zeros(H, np.float32), 1e-6, inp["w_router"], inp["expert_bias"],
                                   inp["gate"], inp["up"], inp["down"], 2, 1.0, "f32")
    np.testing.assert_array_equal(ident, inp["x"].astype(np.float32))
