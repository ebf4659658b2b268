"""Pins the oracle's SMEBU balancing update (the consumer of the layer's expert_counts).

The reference's own checks of steps/moe_balance.py run whole train steps
(tests/jaxtitan/test_train_step.py:352-418); what they assert about the update itself is restated
here on the update alone, next to a hand-computed case and the invariants the formula fixes.
"""

from __future__ import annotations

import math

import numpy as np
import pytest

from oracle import moe_oracle as O

SPEC = dict(load_lr=1e-2, momentum_factor=0.5, clamp=2.0)  # the reference test's policy (:356-366)


def test_two_expert_case_by_hand():
    # counts [3, 1]: mean 2, violation (2-3)/2 = -0.5 and (2-1)/2 = +0.5, delta = lr tanh(clamp v)
    # = -+ 0.01 tanh(1) (already centred), momentum' = 0.5 * 0 + 0.5 * delta
    counts = np.array([[3.0, 1.0]], np.float32)
    r = O.smebu_update(counts, np.zeros((1, 2), np.float32), np.array([[0.25, -0.5]], np.float32), **SPEC)
    step = 0.5 * 0.01 * math.tanh(1.0)
    np.testing.assert_allclose(r.momentum, [[-step, step]], rtol=1e-6)
    np.testing.assert_allclose(r.expert_bias, [[0.25 - step, -0.5 + step]], rtol=1e-6)
    assert abs(float(r.max_vio) - 0.5) < 1e-7 and float(r.load_min) == 1.0 and float(r.load_max) == 3.0
    ent = -(0.75 * math.log(0.75) + 0.25 * math.log(0.25))
    assert abs(float(r.load_entropy) - ent) < 1e-6
    assert abs(float(r.momentum_norm) - step * math.sqrt(2)) < 1e-8
    assert abs(float(r.bias_norm) - math.hypot(0.25 - step, -0.5 + step)) < 1e-6


def test_from_zero_state_bias_equals_momentum():
    # test_train_step.py:382-384
    rng = np.random.default_rng(0)
    counts = rng.integers(0, 50, size=(3, 8)).astype(np.float32)
    zeros = np.zeros_like(counts)
    r = O.smebu_update(counts, zeros, zeros, **SPEC)
    assert not np.allclose(r.momentum, 0.0)
    np.testing.assert_allclose(r.expert_bias, r.momentum, atol=1e-6)


def test_doubling_the_counts_changes_nothing():
    # test_train_step.py:414-418: two accumulated micro-batches of the same tokens (counts * 2)
    # give the momentum of one
    rng = np.random.default_rng(1)
    counts = rng.integers(1, 40, size=(2, 6)).astype(np.float32)
    m = rng.standard_normal(counts.shape).astype(np.float32) * 1e-3
    b = rng.standard_normal(counts.shape).astype(np.float32) * 1e-2
    one = O.smebu_update(counts, m, b, **SPEC)
    two = O.smebu_update(counts * 2, m, b, **SPEC)
    np.testing.assert_allclose(two.momentum, one.momentum, rtol=1e-6, atol=1e-9)
    assert float(two.max_vio) == pytest.approx(float(one.max_vio), rel=1e-6)


def test_balanced_counts_only_decay_the_momentum():
    counts = np.full((2, 5), 7.0, np.float32)
    m = np.arange(10, dtype=np.float32).reshape(2, 5) * 1e-3
    b = np.ones((2, 5), np.float32)
    r = O.smebu_update(counts, m, b, load_lr=5e-4, momentum_factor=0.75, clamp=2.0)
    np.testing.assert_allclose(r.momentum, 0.75 * m, rtol=1e-7)
    np.testing.assert_allclose(r.expert_bias, b + 0.75 * m, rtol=1e-7)
    assert float(r.max_vio) == 0.0 and abs(float(r.load_entropy) - math.log(5)) < 1e-6


def test_direction_centring_and_metrics():
    rng = np.random.default_rng(2)
    counts = rng.integers(0, 100, size=(4, 16)).astype(np.float32)
    counts[1, 3] = 0.0
    zeros = np.zeros_like(counts)
    r = O.smebu_update(counts, zeros, zeros, load_lr=5e-4, momentum_factor=0.5, clamp=2.0)
    # the centred deltas of a layer sum to zero, so from a zero state the momentum does too
    assert np.all(np.abs(r.momentum.sum(axis=1)) < 1e-8)
    for layer in range(4):
        mean = counts[layer].mean()
        # tanh is monotone: more load than another expert never means a larger step up
        order = np.argsort(counts[layer], kind="stable")
        assert np.all(np.diff(r.momentum[layer][order]) <= 1e-12)
        assert r.momentum[layer][np.argmax(counts[layer])] < 0 < r.momentum[layer][np.argmin(counts[layer])]
        assert abs(mean - counts[layer].sum() / 16) < 1e-4
    stats = [O.stats_from_counts(counts[layer], zeros[layer]) for layer in range(4)]
    assert float(r.max_vio) == max(float(s.max_vio) for s in stats)
    assert float(r.load_min) == 0.0 and float(r.load_max) == float(counts.max())
    assert abs(float(r.load_entropy) - np.mean([float(s.load_entropy) for s in stats])) < 1e-6
    assert abs(float(r.momentum_norm) - math.sqrt(float(np.sum(r.momentum.astype(np.float64) ** 2)))) < 1e-9
    # the step is bounded by load_lr whatever the counts
    assert np.all(np.abs(r.momentum) <= 0.5 * 2 * 5e-4 + 1e-9)


def test_all_counts_zero_is_a_no_op_on_direction():
    # mean 0: violation = (0 - 0) / 1e-6 = 0, so nothing moves and no metric is NaN
    counts = np.zeros((1, 4), np.float32)
    r = O.smebu_update(counts, np.zeros_like(counts), np.ones_like(counts), **SPEC)
    assert not r.momentum.any() and np.all(r.expert_bias == 1.0)
    assert float(r.max_vio) == 0.0 and float(r.load_entropy) == 0.0 and math.isfinite(float(r.bias_norm))


def test_shape_mismatch_is_refused():
    with pytest.raises(ValueError, match="router count shape must match MoE balance state"):
        O.smebu_update(np.zeros((2, 4), np.float32), np.zeros((1, 4), np.float32), np.zeros((2, 4), np.float32), **SPEC)
