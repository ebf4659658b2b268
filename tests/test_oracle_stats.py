"""Pins the oracle's router statistics and sequence balance loss."""

from __future__ import annotations

import math

import numpy as np

from oracle import moe_oracle as O


def test_balance_loss_known_answer(kat):
    c = kat["balance_loss"]
    got = O.sequence_balance_loss(np.asarray(c["expert_ids"], np.int32), np.asarray(c["scores"], np.float32), c["top_k"])
    assert abs(float(got) - c["expected"]["loss"]) < 1e-6
    assert abs(float(got) - 0.975) < 1e-6


def test_stats_sums_and_closed_forms():
    # reference test_model.py:905-908: sum(counts) == B*S*K, sum(importance) ~= B*S*route_scale
    rng = np.random.default_rng(2)
    B, S, H, E, K = 2, 4, 8, 3, 2
    x = rng.standard_normal((B * S, H)).astype(np.float32)
    w = rng.standard_normal((H, E)).astype(np.float32)
    r = O.router(x, w, None, K, 1.0, "f32")
    s = O.router_stats(r.expert_ids, r.weights, E)
    assert float(s.expert_counts.sum()) == B * S * K
    assert abs(float(s.importance.sum()) - B * S) < 1e-2
    counts = [float(np.sum(r.expert_ids == e)) for e in range(E)]
    assert s.expert_counts.tolist() == counts
    total = sum(counts)
    mean = total / E
    assert float(s.total_assignments) == total
    assert float(s.load_min) == min(counts) and float(s.load_max) == max(counts)
    assert abs(float(s.load_mean) - mean) < 1e-6
    assert abs(float(s.max_vio) - (max(counts) - mean) / mean) < 1e-6
    ent = -sum(c / total * math.log(c / total) for c in counts if c > 0)
    assert abs(float(s.load_entropy) - ent) < 1e-6
    imp = [float(np.sum(np.where(r.expert_ids == e, r.weights, 0.0).astype(np.float64))) for e in range(E)]
    np.testing.assert_allclose(s.importance, imp, rtol=1e-6)


def test_stats_with_empty_expert():
    ids = np.array([[0, 1], [1, 0]], np.int32)
    s = O.router_stats(ids, np.full((2, 2), 0.5, np.float32), 4)
    assert s.expert_counts.tolist() == [2, 2, 0, 0]
    assert float(s.load_min) == 0 and float(s.max_vio) == 1.0
    assert abs(float(s.load_entropy) - math.log(2)) < 1e-6


def test_zipf_bias_properties():
    inp = O.make_inputs("C4", seed=0, tokens=2048)
    r = O.router(inp["x"][0], inp["w_router"], inp["expert_bias"], 8, 1.0, "bf16")
    counts = np.bincount(r.expert_ids.reshape(-1), minlength=128)
    assert int((counts == 0).sum()) >= 6  # the six disabled experts (and possibly more on a sample)
    top = np.sort(counts)[::-1]
    assert top[:26].sum() / counts.sum() > 0.55  # ~20 % of the experts carry most of the load
