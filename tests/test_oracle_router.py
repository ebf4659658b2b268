"""Pins the oracle's router against the reference's known answers, a float64
closed form and brute force with deliberately tied scores."""

from __future__ import annotations

import itertools
import math

import numpy as np
import pytest

from oracle import moe_oracle as O


def test_bf16_round_matches_known_patterns():
    # exactly representable values are unchanged; ties go to even mantissa
    assert O.bf16_round(np.float32(1.0)) == 1.0
    assert O.bf16_round(np.float32(0.25)) == 0.25
    x = np.array([0x3F808000, 0x3F818000, 0x3F808001, 0x3F80FFFF], dtype=np.uint32).view(np.float32)
    got = O.bf16_bits(x)
    # 1.00390625 is a tie between 0x3F80 and 0x3F81 -> even (0x3F80); 0x3F818000 ties -> 0x3F82
    assert got.tolist() == [0x3F80, 0x3F82, 0x3F81, 0x3F81]
    # agrees with torch's bf16 conversion on random data
    torch = pytest.importorskip("torch")
    r = np.random.default_rng(0).standard_normal(100000).astype(np.float32) * 37.0
    ref = torch.from_numpy(r).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(O.bf16_round(r), ref)


def test_sigmoid_f32_is_within_3ulp_of_float64_and_monotone():
    z = np.concatenate([np.linspace(-40, 40, 400001), np.array([-1e4, -90, -86, 86, 90, 1e4, 0.0])]).astype(np.float32)
    got = O.sigmoid_f32(z)
    ref = 1.0 / (1.0 + np.exp(-np.clip(z.astype(np.float64), -86, 86)))
    ulp = np.spacing(ref.astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(got.astype(np.float64) - ref) / ulp) <= 3.0
    zs = np.sort(z)
    assert np.all(np.diff(O.sigmoid_f32(zs)) >= 0)
    assert got.dtype == np.float32 and np.all(got > 0) and np.all(got <= 1)


@pytest.mark.parametrize("case", ["router_order", "router_bias_scale"])
def test_router_known_answers(kat, case):
    c = kat[case]
    bias = None if c["expert_bias"] is None else np.asarray(c["expert_bias"], np.float32)
    r = O.router(np.asarray(c["x"], np.float32), np.asarray(c["w_router"], np.float32), bias, c["top_k"],
                 c["route_scale"], "f32")
    assert r.expert_ids.dtype == np.int32
    assert r.expert_ids.tolist() == c["expected"]["ids"]
    np.testing.assert_allclose(r.weights, np.asarray(c["expected"]["weights"]), rtol=2e-6)
    np.testing.assert_allclose(r.scores, np.asarray(c["expected"]["scores"]), rtol=2e-6)
    np.testing.assert_allclose(r.weights.sum(-1), c["asserted"]["weight_sum"], rtol=1e-6)
    assert np.all(r.weights > 0)
    if "ids_token0" in c["asserted"]:
        assert r.expert_ids[0].tolist() == c["asserted"]["ids_token0"]
    again = O.router(np.asarray(c["x"], np.float32), np.asarray(c["w_router"], np.float32), bias, c["top_k"],
                     c["route_scale"], "f32")
    assert np.array_equal(again.expert_ids, r.expert_ids) and np.array_equal(again.weights, r.weights)


def test_bias_changes_selection_not_weights():
    logits = np.array([[2.0, 0.0, -2.0, 1.0]], np.float32)
    plain = O.router_from_logits(logits, None, 2, 1.0, "f32")
    biased = O.router_from_logits(logits, np.array([0, 0, 5.0, 0], np.float32), 2, 1.0, "f32")
    assert plain.expert_ids.tolist() == [[0, 3]]
    assert biased.expert_ids.tolist() == [[2, 0]]
    s = [1 / (1 + math.exp(-v)) for v in (2.0, 0.0, -2.0, 1.0)]
    np.testing.assert_allclose(biased.weights[0], [s[2] / (s[2] + s[0]), s[0] / (s[2] + s[0])], rtol=2e-6)


def test_top_k_ties_go_to_lower_index_brute_force():
    # every arrangement of a small multiset with repeated values
    values = [0.5, 0.5, 0.25, 0.75, 0.5]
    for perm in set(itertools.permutations(values)):
        v = np.asarray([perm], dtype=np.float32)
        for k in range(1, 6):
            got = O.top_k_desc(v, k)[0].tolist()
            want = sorted(range(5), key=lambda i: (-perm[i], i))[:k]
            assert got == want
    # saturated logits give equal scores: the index rule decides
    logits = np.array([[30.0, 40.0, 50.0, -3.0]], np.float32)
    r = O.router_from_logits(logits, None, 2, 1.0, "f32")
    assert r.scores[0, 0] == r.scores[0, 1] == r.scores[0, 2] == 1.0
    assert r.expert_ids.tolist() == [[0, 1]]


def test_router_invariants_random_bf16():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((257, 64)).astype(np.float32)
    w = (rng.standard_normal((64, 16)) * 0.2).astype(np.float32)
    r = O.router(x, w, None, 4, 2.5, "bf16")
    assert np.array_equal(r.logits, O.bf16_round(r.logits))
    assert np.array_equal(r.weights, O.bf16_round(r.weights))
    sel = np.take_along_axis(r.scores, r.expert_ids.astype(np.int64), axis=-1)
    assert np.all(np.diff(sel, axis=-1) <= 0)  # descending
    assert all(len(set(row)) == 4 for row in r.expert_ids.tolist())  # distinct
    rest = r.scores.copy()
    np.put_along_axis(rest, r.expert_ids.astype(np.int64), -1.0, axis=-1)
    assert np.all(rest.max(-1) <= sel[:, -1])  # nothing unselected beats the k-th
    np.testing.assert_allclose(r.weights.sum(-1), 2.5, rtol=2e-2)


def test_softmax_scores_against_float64_closed_forms():
    """The softmax score function is not a reference path (moe.py:133 is a sigmoid): it is pinned by what
    the definition fixes."""
    rng = np.random.default_rng(11)
    for experts in (3, 5, 16, 64, 130, 256):
        z = (rng.standard_normal((40, experts)) * 4.0).astype(np.float32)
        z[0, :] = 1.25            # all equal: exactly uniform up to the rounding of one division
        z[1, :] = -200.0
        z[1, experts // 2] = 50.0  # one dominant logit: everything else is clamped at exp(-86)
        s = O.softmax_f32(z)
        z64 = z.astype(np.float64)
        ref = np.exp(z64 - z64.max(-1, keepdims=True))
        ref /= ref.sum(-1, keepdims=True)
        big = ref > 1e-30
        np.testing.assert_allclose(s[big], ref[big], rtol=3e-6)
        assert np.all(s[~big] < 1e-30)
        np.testing.assert_allclose(s.sum(-1), 1.0, rtol=1e-6)
        np.testing.assert_allclose(s[0], 1.0 / experts, rtol=3e-7)
        assert s[1, experts // 2] == 1.0
        # order-preserving: a larger logit never gets a smaller score
        order = np.argsort(z[2])
        assert np.all(np.diff(s[2][order]) >= 0)
    # adding a constant to a row that keeps the differences exact does not change anything
    z = np.array([[0.5, -1.25, 3.0, 2.0]], np.float32)
    assert np.array_equal(O.softmax_f32(z), O.softmax_f32(z + np.float32(8.0)))


def test_softmax_router_selection_and_weights():
    logits = np.array([[2.0, 0.0, -2.0, 1.0]], np.float32)
    r = O.router_from_logits(logits, None, 2, 1.5, "f32", "softmax")
    assert r.expert_ids.tolist() == [[0, 3]]
    e = [math.exp(v) for v in (2.0, 0.0, -2.0, 1.0)]
    s = [v / sum(e) for v in e]
    np.testing.assert_allclose(r.scores[0], s, rtol=2e-6)
    np.testing.assert_allclose(r.weights[0], [1.5 * s[0] / (s[0] + s[3]), 1.5 * s[3] / (s[0] + s[3])], rtol=2e-6)
    # the bias enters the selection only, ties go to the lower index, as with the sigmoid
    biased = O.router_from_logits(logits, np.array([0, 0, 5.0, 0], np.float32), 2, 1.0, "f32", "softmax")
    assert biased.expert_ids.tolist() == [[2, 0]]
    tied = O.router_from_logits(np.zeros((1, 6), np.float32), None, 3, 1.0, "f32", "softmax")
    assert tied.expert_ids.tolist() == [[0, 1, 2]]
    with pytest.raises(ValueError):
        O.router_from_logits(logits, None, 2, 1.0, "f32", "tanh")


def test_router_argument_errors():
    logits = np.zeros((2, 4), np.float32)
    with pytest.raises(ValueError):
        O.router_from_logits(logits, None, 5, 1.0, "f32")
    with pytest.raises(ValueError):
        O.router_from_logits(logits, None, 0, 1.0, "f32")
    with pytest.raises(ValueError):
        O.router_from_logits(logits, None, 2, 0.0, "f32")
    with pytest.raises(ValueError):
        O.router_from_logits(logits, np.zeros(3, np.float32), 2, 1.0, "f32")
