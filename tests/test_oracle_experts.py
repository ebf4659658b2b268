"""Pins the oracle's expert FFN, combine, shared experts and whole layer."""

from __future__ import annotations

import numpy as np
import pytest

from oracle import moe_oracle as O


def _arr(v, dtype=np.float32):
    return np.asarray(v, dtype=dtype)


def expert_major(x, ids, weights, gate, up, down, dtype, shared=None):
    d = O.dispatch(ids, gate.shape[0], O.cast_compute(x, dtype))
    packed_y = O.grouped_swiglu(d.packed_x, gate, up, down, d.group_sizes, dtype)
    return O.combine(packed_y, d.inverse, weights, dtype, shared)


@pytest.mark.parametrize("case", ["expert_swiglu_manual", "local_dispatcher", "dispatcher_equivalence"])
def test_expert_known_answers(kat, case):
    c = kat[case]
    x, ids, w = _arr(c["x"]), _arr(c["expert_ids"], np.int32), _arr(c["weights"])
    gate, up, down = _arr(c["gate"]), _arr(c["up"]), _arr(c["down"])
    want = _arr(c["expected"]["out"], np.float64)
    per_assignment = O.experts_per_assignment(x, ids, w, gate, up, down, "f32")
    grouped = expert_major(x, ids, w, gate, up, down, "f32")
    np.testing.assert_allclose(per_assignment, want, rtol=1e-5, atol=1e-5)
    # the reference's own invariant: expert-major == per-assignment at atol 1e-5 (test_model.py:373-418)
    np.testing.assert_allclose(grouped, per_assignment, rtol=1e-5, atol=1e-5)


def test_manual_case_value(kat):
    c = kat["expert_swiglu_manual"]
    out = O.experts_per_assignment(_arr(c["x"]), _arr(c["expert_ids"], np.int32), _arr(c["weights"]), _arr(c["gate"]),
                                   _arr(c["up"]), _arr(c["down"]), "f32")
    np.testing.assert_allclose(out, [[2.5315552, 3.388143]], rtol=1e-6)


@pytest.mark.parametrize("group", ["edge_patterns", "profile_bench"])
def test_edge_patterns_outputs(kat, group):
    c = kat[group]
    if group == "profile_bench":
        E, H, I, S = c["num_experts"], c["hidden"], c["inter"], c["seq"]
        gate = (np.arange(E * H * I, dtype=np.float32) / np.float32(4096.0)).reshape(E, H, I)
        up = gate[..., ::-1].copy()
        down = (np.arange(E * I * H, dtype=np.float32) / np.float32(4096.0)).reshape(E, I, H)
        x = (np.arange(S * H, dtype=np.float32) / np.float32(512.0)).reshape(S, H)
        w = np.full((S, c["top_k"]), 0.5, np.float32)
    else:
        gate, up, down, x, w = (_arr(c[k]) for k in ("gate", "up", "down", "x", "weights"))
    for name, p in c["patterns"].items():
        ids = _arr(p["expert_ids"], np.int32)
        got = expert_major(x, ids, w, gate, up, down, "f32")
        want = _arr(p["expected_out"], np.float64)
        np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-5, err_msg=name)
        assert np.array_equal(got, expert_major(x, ids, w, gate, up, down, "f32"))  # run twice: identical


def test_single_expert_reduces_to_matmul():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((33, 24)).astype(np.float32)
    gate, up = (rng.standard_normal((1, 24, 40)).astype(np.float32) * 0.2 for _ in range(2))
    down = rng.standard_normal((1, 40, 24)).astype(np.float32) * 0.2
    y = O.grouped_swiglu(x, gate, up, down, np.array([33], np.int32), "f32")
    g = x.astype(np.float64) @ gate[0].astype(np.float64)
    u = x.astype(np.float64) @ up[0].astype(np.float64)
    want = (g / (1 + np.exp(-g)) * u) @ down[0].astype(np.float64)
    np.testing.assert_allclose(y, want, rtol=1e-4, atol=1e-5)


def test_grouped_equals_per_assignment_bf16_and_stage_rounding():
    rng = np.random.default_rng(7)
    T, H, E, K, I = 40, 32, 6, 3, 48
    x = rng.standard_normal((T, H)).astype(np.float32)
    gate, up = (rng.standard_normal((E, H, I)).astype(np.float32) * 0.2 for _ in range(2))
    down = rng.standard_normal((E, I, H)).astype(np.float32) * 0.2
    ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
    w = O.bf16_round(rng.random((T, K)).astype(np.float32))
    a = O.experts_per_assignment(x, ids, w, gate, up, down, "bf16")
    b = expert_major(x, ids, w, gate, up, down, "bf16")
    assert np.array_equal(b, O.bf16_round(b))
    # same rounding points, same per-row dot products: only the BLAS blocking may differ
    np.testing.assert_allclose(a, b, rtol=2e-2, atol=2e-2)
    d = O.dispatch(ids, E, O.bf16_round(x))
    y, g, u, h = O.grouped_swiglu(d.packed_x, gate, up, down, d.group_sizes, "bf16", return_stages=True)
    for stage in (y, g, u, h):
        assert np.array_equal(stage, O.bf16_round(stage))


def test_combine_closed_form_and_token_permutation():
    rng = np.random.default_rng(11)
    T, K, H = 9, 3, 5
    packed_y = rng.standard_normal((T * K, H)).astype(np.float32)
    inverse = rng.permutation(T * K).astype(np.int32)
    w = rng.random((T, K)).astype(np.float32)
    out = O.combine(packed_y, inverse, w, "f32")
    for t in range(T):
        want = sum(packed_y[inverse[t * K + s]].astype(np.float64) * float(w[t, s]) for s in range(K))
        np.testing.assert_allclose(out[t], want, rtol=1e-6, atol=1e-6)
    shared = rng.standard_normal((T, H)).astype(np.float32)
    np.testing.assert_allclose(O.combine(packed_y, inverse, w, "f32", shared), out + shared, rtol=1e-6)


def test_shared_expert_added_unweighted():
    # reference test_model.py:873-884: zeroed routed experts => moe(x) == shared_experts(x)
    rng = np.random.default_rng(13)
    H, I = 16, 24
    x = np.ones((1, 1, H), np.float32)
    shared = tuple(rng.standard_normal(s).astype(np.float32) * 0.3 for s in ((H, I), (H, I), (I, H)))
    zeros = (np.zeros((1, H, I), np.float32), np.zeros((1, H, I), np.float32), np.zeros((1, I, H), np.float32))
    w_r = rng.standard_normal((H, 1)).astype(np.float32)
    r = O.moe_forward(x, w_r, None, *zeros, top_k=1, dtype="f32", shared=shared)
    np.testing.assert_allclose(r.y[0], O.shared_swiglu(x[0], *shared, "f32"), rtol=1e-6, atol=1e-7)
    g = x[0].astype(np.float64) @ shared[0]
    u = x[0].astype(np.float64) @ shared[1]
    np.testing.assert_allclose(r.y[0], (g / (1 + np.exp(-g)) * u) @ shared[2], rtol=1e-4, atol=1e-5)


def test_layer_is_per_token():
    # rows of a small batch equal the same rows inside a larger one (decode == prefill rows)
    inp = O.make_inputs("C1", seed=0, tokens=96)
    args = (inp["w_router"], inp["expert_bias"], inp["gate"], inp["up"], inp["down"])
    full = O.moe_forward(inp["x"], *args, top_k=2, dtype="f32")
    part = O.moe_forward(inp["x"][:, 17:29], *args, top_k=2, dtype="f32")
    np.testing.assert_allclose(part.y, full.y[:, 17:29], rtol=1e-5, atol=1e-6)
    assert np.array_equal(part.route.expert_ids, full.route.expert_ids[17:29])
