"""Pins the oracle's dispatch (histogram, offsets, stable permutation, inverse)."""

from __future__ import annotations

import numpy as np
import pytest

from oracle import moe_oracle as O


def closed_form_positions(flat: np.ndarray, num_experts: int) -> np.ndarray:
    """pos(a) = offsets[id_a] + #{a' < a : id_a' == id_a}, by plain loops."""
    counts = [0] * num_experts
    for v in flat:
        counts[int(v)] += 1
    offsets = [0] * num_experts
    for e in range(1, num_experts):
        offsets[e] = offsets[e - 1] + counts[e - 1]
    seen = [0] * num_experts
    pos = np.zeros(len(flat), dtype=np.int64)
    for a, v in enumerate(flat):
        pos[a] = offsets[int(v)] + seen[int(v)]
        seen[int(v)] += 1
    return pos


def check_invariants(ids: np.ndarray, num_experts: int, d: O.DispatchResult):
    flat = ids.reshape(-1)
    n = flat.size
    assert d.group_sizes.dtype == d.offsets.dtype == d.source_order.dtype == d.inverse.dtype == np.int32
    assert int(d.group_sizes.sum()) == n
    assert sorted(d.source_order.tolist()) == list(range(n))  # a bijection
    assert np.array_equal(d.inverse[d.source_order], np.arange(n))
    assert np.all(np.diff(flat[d.source_order]) >= 0)  # expert-major
    for e in range(num_experts):
        rows = d.source_order[d.offsets[e] : d.offsets[e] + d.group_sizes[e]]
        assert np.all(flat[rows] == e)
        assert np.all(np.diff(rows) > 0)  # stable: ascending assignment index inside a group
    assert np.array_equal(d.inverse, closed_form_positions(flat, num_experts))
    assert np.array_equal(d.offsets, np.concatenate([[0], np.cumsum(d.group_sizes)[:-1]]))


def test_reference_edge_patterns(kat):
    c = kat["edge_patterns"]
    x = np.asarray(c["x"], np.float32)
    for name, p in c["patterns"].items():
        ids = np.asarray(p["expert_ids"], np.int32)
        d = O.dispatch(ids, c["num_experts"], x)
        check_invariants(ids, c["num_experts"], d)
        assert np.array_equal(d.packed_x, x[d.source_order // ids.shape[1]])
        if name == "no_expert_three":
            assert d.group_sizes[3] == 0
        if name == "all_one_expert":
            assert d.group_sizes.tolist() == [ids.size, 0, 0, 0]
            assert np.array_equal(d.source_order, np.arange(ids.size))


@pytest.mark.parametrize("tokens,top_k,experts,seed", [(1, 1, 1, 0), (7, 3, 5, 1), (300, 8, 64, 2), (1025, 2, 128, 3)])
def test_random_ids(tokens, top_k, experts, seed):
    ids = np.random.default_rng(seed).integers(0, experts, size=(tokens, top_k)).astype(np.int32)
    check_invariants(ids, experts, O.dispatch(ids, experts))


def test_empty_and_out_of_range():
    d = O.dispatch(np.zeros((0, 2), np.int32), 4)
    assert d.group_sizes.tolist() == [0, 0, 0, 0] and d.source_order.size == 0
    with pytest.raises(ValueError):
        O.dispatch(np.array([[0, 4]], np.int32), 4)
