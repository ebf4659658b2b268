"""Write tests/golden/kat.json: the known-answer cases of the reference's own tests.

Inputs are transcribed from vpareek2/research tests/jaxtitan/test_model.py (the
line ranges are recorded with each case).  Expected values are what those tests
assert, evaluated here with scalar float64 arithmetic from Python's ``math``
module only -- no NumPy, no oracle code -- so that the fixture is independent of
the code it checks.  Run:  python tests/golden/make_kat.py
"""

from __future__ import annotations

import json
import math
from pathlib import Path


def sigmoid(z: float) -> float:
    return 1.0 / (1.0 + math.exp(-z))


def silu(z: float) -> float:
    return z * sigmoid(z)


def matvec(x: list[float], w: list[list[float]]) -> list[float]:
    """x [H] times w [H][N]."""
    return [sum(x[h] * w[h][n] for h in range(len(x))) for n in range(len(w[0]))]


def top_k(values: list[float], k: int) -> list[int]:
    """Descending, equal values -> lower index first."""
    order = sorted(range(len(values)), key=lambda i: (-values[i], i))
    return order[:k]


def route(x, w, bias, k, scale):
    ids, weights, scores = [], [], []
    for row in x:
        s = [sigmoid(z) for z in matvec(row, w)]
        sel = top_k([s[e] + bias[e] for e in range(len(s))], k)
        denom = sum(s[e] for e in sel) + 1e-20
        ids.append(sel)
        weights.append([s[e] / denom * scale for e in sel])
        scores.append(s)
    return ids, weights, scores


def expert_out(x, e, gate, up, down):
    g = matvec(x, gate[e])
    u = matvec(x, up[e])
    h = [silu(g[i]) * u[i] for i in range(len(g))]
    return matvec(h, down[e])


def experts(x, ids, weights, gate, up, down):
    out = []
    for t, row in enumerate(x):
        acc = [0.0] * len(row)
        for s, e in enumerate(ids[t]):
            y = expert_out(row, e, gate, up, down)
            acc = [acc[h] + y[h] * weights[t][s] for h in range(len(row))]
        out.append(acc)
    return out


def arange(n: int, div: float, start: int = 0) -> list[float]:
    return [(start + i) / div for i in range(n)]


def reshape(flat: list[float], *shape: int):
    if len(shape) == 1:
        return list(flat)
    step = len(flat) // shape[0]
    return [reshape(flat[i * step : (i + 1) * step], *shape[1:]) for i in range(shape[0])]


def main() -> None:
    cases = {}

    # test_model.py:196-214  router is deterministic, ordered, normalised
    w = [[0.0, 1.0, 2.0], [0.0, 0.0, 0.0]]
    x = [[1.0, 0.0], [0.5, 0.0]]
    ids, weights, scores = route(x, w, [0.0] * 3, 2, 1.0)
    cases["router_order"] = dict(
        source="tests/jaxtitan/test_model.py:196-214",
        w_router=w, x=x, top_k=2, route_scale=1.0, expert_bias=None,
        asserted=dict(ids_token0=[2, 1], weight_sum=1.0, weights_positive=True),
        expected=dict(ids=ids, weights=weights, scores=scores),
    )

    # test_model.py:217-239  bias for selection only, route_scale
    w = [[2.0, 0.0, -2.0], [0.0, 0.0, 0.0]]
    x = [[1.0, 0.0]]
    bias = [0.0, 0.0, 1.0]
    ids, weights, scores = route(x, w, bias, 2, 1.5)
    cases["router_bias_scale"] = dict(
        source="tests/jaxtitan/test_model.py:217-239",
        w_router=w, x=x, top_k=2, route_scale=1.5, expert_bias=bias,
        asserted=dict(ids=[[2, 0]], weight_sum=1.5),
        expected=dict(ids=ids, weights=weights, scores=scores),
    )

    # test_model.py:242-252  sequence balance loss
    b_ids = [[[0, 1], [1, 2]]]
    b_scores = [[[0.2, 0.5, 0.3], [0.4, 0.1, 0.5]]]
    counts = [1.0, 2.0, 1.0]
    f_i = [3.0 / (2 * 2) * c for c in counts]
    norm = [[v / sum(row) for v in row] for row in b_scores[0]]
    p_i = [(norm[0][e] + norm[1][e]) / 2.0 for e in range(3)]
    cases["balance_loss"] = dict(
        source="tests/jaxtitan/test_model.py:242-252",
        expert_ids=b_ids, scores=b_scores, top_k=2,
        expected=dict(loss=sum(f_i[e] * p_i[e] for e in range(3))),
    )

    # test_model.py:255-299  expert SwiGLU, manual selected-expert calculation
    gate = [[[1.0, 0.0], [0.0, 1.0]], [[0.5, 0.0], [0.0, 0.5]]]
    up = [[[1.0, 1.0], [1.0, 1.0]], [[2.0, 0.0], [0.0, 2.0]]]
    down = [[[1.0, 0.0], [0.0, 1.0]], [[1.0, 1.0], [1.0, -1.0]]]
    x = [[1.0, 2.0]]
    e_ids = [[1, 0]]
    e_w = [[0.25, 0.75]]
    cases["expert_swiglu_manual"] = dict(
        source="tests/jaxtitan/test_model.py:255-299",
        gate=gate, up=up, down=down, x=x, expert_ids=e_ids, weights=e_w,
        expected=dict(out=experts(x, e_ids, e_w, gate, up, down)),
    )

    # test_model.py:302-322  local dispatcher == experts (arange/8 weights)
    gate = reshape(arange(8, 8.0), 2, 2, 2)
    up = reshape(arange(8, 8.0, 8), 2, 2, 2)
    down = reshape(arange(8, 8.0, 16), 2, 2, 2)
    x = [[1.0, 2.0], [3.0, 4.0]]
    e_ids = [[1, 0], [0, 1]]
    e_w = [[0.25, 0.75], [0.6, 0.4]]
    cases["local_dispatcher"] = dict(
        source="tests/jaxtitan/test_model.py:302-322",
        gate=gate, up=up, down=down, x=x, expert_ids=e_ids, weights=e_w,
        expected=dict(out=experts(x, e_ids, e_w, gate, up, down)),
    )

    # test_model.py:325-418  E=4,H=3,I=5 dispatcher equivalence inputs
    gate = reshape(arange(60, 37.0), 4, 3, 5)
    up = reshape(arange(60, 41.0), 4, 3, 5)[::-1]
    down = reshape(arange(60, 43.0), 4, 5, 3)
    x = reshape(arange(24, 17.0), 8, 3)  # [2,4,3] flattened over batch, seq
    e_ids = [[0, 1], [2, 3], [1, 3], [0, 2], [3, 1], [0, 2], [2, 1], [3, 0]]
    e_w = [[0.25, 0.75], [0.5, 0.5], [0.4, 0.6], [0.2, 0.8], [0.55, 0.45], [0.3, 0.7], [0.65, 0.35], [0.1, 0.9]]
    cases["dispatcher_equivalence"] = dict(
        source="tests/jaxtitan/test_model.py:325-418",
        batch=2, seq=4,
        gate=gate, up=up, down=down, x=x, expert_ids=e_ids, weights=e_w,
        expected=dict(out=experts(x, e_ids, e_w, gate, up, down)),
    )

    # test_model.py:532-691  edge-case id patterns (E=4,H=3,I=4,S=6,K=2, batch 1)
    num_experts, hidden, inter, seq_len, k = 4, 3, 4, 6, 2
    gate = reshape(arange(num_experts * hidden * inter, 37.0), num_experts, hidden, inter)
    up = [[[v / 1.3 for v in row[::-1]] for row in mat] for mat in gate]
    down = reshape(arange(num_experts * inter * hidden, 43.0), num_experts, inter, hidden)
    x = reshape(arange(seq_len * hidden, 17.0), seq_len, hidden)
    e_w = [[0.3, 0.7] for _ in range(seq_len)]
    balanced = [[(t * k + s) % num_experts for s in range(k)] for t in range(seq_len)]
    patterns = dict(
        balanced=balanced,
        no_expert_three=[[v % 3 for v in row] for row in balanced],
        all_one_expert=[[0, 0] for _ in range(seq_len)],
        duplicate_routes=[[t % num_experts] * k for t in range(seq_len)],
    )
    cases["edge_patterns"] = dict(
        source="tests/jaxtitan/test_model.py:532-691",
        gate=gate, up=up, down=down, x=x, weights=e_w, num_experts=num_experts,
        patterns={
            name: dict(expert_ids=ids_p, expected_out=experts(x, ids_p, e_w, gate, up, down))
            for name, ids_p in patterns.items()
        },
    )

    # src/jaxtitan/runtime/profile_bench.py:138-162  the reference micro-benchmark's inputs
    hidden, inter, num_experts, seq_len, k = 32, 64, 4, 16, 2
    gate = reshape(arange(num_experts * hidden * inter, 4096.0), num_experts, hidden, inter)
    up = [[row[::-1] for row in mat] for mat in gate]
    down = reshape(arange(num_experts * inter * hidden, 4096.0), num_experts, inter, hidden)
    x = reshape(arange(seq_len * hidden, 512.0), seq_len, hidden)
    e_w = [[0.5, 0.5] for _ in range(seq_len)]
    balanced = [[(t * k + s) % num_experts for s in range(k)] for t in range(seq_len)]
    skewed = [[0, 0] for _ in range(seq_len)]
    cases["profile_bench"] = dict(
        source="src/jaxtitan/runtime/profile_bench.py:138-162",
        # inputs are arange formulas; the test rebuilds them instead of storing 24k numbers:
        # gate = arange(E*H*I)/4096 as [E,H,I]; up = flip(gate, last axis); down = arange(E*I*H)/4096 as [E,I,H];
        # x = arange(S*H)/512 as [S,H]; weights = 0.5
        hidden=hidden, inter=inter, num_experts=num_experts, seq=seq_len, top_k=k,
        patterns=dict(
            balanced=dict(expert_ids=balanced, expected_out=experts(x, balanced, e_w, gate, up, down)),
            skewed=dict(expert_ids=skewed, expected_out=experts(x, skewed, e_w, gate, up, down)),
        ),
    )

    path = Path(__file__).with_name("kat.json")
    path.write_text(json.dumps(cases) + "\n")
    print(f"wrote {path} ({path.stat().st_size} bytes, {len(cases)} cases)")


if __name__ == "__main__":
    main()
