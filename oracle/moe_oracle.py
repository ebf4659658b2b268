"""CPU oracle for the MoE expert-layer forward.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only ``tests/``, the smoke
entry and the ``cpu_baseline`` leg of the benchmark may import it.  It restates,
in NumPy, the algorithm of the reference layer
(``src/jaxtitan/models/components/moe.py`` in vpareek2/research):

* ``router``            <- ``SigmoidTopKRouter.__call__``        moe.py:131-147
* ``experts_per_assignment`` <- ``ExpertSwiGLU.local_forward/__call__`` moe.py:174-195
* ``dispatch``          <- ``local_dispatch`` (ep_size == 1)     moe.py:583-602
* ``grouped_swiglu``    <- the three ``ragged_dot`` calls        moe.py:638-641
* ``combine``           <- unpermute / weight / reduce           moe.py:663-671
* ``shared_swiglu``     <- ``SharedSwiGLU.__call__``             moe.py:361-364
* ``router_stats``      <- ``_router_stats``                     moe.py:794-825
* ``sequence_balance_loss`` <- ``_sequence_balance_loss``        moe.py:828-840
* ``moe_forward``       <- ``SparseMoE.forward_with_output``     moe.py:418-446
* ``smebu_update``      <- ``apply_moe_balance_update``          steps/moe_balance.py:97-162, 174-184
* ``rmsnorm`` / ``ffn_block_forward`` <- the block around the layer  blocks.py:224-230, norm.py:12-31

The arithmetic the reference delegates to jax 0.10.0 / jaxlib 0.10.0 (pinned
in the reference's ``uv.lock``; absent from this environment) is restated from
its published contract: ``lax.top_k`` returns values in descending order with
equal elements ordered by lower index first; ``argsort(stable=True)`` is a
stable ascending sort; ``ragged_dot(lhs, rhs, group_sizes)`` multiplies the
rows of consecutive groups by ``rhs[g]``; ``nn.sigmoid(z) = 1/(1+exp(-z))``;
``nn.silu(z) = z * sigmoid(z)``.

Compute dtypes: ``"f32"`` and ``"bf16"``.  bf16 is emulated on float32 arrays
with round-to-nearest-even (``bf16_round``); the rounding points are those of
the reference with bf16 compute (every dot has a bf16 result accumulated in
fp32; route weights are cast to bf16; the sum over k accumulates in fp32 and
rounds once).  One choice is not fixed by the reference and is made here: the
elementwise chain ``silu(g) * u`` is evaluated in fp32 on the bf16 values of
``g`` and ``u`` and rounded once.

Parity status of each function (what pins it is exercised in
``tests/test_oracle_*.py``):

* router: pinned by the reference's known-answer tests
  (tests/jaxtitan/test_model.py:196-239), a float64 closed form, and brute-force
  top-k with deliberately tied scores.
* top-k behaviour on NaN / Inf scores: PARITY UNPINNED (nothing in the
  reference's tests reaches it; inputs of every configuration are finite).
* the softmax score function (``softmax_f32``, ``score_func="softmax"``): PARITY UNPINNED
  against the reference, which has no such router; pinned by float64 closed forms only.
* dispatch: pinned by ``np.bincount`` / ``np.cumsum`` / stable ``np.argsort``, a
  closed-form rank, permutation invariants and the reference's edge patterns
  (test_model.py:580-587).
* experts / grouped_swiglu / combine: pinned by the reference's known-answer
  tests (test_model.py:255-418), by the reference's own invariant
  "expert-major == per-assignment" and by the one-expert special case that
  reduces to a plain matmul.
* shared_swiglu: pinned by test_model.py:873-884 (zeroed routed experts).
* router_stats / sequence_balance_loss: pinned by test_model.py:242-252 and
  :905-908 and closed forms.
* smebu_update: pinned by a hand-computed two-expert case in float64, the reference's two
  train-step properties (tests/jaxtitan/test_train_step.py:352-388: from a zero state the updated
  bias equals the momentum and is non-zero; :391-418: doubling every count leaves the momentum
  unchanged), and invariants (balanced counts give a pure momentum decay; the centred deltas sum to
  zero; overloaded experts move down, underloaded ones up; the metrics equal the router
  statistics of each layer).
* rmsnorm: pinned by the reference's known-answer test (tests/jaxtitan/test_kernels.py:192-204),
  a float64 closed form and the scale-invariance property rmsnorm(c x) = rmsnorm(x) at eps = 0.
  Which of two equally valid fp32 multiplication orders flax uses: PARITY UNPINNED at the
  last-ulp level (flax is absent; nothing in the reference's tests distinguishes them).

The scores use a fully specified fp32 sigmoid (``sigmoid_f32``) built only
from IEEE-754 add, multiply, divide, round-to-integer and power-of-two scaling,
each rounded separately, so that a GPU kernel can reproduce the routing
decision bit for bit from the same logits.  It agrees with the mathematical
sigmoid to about 2 ulp, which ``tests/test_oracle_router.py`` checks.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np

F32 = np.float32


# --------------------------------------------------------------------------
# bf16 emulation
# --------------------------------------------------------------------------
def bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> uint16 bf16 bit pattern, round-to-nearest-even (NaN kept quiet)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    rounded = (u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))) >> np.uint32(16)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    rounded = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x0040), rounded)
    return rounded.astype(np.uint16)


def bf16_from_bits(b: np.ndarray) -> np.ndarray:
    """uint16 bf16 bit pattern -> float32."""
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round float32 values to the nearest bf16 value, returned as float32."""
    return bf16_from_bits(bf16_bits(x))


def cast_compute(x: np.ndarray, dtype: str) -> np.ndarray:
    """Cast to the compute dtype (held in float32 storage)."""
    x = np.asarray(x, dtype=np.float32)
    if dtype == "bf16":
        return bf16_round(x)
    if dtype == "f32":
        return x
    raise ValueError(f"unsupported compute dtype {dtype!r}")


# --------------------------------------------------------------------------
# fully specified fp32 sigmoid
# --------------------------------------------------------------------------
_LOG2E = F32(1.4426950408889634)
_LN2_HI = F32(0.693145751953125)  # 0x3f317200, low mantissa bits zero: n*_LN2_HI is exact
_LN2_LO = F32(1.428606765330187e-06)
_EXP_POLY = tuple(
    F32(c)
    for c in (
        1.9875691500e-4,
        1.3981999507e-3,
        8.3334519073e-3,
        4.1665795894e-2,
        1.6666665459e-1,
        5.0000001201e-1,
    )
)
_EXP_CLAMP = F32(86.0)


def exp_f32(x: np.ndarray) -> np.ndarray:
    """exp(x) for float32 x in [-86, 86] by a fixed sequence of fp32 operations.

    n = rint(x*log2e); r = (x - n*ln2_hi) - n*ln2_lo;
    p = Horner(r) with separately rounded multiply and add; result = p * 2**n.
    """
    x = np.asarray(x, dtype=np.float32)
    n = np.rint(x * _LOG2E).astype(np.float32)
    r = (x - n * _LN2_HI) - n * _LN2_LO
    p = np.full_like(r, _EXP_POLY[0])
    for c in _EXP_POLY[1:]:
        p = p * r + c
    rr = r * r
    p = p * rr
    p = p + r
    p = p + F32(1.0)
    return np.ldexp(p, n.astype(np.int32)).astype(np.float32)


def sigmoid_f32(z: np.ndarray) -> np.ndarray:
    """1 / (1 + exp(-z)) in float32 with the fixed operation order above."""
    z = np.asarray(z, dtype=np.float32)
    t = np.minimum(np.maximum(-z, -_EXP_CLAMP), _EXP_CLAMP)
    e = exp_f32(t)
    return (F32(1.0) / (F32(1.0) + e)).astype(np.float32)


def softmax_f32(logits: np.ndarray) -> np.ndarray:
    """softmax over the last axis in float32 by a fixed sequence of operations.

    The reference has no softmax router (moe.py:133 is a sigmoid); the benchmark's second
    configuration names one, so it is offered as a score function of the same router and restated
    here only from its definition: m = max_e z_e;  p_e = exp(max(z_e - m, -86));  the p_e are added
    in four runs of ceil(E/4) consecutive experts, each run in index order, the four run sums as
    (s0 + s1) + (s2 + s3);  score_e = p_e / sum.  PARITY UNPINNED against any reference
    implementation; pinned here by float64 closed forms (tests/test_oracle_router.py).
    """
    z = np.asarray(logits, dtype=np.float32)
    num_experts = z.shape[-1]
    m = np.max(z, axis=-1, keepdims=True)
    p = exp_f32(np.maximum(z - m, -_EXP_CLAMP))
    run = (num_experts + 3) // 4
    sums = []
    for q in range(4):
        acc = np.zeros(z.shape[:-1], dtype=np.float32)
        for e in range(q * run, min(num_experts, (q + 1) * run)):
            acc = acc + p[..., e]
        sums.append(acc)
    total = (sums[0] + sums[1]) + (sums[2] + sums[3])
    return (p / total[..., None]).astype(np.float32)


SCORE_FUNCS = ("sigmoid", "softmax")


def silu_f32(z: np.ndarray) -> np.ndarray:
    """z * sigmoid(z) in float32 (plain libm exp; outputs are tolerance-checked)."""
    z = np.asarray(z, dtype=np.float32)
    return (z / (F32(1.0) + np.exp(-z, dtype=np.float32))).astype(np.float32)


# --------------------------------------------------------------------------
# router  (moe.py:131-147)
# --------------------------------------------------------------------------
@dataclass
class RouterResult:
    expert_ids: np.ndarray  # [T, K] int32
    weights: np.ndarray  # [T, K] float32 storage, values in the compute dtype
    scores: np.ndarray  # [T, E] float32
    logits: np.ndarray  # [T, E] float32 (after the compute-dtype rounding)


def router_logits(x: np.ndarray, w_router: np.ndarray, dtype: str) -> np.ndarray:
    """Linear without bias in the compute dtype, upcast to fp32 (moe.py:132)."""
    xc = cast_compute(x, dtype)
    wc = cast_compute(w_router, dtype)
    logits = np.matmul(xc, wc, dtype=np.float32)
    return cast_compute(logits, dtype)


def top_k_desc(values: np.ndarray, k: int) -> np.ndarray:
    """Indices of the k largest entries per row, descending, ties -> lower index."""
    order = np.argsort(-values, axis=-1, kind="stable")
    return order[..., :k].astype(np.int32)


def router_from_logits(
    logits: np.ndarray,
    expert_bias: np.ndarray | None,
    top_k: int,
    route_scale: float,
    dtype: str,
    score_func: str = "sigmoid",
) -> RouterResult:
    """Everything after the projection (moe.py:133-147).  score_func "softmax" replaces the sigmoid of
    moe.py:133 by softmax_f32 and leaves the rest as it is (not a reference path)."""
    logits = np.asarray(logits, dtype=np.float32)
    num_experts = logits.shape[-1]
    if top_k <= 0 or top_k > num_experts:
        raise ValueError("router top_k must be positive and <= num_experts")
    if route_scale <= 0.0:
        raise ValueError("router route_scale must be positive")
    if score_func not in SCORE_FUNCS:
        raise ValueError(f"router score_func must be one of {SCORE_FUNCS}")
    scores = sigmoid_f32(logits) if score_func == "sigmoid" else softmax_f32(logits)
    if expert_bias is None:
        expert_bias = np.zeros((num_experts,), dtype=np.float32)
    expert_bias = np.asarray(expert_bias, dtype=np.float32)
    if expert_bias.shape != (num_experts,):
        raise ValueError(f"expert_bias must have shape [{num_experts}]")
    ids = top_k_desc(scores + expert_bias, top_k)
    top = np.take_along_axis(scores, ids.astype(np.int64), axis=-1)
    denom = top[..., 0].copy()
    for s in range(1, top_k):  # sequential fp32 sum in slot order
        denom = denom + top[..., s]
    denom = denom + F32(1e-20)
    weights = (top / denom[..., None]) * F32(route_scale)
    return RouterResult(
        expert_ids=ids,
        weights=cast_compute(weights.astype(np.float32), dtype),
        scores=scores,
        logits=logits,
    )


def router(
    x: np.ndarray,
    w_router: np.ndarray,
    expert_bias: np.ndarray | None,
    top_k: int,
    route_scale: float = 1.0,
    dtype: str = "f32",
    score_func: str = "sigmoid",
) -> RouterResult:
    """x [T,H], w_router [H,E] -> ids, weights, scores."""
    return router_from_logits(router_logits(x, w_router, dtype), expert_bias, top_k, route_scale, dtype, score_func)


# --------------------------------------------------------------------------
# dispatch  (moe.py:583-602 with ep_size == 1)
# --------------------------------------------------------------------------
@dataclass
class DispatchResult:
    group_sizes: np.ndarray  # [E] int32   (send_sizes)
    offsets: np.ndarray  # [E] int32   (input_offsets, exclusive prefix sum)
    source_order: np.ndarray  # [A] int32   assignment occupying packed row j
    inverse: np.ndarray  # [A] int32   packed row of assignment a
    packed_x: np.ndarray | None  # [A, H]      x[source_order // K]


def dispatch(expert_ids: np.ndarray, num_experts: int, x: np.ndarray | None = None) -> DispatchResult:
    """expert_ids [T,K] (any ints in [0,E)); flatten order a = t*K + s."""
    ids = np.asarray(expert_ids)
    top_k = ids.shape[-1]
    flat = ids.reshape(-1).astype(np.int64)
    if flat.size and (flat.min() < 0 or flat.max() >= num_experts):
        raise ValueError("expert id out of range")
    source_order = np.argsort(flat, kind="stable").astype(np.int32)
    inverse = np.argsort(source_order, kind="stable").astype(np.int32)
    group_sizes = np.bincount(flat, minlength=num_experts).astype(np.int32)
    offsets = (np.cumsum(group_sizes, dtype=np.int64) - group_sizes).astype(np.int32)
    packed_x = None
    if x is not None:
        x2 = np.asarray(x).reshape(-1, np.asarray(x).shape[-1])
        packed_x = x2[source_order // top_k]
    return DispatchResult(group_sizes, offsets, source_order, inverse, packed_x)


# --------------------------------------------------------------------------
# experts
# --------------------------------------------------------------------------
def _swiglu_act(g: np.ndarray, u: np.ndarray, dtype: str) -> np.ndarray:
    return cast_compute(silu_f32(g) * u, dtype)


def grouped_swiglu(
    packed_x: np.ndarray,
    gate: np.ndarray,
    up: np.ndarray,
    down: np.ndarray,
    group_sizes: np.ndarray,
    dtype: str,
    return_stages: bool = False,
):
    """Three grouped matmuls over contiguous row groups (moe.py:638-641).

    packed_x [A,H]; gate, up [E,H,I]; down [E,I,H]; rows
    offsets[e] .. offsets[e]+group_sizes[e]-1 use expert e.  Returns packed_y [A,H].
    """
    xc = cast_compute(packed_x, dtype)
    num_experts, hidden, inter = gate.shape
    rows = xc.shape[0]
    gate_x = np.zeros((rows, inter), dtype=np.float32)
    up_x = np.zeros((rows, inter), dtype=np.float32)
    act = np.zeros((rows, inter), dtype=np.float32)
    packed_y = np.zeros((rows, hidden), dtype=np.float32)
    start = 0
    for e in range(num_experts):
        n = int(group_sizes[e])
        if n == 0:
            continue
        sl = slice(start, start + n)
        g = cast_compute(np.matmul(xc[sl], cast_compute(gate[e], dtype), dtype=np.float32), dtype)
        u = cast_compute(np.matmul(xc[sl], cast_compute(up[e], dtype), dtype=np.float32), dtype)
        h = _swiglu_act(g, u, dtype)
        packed_y[sl] = cast_compute(np.matmul(h, cast_compute(down[e], dtype), dtype=np.float32), dtype)
        if return_stages:
            gate_x[sl], up_x[sl], act[sl] = g, u, h
        start += n
    if return_stages:
        return packed_y, gate_x, up_x, act
    return packed_y


def experts_per_assignment(
    x: np.ndarray,
    expert_ids: np.ndarray,
    weights: np.ndarray,
    gate: np.ndarray,
    up: np.ndarray,
    down: np.ndarray,
    dtype: str,
) -> np.ndarray:
    """Semantic reference: one selected expert per (token, slot) (moe.py:174-195).

    x [T,H]; expert_ids, weights [T,K].  Pure loops; small inputs only.
    """
    xc = cast_compute(x, dtype)
    wc = cast_compute(weights, dtype)
    tokens, hidden = xc.shape
    top_k = expert_ids.shape[-1]
    out = np.zeros((tokens, hidden), dtype=np.float32)
    for t in range(tokens):
        acc = np.zeros((hidden,), dtype=np.float32)
        for s in range(top_k):
            e = int(expert_ids[t, s])
            g = cast_compute(np.matmul(xc[t], cast_compute(gate[e], dtype), dtype=np.float32), dtype)
            u = cast_compute(np.matmul(xc[t], cast_compute(up[e], dtype), dtype=np.float32), dtype)
            h = _swiglu_act(g, u, dtype)
            y = cast_compute(np.matmul(h, cast_compute(down[e], dtype), dtype=np.float32), dtype)
            acc = acc + cast_compute(y * wc[t, s], dtype)
        out[t] = cast_compute(acc, dtype)
    return out


def combine(
    packed_y: np.ndarray,
    inverse: np.ndarray,
    weights: np.ndarray,
    dtype: str,
    shared_y: np.ndarray | None = None,
) -> np.ndarray:
    """out[t] = sum_s round(Y[inverse[t*K+s]] * w[t,s]) (+ shared), moe.py:663-671, :415.

    The sum over slots is sequential in fp32 and rounded once to the compute
    dtype; the shared-expert output is then added in the compute dtype.
    """
    wc = cast_compute(weights, dtype)
    tokens, top_k = wc.shape
    yc = cast_compute(packed_y, dtype)
    inv = np.asarray(inverse).reshape(tokens, top_k).astype(np.int64)
    acc = np.zeros((tokens, yc.shape[1]), dtype=np.float32)
    for s in range(top_k):
        acc = acc + cast_compute(yc[inv[:, s]] * wc[:, s : s + 1], dtype)
    out = cast_compute(acc, dtype)
    if shared_y is not None:
        out = cast_compute(out + cast_compute(shared_y, dtype), dtype)
    return out


def shared_swiglu(x: np.ndarray, gate: np.ndarray, up: np.ndarray, down: np.ndarray, dtype: str) -> np.ndarray:
    """Dense SwiGLU: down(silu(gate(x)) * up(x)) (moe.py:361-364; execution.py:253-273)."""
    xc = cast_compute(x, dtype)
    g = cast_compute(np.matmul(xc, cast_compute(gate, dtype), dtype=np.float32), dtype)
    u = cast_compute(np.matmul(xc, cast_compute(up, dtype), dtype=np.float32), dtype)
    h = _swiglu_act(g, u, dtype)
    return cast_compute(np.matmul(h, cast_compute(down, dtype), dtype=np.float32), dtype)


# --------------------------------------------------------------------------
# router statistics and the sequence balance loss
# --------------------------------------------------------------------------
@dataclass
class RouterStatsResult:
    expert_counts: np.ndarray  # [E] float32
    importance: np.ndarray  # [E] float32
    total_assignments: np.float32
    load_min: np.float32
    load_max: np.float32
    load_mean: np.float32
    max_vio: np.float32
    load_entropy: np.float32


def stats_from_counts(counts: np.ndarray, importance: np.ndarray) -> RouterStatsResult:
    """The scalar fields derived from the two [E] vectors (moe.py:806-813)."""
    counts = np.asarray(counts, dtype=np.float32)
    num_experts = counts.shape[0]
    total = np.float32(counts.sum(dtype=np.float32))
    mean = np.float32(total / F32(num_experts))
    load_min = np.float32(counts.min())
    load_max = np.float32(counts.max())
    max_vio = np.float32((load_max - mean) / np.maximum(mean, F32(1e-6)))
    prob = counts / np.maximum(total, F32(1e-6))
    safe = np.where(prob > 0, prob, F32(1.0))
    entropy = np.float32(-np.sum(np.where(prob > 0, prob * np.log(safe), F32(0.0)), dtype=np.float32))
    return RouterStatsResult(
        counts, np.asarray(importance, dtype=np.float32), total, load_min, load_max, mean, max_vio, entropy
    )


def router_stats(expert_ids: np.ndarray, weights: np.ndarray, num_experts: int) -> RouterStatsResult:
    """counts[e] = #assignments to e; importance[e] = sum of their (already rounded) weights."""
    flat = np.asarray(expert_ids).reshape(-1).astype(np.int64)
    w = np.asarray(weights, dtype=np.float32).reshape(-1)
    counts = np.bincount(flat, minlength=num_experts).astype(np.float32)
    importance = np.bincount(flat, weights=w.astype(np.float64), minlength=num_experts).astype(np.float32)
    return stats_from_counts(counts, importance)


def sequence_balance_loss(expert_ids: np.ndarray, scores: np.ndarray, top_k: int) -> np.float32:
    """sum_i f_i p_i / B with ids [B,S,K] and scores [B,S,E] (moe.py:828-840)."""
    if scores.ndim != 3:
        raise ValueError("router scores must have shape [batch, seq, experts]")
    batch, seq_len, num_experts = scores.shape
    ids = np.asarray(expert_ids).reshape(batch, seq_len * top_k).astype(np.int64)
    selected = np.stack([np.bincount(ids[b], minlength=num_experts) for b in range(batch)]).astype(np.float32)
    f_i = F32(num_experts / (top_k * seq_len)) * selected
    scores = np.asarray(scores, dtype=np.float32)
    normalized = scores / np.maximum(scores.sum(axis=-1, keepdims=True, dtype=np.float32), F32(1e-20))
    p_i = normalized.mean(axis=1, dtype=np.float32)
    return np.float32(np.sum(f_i * p_i, dtype=np.float32) / F32(batch))


# --------------------------------------------------------------------------
# SMEBU balancing update, the consumer of expert_counts  (steps/moe_balance.py:97-162)
# --------------------------------------------------------------------------
@dataclass
class SmebuResult:
    momentum: np.ndarray  # [L,E] float32
    expert_bias: np.ndarray  # [L,E] float32
    max_vio: np.float32  # max over layers
    load_min: np.float32  # min over layers
    load_max: np.float32  # max over layers
    load_entropy: np.float32  # mean over layers
    bias_norm: np.float32  # sqrt of the sum of squares of every updated bias
    momentum_norm: np.float32


def smebu_update(
    router_counts: np.ndarray,
    momentum: np.ndarray,
    expert_bias: np.ndarray,
    load_lr: float,
    momentum_factor: float,
    clamp: float,
) -> SmebuResult:
    """One non-gradient balancing step for L layers of E experts, all in float32.

    Per layer (steps/moe_balance.py:123-146): mean = sum(counts)/E; violation = (mean - counts) /
    max(mean, 1e-6); delta = load_lr * tanh(clamp * violation); delta -= mean(delta);
    momentum' = f * momentum + (1 - f) * delta; bias' = f32(bias) + momentum' (:180);
    metrics as in :139-161.
    """
    counts = np.asarray(router_counts, dtype=np.float32)
    momentum = np.asarray(momentum, dtype=np.float32)
    bias = np.asarray(expert_bias, dtype=np.float32)
    if counts.ndim != 2 or counts.shape != momentum.shape or counts.shape != bias.shape:
        raise ValueError("router count shape must match MoE balance state")
    layers, num_experts = counts.shape
    lr, factor, cl = F32(load_lr), F32(momentum_factor), F32(clamp)
    next_momentum = np.empty_like(momentum)
    next_bias = np.empty_like(bias)
    max_vios, mins, maxes, entropies = [], [], [], []
    bias_sq = F32(0.0)
    momentum_sq = F32(0.0)
    for layer in range(layers):
        c = counts[layer]
        count_sum = np.float32(c.sum(dtype=np.float32))
        mean = np.float32(count_sum / F32(num_experts))
        violation = (mean - c) / np.maximum(mean, F32(1e-6))
        delta = lr * np.tanh(cl * violation)
        delta = delta - np.float32(delta.mean(dtype=np.float32))
        m = factor * momentum[layer] + (F32(1.0) - factor) * delta
        next_momentum[layer] = m
        next_bias[layer] = bias[layer] + m
        st = stats_from_counts(c, np.zeros_like(c))
        max_vios.append(st.max_vio)
        mins.append(st.load_min)
        maxes.append(st.load_max)
        entropies.append(st.load_entropy)
        momentum_sq = np.float32(momentum_sq + np.sum(np.square(m), dtype=np.float32))
        bias_sq = np.float32(bias_sq + np.sum(np.square(next_bias[layer]), dtype=np.float32))
    return SmebuResult(
        next_momentum,
        next_bias,
        np.float32(max(max_vios)),
        np.float32(min(mins)),
        np.float32(max(maxes)),
        np.float32(np.mean(np.asarray(entropies, dtype=np.float32), dtype=np.float32)),
        np.float32(np.sqrt(bias_sq)),
        np.float32(np.sqrt(momentum_sq)),
    )


# --------------------------------------------------------------------------
# the layer  (moe.py:411-446)
# --------------------------------------------------------------------------
@dataclass
class MoeResult:
    y: np.ndarray  # [B,S,H] float32 storage, compute-dtype values
    route: RouterResult
    dispatch: DispatchResult
    packed_y: np.ndarray
    stats: RouterStatsResult
    aux_loss: np.float32 | None


def moe_forward(
    x: np.ndarray,
    w_router: np.ndarray,
    expert_bias: np.ndarray | None,
    gate: np.ndarray,
    up: np.ndarray,
    down: np.ndarray,
    top_k: int,
    route_scale: float = 1.0,
    dtype: str = "f32",
    shared: tuple[np.ndarray, np.ndarray, np.ndarray] | None = None,
    with_aux_loss: bool = False,
    score_func: str = "sigmoid",
) -> MoeResult:
    """Expert-major formulation of the whole layer; x [B,S,H]."""
    batch, seq_len, hidden = x.shape
    num_experts = gate.shape[0]
    x2 = np.asarray(x, dtype=np.float32).reshape(batch * seq_len, hidden)
    route = router(x2, w_router, expert_bias, top_k, route_scale, dtype, score_func)
    disp = dispatch(route.expert_ids, num_experts, cast_compute(x2, dtype))
    packed_y = grouped_swiglu(disp.packed_x, gate, up, down, disp.group_sizes, dtype)
    shared_y = None
    if shared is not None:
        shared_y = shared_swiglu(x2, shared[0], shared[1], shared[2], dtype)
    y = combine(packed_y, disp.inverse, route.weights, dtype, shared_y)
    stats = router_stats(route.expert_ids, route.weights, num_experts)
    aux = None
    if with_aux_loss:
        aux = sequence_balance_loss(
            route.expert_ids.reshape(batch, seq_len, top_k),
            route.scores.reshape(batch, seq_len, num_experts),
            top_k,
        )
    return MoeResult(y.reshape(batch, seq_len, hidden), route, disp, packed_y, stats, aux)


# --------------------------------------------------------------------------
# the decoder block around the layer: x + post_norm(mlp(pre_norm(x)))
# --------------------------------------------------------------------------
def rmsnorm(x: np.ndarray, scale: np.ndarray, eps: float, dtype: str) -> np.ndarray:
    """RMSNorm over the last axis with a float32 scale.

    The modules are flax ``nnx.RMSNorm`` (models/components/norm.py:12-31; flax 0.12.7 in
    the reference's ``uv.lock``, absent here), whose published algorithm is: statistics in
    float32, ``mul = rsqrt(mean(x^2) + eps) * scale``, ``y = x * mul``, cast to the compute
    dtype.  The reference's own ``rmsnorm_reference`` (kernels/rmsnorm.py:14-21) multiplies in
    the order ``(x * inv_rms) * weight``; both orders round to the same bf16 value except for
    results that sit within one fp32 ulp of a bf16 rounding boundary.  The sum of squares is
    accumulated by ``numpy.sum`` (pairwise), not in the order of any particular kernel.
    """
    xc = cast_compute(x, dtype).astype(np.float32)
    var = np.sum(xc * xc, axis=-1, keepdims=True, dtype=np.float32) / np.float32(xc.shape[-1])
    inv = np.float32(1.0) / np.sqrt(var + np.float32(eps), dtype=np.float32)
    mul = inv * np.asarray(scale, dtype=np.float32)
    return cast_compute(xc * mul, dtype)


def ffn_block_forward(x, pre_scale, post_scale, eps, w_router, expert_bias, gate, up, down, top_k,
                      route_scale=1.0, dtype="f32", shared=None):
    """x + ffn_post_norm(mlp(ffn_pre_norm(x))) of the decoder block (blocks.py:224-230); x [B,S,H].

    Returns (out [B,S,H], MoeResult of the inner layer).
    """
    xc = cast_compute(np.asarray(x, dtype=np.float32), dtype)
    normed = rmsnorm(xc, pre_scale, eps, dtype)
    inner = moe_forward(normed, w_router, expert_bias, gate, up, down, top_k, route_scale, dtype, shared)
    out = cast_compute(xc + rmsnorm(inner.y, post_scale, eps, dtype), dtype)
    return out, inner


# --------------------------------------------------------------------------
# seeded synthetic inputs of the benchmark configurations
# --------------------------------------------------------------------------
CONFIGS = {
    "C1": dict(batch=1, seq=2048, H=512, E=8, K=2, I=1024, Ns=0, dtype="f32"),
    "C2": dict(batch=4, seq=2048, H=1024, E=16, K=2, I=2816, Ns=0, dtype="bf16"),
    "C3": dict(batch=8, seq=2048, H=2048, E=64, K=8, I=1408, Ns=2, dtype="bf16"),
    "C4": dict(batch=8, seq=2048, H=2048, E=128, K=8, I=768, Ns=0, dtype="bf16", skew=True),
    "C5": dict(batch=64, seq=1, H=2048, E=64, K=8, I=1408, Ns=0, dtype="bf16"),
}


def zipf_expert_bias(num_experts: int) -> np.ndarray:
    """Selection-only bias that skews routing: -0.085*1.2*ln(rank), 6 experts disabled."""
    rank = 1 + np.random.Generator(np.random.PCG64(1)).permutation(num_experts)
    bias = (-0.085 * 1.2 * np.log(rank.astype(np.float64))).astype(np.float32)
    bias[rank > num_experts - 6] = F32(-4.0)
    return bias


def make_inputs(name: str, seed: int = 0, tokens: int | None = None) -> dict:
    """x~N(0,1); weights~N(0,0.02); draw order x, W_r, gate, up, down, shared_*.

    ``tokens`` overrides the token count (a [1, tokens, H] batch) without
    changing the weights that are drawn for the configuration.
    """
    cfg = dict(CONFIGS[name])
    rng = np.random.Generator(np.random.PCG64(seed))
    B, S, H, E, K, I, Ns = (cfg[k] for k in ("batch", "seq", "H", "E", "K", "I", "Ns"))
    x = rng.standard_normal((B, S, H), dtype=np.float32)
    if tokens is not None:
        x = x.reshape(B * S, H)[:tokens].reshape(1, tokens, H)
    sd = F32(0.02)
    w_router = rng.standard_normal((H, E), dtype=np.float32) * sd
    gate = rng.standard_normal((E, H, I), dtype=np.float32) * sd
    up = rng.standard_normal((E, H, I), dtype=np.float32) * sd
    down = rng.standard_normal((E, I, H), dtype=np.float32) * sd
    shared = None
    if Ns:
        shared = (
            rng.standard_normal((H, I * Ns), dtype=np.float32) * sd,
            rng.standard_normal((H, I * Ns), dtype=np.float32) * sd,
            rng.standard_normal((I * Ns, H), dtype=np.float32) * sd,
        )
    bias = zipf_expert_bias(E) if cfg.get("skew") else np.zeros((E,), dtype=np.float32)
    return dict(cfg=cfg, x=x, w_router=w_router, expert_bias=bias, gate=gate, up=up, down=down, shared=shared)
