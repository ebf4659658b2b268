"""CPU oracle for the backward pass of the MoE expert layer.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only ``tests/`` may import it.

The reference has no hand-written backward: it differentiates
``SparseMoE.forward_with_output`` (src/jaxtitan/models/components/moe.py:409-430)
with ``jax.grad`` (jax 0.10.0, pinned in the reference's ``uv.lock``; absent from
this environment).  What that yields is fixed by the chain rule applied to the
forward formulas, which this module restates in float64, operator by operator:

* ``experts_backward``  <- VJP of dispatch + ``ExpertSwiGLU`` + combine   moe.py:583-671
* ``shared_backward``   <- VJP of ``SharedSwiGLU.__call__``               moe.py:361-364
* ``router_backward``   <- VJP of ``SigmoidTopKRouter.__call__``          moe.py:131-147
* ``moe_backward``      <- VJP of the layer (sum of the three over x)     moe.py:409-430

Inputs are taken as they are (callers round them to the compute dtype first);
all arithmetic is float64 and nothing is rounded on the way, i.e. this is the
exact gradient of the un-rounded forward function at the given inputs.  The
selection (``expert_ids``) is piecewise constant and carries no gradient, and the
expert bias only enters the selection (moe.py:139-140).

Parity status (exercised in ``tests/test_oracle_grad.py``):

* experts_backward: pinned by central finite differences of the dense
  formulation the reference's own gradient test differentiates
  (tests/jaxtitan/test_model.py:596-603: gather the selected expert matrices,
  three einsums, weighted sum) on that test's inputs and its four routing
  patterns (balanced, one expert unused, all on one expert, duplicate routes),
  for all five differentiable arguments.
* shared_backward: pinned by finite differences of a plain two-matmul SwiGLU.
* router_backward: pinned by finite differences of the float64 closed form
  ``scale * p / (sum p + 1e-20)`` with the selection held fixed, including the
  extra cotangent on the scores.
* moe_backward: pinned by finite differences of the float64 layer built from the
  three closed forms above with the selection held fixed.
* sequence_balance_loss_backward: pinned by finite differences of the float64 closed
  form of the loss with the counts held fixed.
* route_weight_grad_rounded: the same inner product as experts_backward's d_weights with the
  four bf16 roundings a bf16 implementation makes on the way (the two products, the
  activation, dy Wd^T); pinned against experts_backward by the first-order error bound that
  those roundings allow (returned beside the value) and, with rounding switched off, by
  equality with experts_backward.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np


def _f64(a):
    return np.asarray(a, dtype=np.float64)


def _sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


@dataclass
class ExpertsGrad:
    dx: np.ndarray  # [T,H]
    d_weights: np.ndarray  # [T,K]
    d_gate: np.ndarray  # [E,H,I]
    d_up: np.ndarray  # [E,H,I]
    d_down: np.ndarray  # [E,I,H]


def experts_backward(x, expert_ids, weights, gate, up, down, dy) -> ExpertsGrad:
    """Gradient of y[t] = sum_s w[t,s] * (silu(x[t] Wg[e]) * (x[t] Wu[e])) Wd[e], e = ids[t,s]."""
    x, weights, gate, up, down, dy = (_f64(a) for a in (x, weights, gate, up, down, dy))
    ids = np.asarray(expert_ids)
    E = gate.shape[0]
    dx = np.zeros_like(x)
    d_weights = np.zeros_like(weights)
    d_gate, d_up, d_down = np.zeros_like(gate), np.zeros_like(up), np.zeros_like(down)
    for e in range(E):
        t_idx, s_idx = np.nonzero(ids == e)
        if t_idx.size == 0:
            continue
        xe, dye = x[t_idx], dy[t_idx]
        g, u = xe @ gate[e], xe @ up[e]
        sig = _sigmoid(g)
        h = g * sig * u
        yp = h @ down[e]
        w = weights[t_idx, s_idx][:, None]
        d_weights[t_idx, s_idx] = np.sum(dye * yp, axis=-1)
        dyp = dye * w
        dh = dyp @ down[e].T
        d_down[e] = h.T @ dyp
        dg = dh * u * sig * (1.0 + g * (1.0 - sig))
        du = dh * g * sig
        d_gate[e] = xe.T @ dg
        d_up[e] = xe.T @ du
        np.add.at(dx, t_idx, dg @ gate[e].T + du @ up[e].T)
    return ExpertsGrad(dx, d_weights, d_gate, d_up, d_down)


def _bf16(a):
    """float64 -> nearest bf16 (ties to even), returned as float64."""
    b = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    b = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16) << 16
    return b.astype(np.uint32).view(np.float32).astype(np.float64)


def route_weight_grad_rounded(x, expert_ids, gate, up, down, dy, rounded=True):
    """d_weights[t,s] = <dy[t], y_e(x[t])> evaluated as <Z, h> with Z = dy[t] Wd[e]^T and
    h = silu(g) u, g = x[t] Wg[e], u = x[t] Wu[e] (the same number: both are dy^T Wd^T h), where a
    bf16 implementation rounds g, u, h and Z to bf16 before the inner product and the result after it.

    Returns (value, budget), both [T,K].  budget[t,s] = 2^-8 * (sum_i |Z_i h_i| (3 + kappa_i) + |value|)
    with kappa = |d ln silu(g) / d ln g| = |1 + g (1 - sigmoid(g))|: the first-order bound on
    |value - exact| from one relative rounding of at most 2^-8 (the unit roundoff of bf16: half a
    unit in the last of its 8 significant bits) on each of Z, u, h (factor 1 each) and g
    (factor kappa), plus the rounding of the result.  With cancellation in the sum the exact value can
    be far smaller than sum_i |Z_i h_i|, which is why a bound relative to the value itself (or, for a
    tensor of one element, to the tensor's maximum) does not hold for this quantity.
    """
    x, gate, up, down, dy = (_f64(a) for a in (x, gate, up, down, dy))
    ids = np.asarray(expert_ids)
    rnd = _bf16 if rounded else (lambda a: a)
    value = np.zeros(ids.shape)
    budget = np.zeros(ids.shape)
    for e in range(gate.shape[0]):
        t_idx, s_idx = np.nonzero(ids == e)
        if t_idx.size == 0:
            continue
        g, u = rnd(x[t_idx] @ gate[e]), rnd(x[t_idx] @ up[e])
        sig = _sigmoid(g)
        h = rnd(g * sig * u)
        z = rnd(dy[t_idx] @ down[e].T)
        value[t_idx, s_idx] = rnd(np.sum(z * h, axis=-1))
        kappa = np.abs(1.0 + g * (1.0 - sig))
        budget[t_idx, s_idx] = 2.0**-8 * (np.sum(np.abs(z * h) * (3.0 + kappa), axis=-1) + np.abs(value[t_idx, s_idx]))
    return value, budget


@dataclass
class SharedGrad:
    dx: np.ndarray
    d_gate: np.ndarray
    d_up: np.ndarray
    d_down: np.ndarray


def shared_backward(x, gate, up, down, dy) -> SharedGrad:
    """Gradient of y = (silu(x Wg) * (x Wu)) Wd."""
    x, gate, up, down, dy = (_f64(a) for a in (x, gate, up, down, dy))
    g, u = x @ gate, x @ up
    sig = _sigmoid(g)
    h = g * sig * u
    dh = dy @ down.T
    dg = dh * u * sig * (1.0 + g * (1.0 - sig))
    du = dh * g * sig
    return SharedGrad(dg @ gate.T + du @ up.T, x.T @ dg, x.T @ du, h.T @ dy)


@dataclass
class RouterGrad:
    dx: np.ndarray  # [T,H]
    d_w_router: np.ndarray  # [H,E]
    d_logits: np.ndarray  # [T,E]


def _softmax(z):
    e = np.exp(z - z.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


def router_backward(x, w_router, expert_ids, d_weights, d_scores, route_scale, scores=None,
                    score_func="sigmoid") -> RouterGrad:
    """Gradient of weights = scale * p / (sum p + 1e-20), p = score(x W)[ids], plus a cotangent on the scores.
    score = sigmoid (the reference's router) or softmax over the experts (the attribute this build adds).

    ``scores`` overrides score(x W) (pass the forward's own scores to follow its rounding).
    """
    x, w_router, d_weights = _f64(x), _f64(w_router), _f64(d_weights)
    ids = np.asarray(expert_ids)
    T = x.shape[0]
    if scores is not None:
        sc = _f64(scores)
    else:
        sc = _sigmoid(x @ w_router) if score_func == "sigmoid" else _softmax(x @ w_router)
    rows = np.arange(T)[:, None]
    p = sc[rows, ids]
    S = p.sum(-1, keepdims=True) + 1e-20
    dp = route_scale * (d_weights / S - np.sum(d_weights * p, axis=-1, keepdims=True) / S**2)
    d_sc = np.zeros_like(sc) if d_scores is None else _f64(d_scores).copy()
    np.add.at(d_sc, (np.broadcast_to(rows, ids.shape), ids), dp)
    if score_func == "sigmoid":
        d_logits = d_sc * sc * (1.0 - sc)
    else:  # softmax Jacobian: d z_e = s_e (g_e - sum_j g_j s_j)
        d_logits = sc * (d_sc - np.sum(d_sc * sc, axis=-1, keepdims=True))
    return RouterGrad(d_logits @ w_router.T, x.T @ d_logits, d_logits)


@dataclass
class LayerGrad:
    dx: np.ndarray
    d_w_router: np.ndarray
    d_gate: np.ndarray
    d_up: np.ndarray
    d_down: np.ndarray
    d_shared: tuple | None  # (d_gate, d_up, d_down) of the shared experts
    d_weights: np.ndarray  # [T,K], the intermediate cotangent of the route weights


def moe_backward(x, w_router, gate, up, down, shared, expert_ids, weights, dy, d_scores, route_scale,
                 scores=None, score_func="sigmoid") -> LayerGrad:
    """Gradient of the layer y = routed(x) + shared(x) for the cotangents dy and d_scores.

    ``weights`` are the route weights the forward used; ``expert_ids`` its selection.
    """
    eg = experts_backward(x, expert_ids, weights, gate, up, down, dy)
    rg = router_backward(x, w_router, expert_ids, eg.d_weights, d_scores, route_scale, scores, score_func)
    dx = eg.dx + rg.dx
    d_shared = None
    if shared is not None:
        sg = shared_backward(x, shared[0], shared[1], shared[2], dy)
        dx = dx + sg.dx
        d_shared = (sg.d_gate, sg.d_up, sg.d_down)
    return LayerGrad(dx, rg.d_w_router, eg.d_gate, eg.d_up, eg.d_down, d_shared, eg.d_weights)


def sequence_balance_loss_backward(expert_ids, scores, top_k, d_loss=1.0) -> np.ndarray:
    """Gradient with respect to the scores of _sequence_balance_loss (moe.py:828-840):
    loss = sum_{b,e} f[b,e] * mean_s( scores[b,s,e] / max(sum_e scores[b,s,:], 1e-20) ) / B with
    f[b,e] = E / (K*S) * count[b,e]; the counts come from one_hot(ids) and carry no gradient.
    Pinned in tests/test_oracle_grad.py by central finite differences of an independently written
    float64 forward."""
    ids = np.asarray(expert_ids)
    sc = _f64(scores)
    B, S, E = sc.shape
    counts = np.zeros((B, E))
    for b in range(B):
        counts[b] = np.bincount(ids[b].reshape(-1), minlength=E)[:E]
    f = counts * (E / (top_k * S))
    total = sc.sum(-1, keepdims=True)
    clamped = total <= 1e-20
    denom = np.where(clamped, 1e-20, total)
    dot = np.sum(f[:, None, :] * sc, axis=-1, keepdims=True)
    second = np.where(clamped, 0.0, dot / denom**2)
    return d_loss / (B * S) * (f[:, None, :] / denom - second)
