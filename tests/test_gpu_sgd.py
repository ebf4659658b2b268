"""Three steps of gradient descent through the GPU backward pass against the same three steps through
the float64 gradient oracle.

The specification is the reference's multi-step test of its expert dispatcher
(tests/jaxtitan/test_model.py:694-764): fixed routing, loss = mean(output^2), plain SGD with learning
rate 1e-3 on the three expert tensors for three steps, parameters equal to rtol = atol = 1e-5 in fp32
and finite.  The first test is that case on its inputs; the second runs the whole layer (router
included, shared experts, a second loss term on the scores) through the torch autograd function, with
every parameter trained, the oracle stepped the same way from the same start.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import moe_grad_oracle as G
from oracle import moe_oracle as O
from research_amd import autograd, grad, ops
from test_gpu_parity import dev, host

pytestmark = pytest.mark.gpu

STEPS = 3
LR = 1e-3   # the reference's learning rate
LR2 = 0.05  # whole-layer case: large enough that three steps move every parameter far beyond the tolerance
TOL = dict(rtol=1e-5, atol=1e-5)


def reference_inputs():
    """Inputs of test_model.py:696-713."""
    E, H, I, S, K = 4, 3, 4, 6, 2
    x = np.arange(S * H, dtype=np.float64).reshape(S, H) / 17.0
    ids = (np.arange(S * K, dtype=np.int32).reshape(S, K) % E).astype(np.int32)
    weights = np.tile(np.array([0.3, 0.7]), (S, 1))
    gate = np.arange(E * H * I, dtype=np.float64).reshape(E, H, I) / 37.0
    up = np.flip(gate, axis=-1) / 1.3
    down = np.arange(E * I * H, dtype=np.float64).reshape(E, I, H) / 43.0
    return x, ids, weights, gate, up, down


def oracle_experts_output(x, ids, weights, gate, up, down):
    out = np.zeros_like(x)
    for t in range(x.shape[0]):
        for s in range(ids.shape[1]):
            e = ids[t, s]
            g, u = x[t] @ gate[e], x[t] @ up[e]
            out[t] += weights[t, s] * ((g / (1.0 + np.exp(-g)) * u) @ down[e])
    return out


def gpu_expert_sgd(gpu, x, ids, weights, gate, up, down):
    xd, wd = dev(x.astype(np.float32), gpu, "f32"), dev(weights.astype(np.float32), gpu, "f32")
    params = [dev(a.astype(np.float32), gpu, "f32") for a in (gate, up, down)]
    plan = ops.dispatch(dev(ids, gpu), gate.shape[0])
    for _ in range(STEPS):
        packed_y, _, res = grad.grouped_swiglu_train(xd, plan.source_order, ids.shape[1], *params, plan.group_sizes,
                                                     plan.offsets)
        y = ops.combine(packed_y, plan.inverse, wd)
        dy = (y * (2.0 / y.numel())).contiguous()  # d mean(y^2) / dy
        g = grad.experts_backward(xd, dy, plan, wd, *params, res)
        params = [p - LR * d for p, d in zip(params, (g.d_gate, g.d_up, g.d_down))]
    return params


def test_three_sgd_steps_on_the_reference_case_fp32(gpu):
    x, ids, weights, gate, up, down = reference_inputs()
    want = [gate.copy(), up.copy(), down.copy()]
    for _ in range(STEPS):
        y = oracle_experts_output(x, ids, weights, *want)
        g = G.experts_backward(x, ids, weights, *want, 2.0 * y / y.size)
        want = [p - LR * d for p, d in zip(want, (g.d_gate, g.d_up, g.d_down))]
    got = gpu_expert_sgd(gpu, x, ids, weights, gate, up, down)
    again = gpu_expert_sgd(gpu, x, ids, weights, gate, up, down)
    for name, a, b, ref, start in zip(("gate", "up", "down"), got, again, want, (gate, up, down)):
        assert bool(torch.isfinite(a).all())
        assert torch.equal(a, b), f"{name}: two identical runs differ"
        np.testing.assert_allclose(host(a), ref, err_msg=name, **TOL)
        # the steps did move the parameters by more than the tolerance, so the comparison means something
        assert np.max(np.abs(ref - start)) > 1e-4, name


def test_three_sgd_steps_of_the_whole_layer_through_autograd_fp32(gpu):
    rng = np.random.default_rng(5)
    T, H, E, K, I, Is = 48, 32, 6, 2, 40, 24
    x = rng.standard_normal((T, H))
    start = dict(
        w_router=rng.standard_normal((H, E)) * 0.3,
        gate=rng.standard_normal((E, H, I)) * 0.2, up=rng.standard_normal((E, H, I)) * 0.2,
        down=rng.standard_normal((E, I, H)) * 0.2,
        sg=rng.standard_normal((H, Is)) * 0.2, su=rng.standard_normal((H, Is)) * 0.2,
        sd=rng.standard_normal((Is, H)) * 0.2,
    )
    names = list(start)
    f32 = lambda a: a.astype(np.float32)
    score_target = rng.standard_normal((T, E)) * 0.1

    # ---- GPU: torch autograd over the native forward/backward ----
    def gpu_run():
        xd = dev(f32(x), gpu, "f32")
        tgt = dev(f32(score_target), gpu, "f32")
        p = {k: dev(f32(v), gpu, "f32").requires_grad_(True) for k, v in start.items()}
        selections = []
        for _ in range(STEPS):
            y, scores, ids = autograd.moe_layer(xd, p["w_router"], None, p["gate"], p["up"], p["down"], K, 1.0,
                                                shared=(p["sg"], p["su"], p["sd"]))
            loss = (y * y).sum() / T + (scores * tgt).sum() / T
            grads = torch.autograd.grad(loss, [p[k] for k in names])
            selections.append(host(ids).copy())
            p = {k: (p[k] - LR2 * g).detach().requires_grad_(True) for k, g in zip(names, grads)}
        return {k: v.detach() for k, v in p.items()}, selections

    got, selections = gpu_run()
    again, _ = gpu_run()

    # ---- oracle: fp32 forward for the selection and the route weights, float64 gradients ----
    want = {k: f32(v).astype(np.float64) for k, v in start.items()}
    x32 = f32(x).astype(np.float64)
    for step in range(STEPS):
        route = O.router(f32(x32), f32(want["w_router"]), None, K, 1.0, "f32")
        assert np.array_equal(route.expert_ids, selections[step]), "selection differs (a near-tie in the test inputs)"
        ids = route.expert_ids
        logits = x32 @ want["w_router"]
        scores = 1.0 / (1.0 + np.exp(-logits))
        top = np.take_along_axis(scores, ids.astype(np.int64), axis=-1)
        weights = top / (top.sum(-1, keepdims=True) + 1e-20)
        y = oracle_experts_output(x32, ids, weights, want["gate"], want["up"], want["down"])
        gs, us = x32 @ want["sg"], x32 @ want["su"]
        y = y + (gs / (1.0 + np.exp(-gs)) * us) @ want["sd"]
        g = G.moe_backward(x32, want["w_router"], want["gate"], want["up"], want["down"],
                           (want["sg"], want["su"], want["sd"]), ids, weights, 2.0 * y / T, score_target / T, 1.0)
        grads = dict(w_router=g.d_w_router, gate=g.d_gate, up=g.d_up, down=g.d_down, sg=g.d_shared[0],
                     su=g.d_shared[1], sd=g.d_shared[2])
        want = {k: want[k] - LR2 * grads[k] for k in names}

    for k in names:
        assert bool(torch.isfinite(got[k]).all())
        assert torch.equal(got[k], again[k]), f"{k}: two identical runs differ"
        np.testing.assert_allclose(host(got[k]), want[k], err_msg=k, **TOL)
    for k in names:  # every parameter moved by much more than the tolerance
        assert float(np.max(np.abs(want[k] - f32(start[k])))) > 1e-3, k
