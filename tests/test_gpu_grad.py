"""Parity of the backward pass (through the C ABI) with the float64 gradient oracle, on the GPU.

The specification is the reference's own gradient test of the expert dispatcher
(tests/jaxtitan/test_model.py:549-691): gradients with respect to x, the route weights and the
three expert matrices on four routing patterns, rtol = atol = 1e-5 in fp32, and bit-identical
results when the call is repeated.  bf16 results are held to max|g-ref|/max|ref| <= 2e-2 per
tensor, the bar of the forward pass.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import moe_grad_oracle as G
from oracle import moe_oracle as O
from research_amd import grad, ops
from test_gpu_parity import BF16_MAX_REL, dev, host, random_problem, report
from test_oracle_grad import SINGLE_TOKEN_SHAPES, reference_case

pytestmark = pytest.mark.gpu

F32_GRAD_TOL = dict(rtol=1e-5, atol=1e-5)


def expert_grads(gpu, x, ids, w, gate, up, down, dy, dtype, dx_extra=None):
    xd, gd, ud, dd, wd, dyd = (dev(a.astype(np.float32), gpu, dtype) for a in (x, gate, up, down, w, dy))
    plan = ops.dispatch(dev(ids.astype(np.int32), gpu), gate.shape[0])
    packed_y, act, res = grad.grouped_swiglu_train(xd, plan.source_order, ids.shape[1], gd, ud, dd, plan.group_sizes,
                                                   plan.offsets)
    extra = None if dx_extra is None else dev(dx_extra.astype(np.float32), gpu, dtype)
    return grad.experts_backward(xd, dyd, plan, wd, gd, ud, dd, res, dx_extra=extra), (packed_y, act, res, plan)


@pytest.mark.parametrize("pattern", ["balanced", "no_expert_three", "all_one_expert", "duplicate_routes"])
@pytest.mark.parametrize("batch", [1, 2])
def test_expert_gradients_on_the_reference_case_fp32(gpu, pattern, batch):
    x, gate, up, down, weights, patterns, cot = reference_case(batch)
    ids = patterns[pattern]
    want = G.experts_backward(x, ids, weights, gate, up, down, cot)
    got, _ = expert_grads(gpu, x, ids, weights, gate, up, down, cot, "f32")
    again, _ = expert_grads(gpu, x, ids, weights, gate, up, down, cot, "f32")
    for name in ("dx", "d_weights", "d_gate", "d_up", "d_down"):
        g = getattr(got, name)
        assert bool(torch.isfinite(g).all())
        np.testing.assert_allclose(host(g), getattr(want, name), err_msg=f"{pattern} {name}", **F32_GRAD_TOL)
        assert torch.equal(g, getattr(again, name)), f"{name} differs between two identical calls"


@pytest.mark.parametrize(
    "tokens,hidden,experts,top_k,inter,dtype",
    [(70, 32, 4, 2, 64, "f32"), (200, 192, 8, 2, 320, "f32"), (300, 64, 6, 3, 96, "bf16"), (257, 200, 5, 2, 136, "bf16"),
     (700, 1024, 16, 2, 704, "bf16"), (512, 2048, 64, 8, 1408, "bf16")]
    # one token: the route-weight gradient is a tensor of one or two elements whose terms can cancel
    + [shape + ("bf16",) for shape in SINGLE_TOKEN_SHAPES],
)
def test_expert_gradients_match_oracle(gpu, tokens, hidden, experts, top_k, inter, dtype):
    std = 0.02 if hidden >= 512 else 0.2
    x, gate, up, down, ids, w = random_problem(100 + tokens, tokens, hidden, experts, top_k, inter, std)
    rng = np.random.default_rng(tokens)
    ids[: tokens // 4] = ids[0]  # skew; leaves some experts with few rows
    dy = rng.standard_normal((tokens, hidden)).astype(np.float32)
    extra = rng.standard_normal((tokens, hidden)).astype(np.float32)
    cast = lambda a: O.cast_compute(a, dtype)
    want = G.experts_backward(cast(x), ids, cast(w), cast(gate), cast(up), cast(down), cast(dy))
    got, (packed_y, act, res, plan) = expert_grads(gpu, x, ids, w, gate, up, down, dy, dtype, dx_extra=extra)
    # the training forward returns what the plain forward returns, and the two products it keeps
    d = O.dispatch(ids, experts, cast(x))
    ref_y, ref_g, ref_u, _ = O.grouped_swiglu(d.packed_x, gate, up, down, d.group_sizes, dtype, return_stages=True)
    plain = ops.grouped_swiglu_gather(dev(x, gpu, dtype), plan.source_order, top_k, dev(gate, gpu, dtype),
                                      dev(up, gpu, dtype), dev(down, gpu, dtype), plan.group_sizes,
                                      plan.offsets) if dtype == "bf16" and hidden % 64 == 0 and inter % 64 == 0 else None
    if plain is not None:
        assert torch.equal(plain, packed_y)
    tag = f"grad {dtype} T={tokens} H={hidden} E={experts} K={top_k} I={inter}"
    wants = dict(dx=want.dx + cast(extra), d_weights=want.d_weights, d_gate=want.d_gate, d_up=want.d_up,
                 d_down=want.d_down)
    if dtype == "bf16":
        assert report(tag + " gate_pre", host(res.gate_pre), ref_g) <= BF16_MAX_REL
        assert report(tag + " up_pre", host(res.up_pre), ref_u) <= BF16_MAX_REL
        assert report(tag + " packed_y", host(packed_y), ref_y) <= BF16_MAX_REL
        for name, ref in wants.items():
            r = report(f"{tag} {name}", host(getattr(got, name)), ref.astype(np.float32))
            if name != "d_weights":
                assert r <= BF16_MAX_REL
        # The route-weight gradient is an inner product <Z, h> of bf16-rounded factors whose terms can cancel:
        # each element is held to the first-order budget of those roundings (test_oracle_grad pins the
        # budget on the CPU), not to the tensor's maximum, which for one token is the element itself.
        value, budget = G.route_weight_grad_rounded(cast(x), ids, cast(gate), cast(up), cast(down), cast(dy))
        dw = host(got.d_weights).astype(np.float64)
        print(f"[parity] {tag} d_weights: max err/budget = {float(np.max(np.abs(dw - want.d_weights) / budget)):.3f}; "
              f"against the rounded evaluation: {float(np.max(np.abs(dw - value) / budget)):.3f}", flush=True)
        assert np.all(np.abs(dw - want.d_weights) <= budget)
        # and the kernel's own value to the same evaluation with the same roundings made in float64: what is
        # left between the two is a factor that the kernel's fp32 sums rounded the other way
        assert np.all(np.abs(dw - value) <= 0.5 * budget)
    else:
        np.testing.assert_allclose(host(res.gate_pre), ref_g, rtol=2e-5, atol=2e-5)
        np.testing.assert_allclose(host(res.up_pre), ref_u, rtol=2e-5, atol=2e-5)
        for name, ref in wants.items():
            scale = float(np.max(np.abs(ref))) or 1.0
            np.testing.assert_allclose(host(getattr(got, name)) / scale, ref / scale, rtol=1e-4, atol=2e-5,
                                       err_msg=name)
    # experts that received no row get exactly zero weight gradients
    for e in np.nonzero(host(plan.group_sizes) == 0)[0]:
        assert not got.d_gate[e].any() and not got.d_up[e].any() and not got.d_down[e].any()


@pytest.mark.parametrize("tokens,hidden,experts,top_k,inter", [(1500, 512, 64, 4, 384), (900, 1024, 40, 2, 704)])
def test_expert_gradients_with_one_dominant_group(gpu, tokens, hidden, experts, top_k, inter):
    """Very unequal groups: one expert takes a slot of most tokens, a third of the experts get nothing.

    The weight-gradient launch then has more (group, tile) pairs than workgroups and hands them out
    longest group first; every pair must still be computed exactly once.
    """
    x, gate, up, down, ids, w = random_problem(7 + tokens, tokens, hidden, experts, top_k, inter, 0.02)
    rng = np.random.default_rng(tokens)
    live = experts - experts // 3
    ids = np.stack([rng.permutation(live)[:top_k] for _ in range(tokens)]).astype(np.int32)
    heavy = rng.random(tokens) < 0.8
    ids[heavy, 0] = 0
    for t in np.nonzero(heavy)[0]:  # keep the slots of a token distinct
        dup = np.nonzero(ids[t, 1:] == 0)[0]
        if dup.size:
            ids[t, 1 + dup[0]] = live - 1 if live - 1 not in ids[t] else next(e for e in range(1, live) if e not in ids[t])
    dy = rng.standard_normal((tokens, hidden)).astype(np.float32)
    cast = lambda a: O.cast_compute(a, "bf16")
    want = G.experts_backward(cast(x), ids, cast(w), cast(gate), cast(up), cast(down), cast(dy))
    got, (_, _, _, plan) = expert_grads(gpu, x, ids, w, gate, up, down, dy, "bf16")
    again, _ = expert_grads(gpu, x, ids, w, gate, up, down, dy, "bf16")
    sizes = host(plan.group_sizes)
    assert sizes.max() > 10 * np.median(sizes[sizes > 0]) and (sizes == 0).sum() >= experts // 3
    tag = f"dominant group T={tokens} H={hidden} E={experts} K={top_k} I={inter}"
    for name in ("dx", "d_weights", "d_gate", "d_up", "d_down"):
        ref = getattr(want, name).astype(np.float32)
        assert report(f"{tag} {name}", host(getattr(got, name)), ref) <= BF16_MAX_REL
        assert torch.equal(getattr(got, name), getattr(again, name)), f"{name} differs between two identical calls"
    # per expert, so that a small expert's matrices are not hidden behind the dominant one's scale
    for name in ("d_gate", "d_up", "d_down"):
        g, ref = host(getattr(got, name)), getattr(want, name).astype(np.float32)
        for e in range(experts):
            if sizes[e] == 0:
                assert not g[e].any()
            else:
                scale = float(np.max(np.abs(ref[e])))
                assert float(np.max(np.abs(g[e] - ref[e]))) <= BF16_MAX_REL * scale, f"{tag} {name}[{e}]"


@pytest.mark.parametrize("tokens,hidden,experts,top_k,inter,dtype",
                         [(90, 64, 5, 2, 96, "f32"), (600, 256, 8, 4, 192, "bf16"), (3000, 128, 12, 4, 128, "bf16")])
def test_expert_gradients_with_dropped_ids(gpu, tokens, hidden, experts, top_k, inter, dtype):
    """Ids outside [0, E) are dropped by the dispatch (inverse = -1, fewer packed rows than assignments).

    The backward pass must then stay inside the rows that exist: the gradients equal those of the
    same problem with the dropped assignments simply absent, and the route-weight gradient of a dropped
    assignment is exactly zero.  The buffers the tail of the plan would index are poisoned first.
    """
    x, gate, up, down, ids, w = random_problem(31 + tokens, tokens, hidden, experts, top_k, inter, 0.1)
    rng = np.random.default_rng(tokens)
    drop = rng.random(ids.shape) < 0.2
    ids = ids.copy()
    ids[drop] = np.where(rng.random(int(drop.sum())) < 0.5, experts + 3, -1)
    dy = rng.standard_normal((tokens, hidden)).astype(np.float32)
    cast = lambda a: O.cast_compute(a, dtype)
    want = G.experts_backward(cast(x), ids, cast(w), cast(gate), cast(up), cast(down), cast(dy))
    assert not want.d_weights[drop].any()
    xd, gd, ud, dd, wd, dyd = (dev(a.astype(np.float32), gpu, dtype) for a in (x, gate, up, down, w, dy))
    plan = ops.dispatch(dev(ids.astype(np.int32), gpu), experts)
    sizes = host(plan.group_sizes)
    kept = int(sizes.sum())
    assert kept == int((~drop).sum()) < tokens * top_k
    assert np.array_equal(host(plan.inverse).reshape(ids.shape) < 0, drop)
    # what lies past the last group is not part of the plan: make any use of it show
    plan.source_order[kept:] = 0x3FFFFFFF
    _, _, res = grad.grouped_swiglu_train(xd, plan.source_order, top_k, gd, ud, dd, plan.group_sizes, plan.offsets)
    res.gate_pre[kept:] = float("nan")
    res.up_pre[kept:] = float("nan")
    got = grad.experts_backward(xd, dyd, plan, wd, gd, ud, dd, res)
    again = grad.experts_backward(xd, dyd, plan, wd, gd, ud, dd, res)
    tag = f"dropped ids {dtype} T={tokens} E={experts} K={top_k}"
    for name in ("dx", "d_weights", "d_gate", "d_up", "d_down"):
        g, ref = getattr(got, name), getattr(want, name).astype(np.float32)
        assert bool(torch.isfinite(g).all()), name
        assert torch.equal(g, getattr(again, name)), f"{name} differs between two identical calls"
        if dtype == "bf16":
            assert report(f"{tag} {name}", host(g), ref) <= BF16_MAX_REL
        else:
            scale = float(np.max(np.abs(ref))) or 1.0
            np.testing.assert_allclose(host(g) / scale, ref / scale, rtol=1e-4, atol=2e-5, err_msg=name)
    assert not host(got.d_weights)[drop].any()


# the 4096-token cases take the path that splits a long one-group reduction into partial sums
@pytest.mark.parametrize("tokens,hidden,inter,dtype", [(5, 16, 24, "f32"), (300, 1024, 704, "bf16"), (130, 72, 40, "bf16"),
                                                       (4096, 512, 704, "bf16"), (64, 1024, 704, "bf16")])
def test_shared_gradients_match_oracle(gpu, tokens, hidden, inter, dtype):
    rng = np.random.default_rng(7)
    std = 0.02 if hidden >= 512 else 0.2
    x = rng.standard_normal((tokens, hidden)).astype(np.float32)
    gate, up = (rng.standard_normal((hidden, inter)).astype(np.float32) * std for _ in range(2))
    down = rng.standard_normal((inter, hidden)).astype(np.float32) * std
    dy = rng.standard_normal((tokens, hidden)).astype(np.float32)
    cast = lambda a: O.cast_compute(a, dtype)
    want = G.shared_backward(cast(x), cast(gate), cast(up), cast(down), cast(dy))
    xd, gd, ud, dd, dyd = (dev(a, gpu, dtype) for a in (x, gate, up, down, dy))
    y, res = grad.shared_swiglu_train(xd, gd, ud, dd)
    assert torch.equal(y, ops.shared_swiglu(xd, gd, ud, dd))
    got = grad.shared_backward(xd, dyd, gd, ud, dd, res)
    for name, g, ref in zip(("dx", "d_gate", "d_up", "d_down"), got, (want.dx, want.d_gate, want.d_up, want.d_down)):
        if dtype == "bf16":
            assert report(f"shared grad T={tokens} H={hidden} I={inter} {name}", host(g), ref.astype(np.float32)) <= BF16_MAX_REL
        else:
            np.testing.assert_allclose(host(g), ref, rtol=1e-4, atol=2e-5, err_msg=name)


@pytest.mark.parametrize("tokens,hidden,experts,top_k,dtype,with_scores",
                         [(6, 5, 7, 3, "f32", True), (300, 256, 64, 8, "bf16", True), (129, 72, 10, 2, "bf16", False),
                          (512, 2048, 128, 8, "bf16", True), (4100, 256, 64, 8, "bf16", True)])
def test_router_gradients_match_oracle(gpu, tokens, hidden, experts, top_k, dtype, with_scores):
    rng = np.random.default_rng(11)
    x = rng.standard_normal((tokens, hidden)).astype(np.float32)
    w = (rng.standard_normal((hidden, experts)) * (0.02 if hidden >= 256 else 0.3)).astype(np.float32)
    d_weights = rng.standard_normal((tokens, top_k)).astype(np.float32)
    d_scores = rng.standard_normal((tokens, experts)).astype(np.float32) if with_scores else None
    scale = 2.5
    xd, wd = dev(x, gpu, dtype), dev(w, gpu, dtype)
    fwd = ops.router(xd, wd, None, top_k, scale)
    cast = lambda a: O.cast_compute(a, dtype)
    want = G.router_backward(cast(x), cast(w), host(fwd.expert_ids), cast(d_weights), d_scores, scale,
                             scores=host(fwd.scores))
    dx, d_w = grad.router_backward(xd, wd, fwd.scores, fwd.expert_ids, dev(d_weights, gpu, dtype),
                                   None if d_scores is None else dev(d_scores, gpu), scale)
    tag = f"router grad {dtype} T={tokens} H={hidden} E={experts} K={top_k}"
    if dtype == "bf16":
        assert report(tag + " dx", host(dx), want.dx.astype(np.float32)) <= BF16_MAX_REL
        assert report(tag + " d_w_router", host(d_w), want.d_w_router.astype(np.float32)) <= BF16_MAX_REL
    else:
        np.testing.assert_allclose(host(dx), want.dx, rtol=1e-4, atol=2e-5)
        np.testing.assert_allclose(host(d_w), want.d_w_router, rtol=1e-4, atol=2e-5)


def layer_case(gpu, name, tokens, top_k, dtype, tag):
    inp = O.make_inputs(name, seed=0, tokens=tokens)
    cfg = inp["cfg"]
    T = inp["x"].shape[0] * inp["x"].shape[1]
    x2 = inp["x"].reshape(T, cfg["H"])
    rng = np.random.default_rng(17)
    dy = rng.standard_normal(x2.shape).astype(np.float32)
    d_scores = (rng.standard_normal((T, cfg["E"])) * 0.1).astype(np.float32)
    params = [dev(inp[k], gpu, dtype) for k in ("w_router", "gate", "up", "down")]
    shared = None if inp["shared"] is None else tuple(dev(m, gpu, dtype) for m in inp["shared"])
    xd = dev(x2, gpu, dtype)
    result, residuals = grad.moe_forward_train(xd, params[0], dev(inp["expert_bias"], gpu), params[1], params[2],
                                               params[3], top_k, 1.0, shared=shared)
    plain = ops.moe_forward(xd, params[0], dev(inp["expert_bias"], gpu), params[1], params[2], params[3], top_k, 1.0,
                            shared=shared)
    assert torch.equal(plain.expert_ids, result.expert_ids) and torch.equal(plain.y, result.y)
    got = grad.moe_backward(xd, dev(dy, gpu, dtype), dev(d_scores, gpu), params[0], params[1], params[2], params[3],
                            shared, result, residuals, 1.0)
    again = grad.moe_backward(xd, dev(dy, gpu, dtype), dev(d_scores, gpu), params[0], params[1], params[2],
                              params[3], shared, result, residuals, 1.0)
    cast = lambda a: O.cast_compute(a, dtype)
    want = G.moe_backward(cast(x2), cast(inp["w_router"]), cast(inp["gate"]), cast(inp["up"]), cast(inp["down"]),
                          None if inp["shared"] is None else tuple(cast(m) for m in inp["shared"]),
                          host(result.expert_ids), host(result.weights), cast(dy), d_scores, 1.0,
                          scores=host(result.scores))
    pairs = [("dx", got.dx, want.dx, again.dx), ("d_w_router", got.d_w_router, want.d_w_router, again.d_w_router),
             ("d_gate", got.d_gate, want.d_gate, again.d_gate), ("d_up", got.d_up, want.d_up, again.d_up),
             ("d_down", got.d_down, want.d_down, again.d_down)]
    if shared is not None:
        for i, n in enumerate(("d_shared_gate", "d_shared_up", "d_shared_down")):
            pairs.append((n, got.d_shared[i], want.d_shared[i], again.d_shared[i]))
    for n, g, ref, g2 in pairs:
        assert torch.equal(g, g2), f"{n} differs between two identical calls"
        if dtype == "bf16":
            assert report(f"{tag} {n}", host(g), ref.astype(np.float32)) <= BF16_MAX_REL
        else:
            scale = float(np.max(np.abs(ref))) or 1.0
            np.testing.assert_allclose(host(g) / scale, ref / scale, rtol=1e-4, atol=3e-5, err_msg=n)


def test_layer_gradients_c1_fp32_sample(gpu):
    layer_case(gpu, "C1", 256, 2, "f32", "C1 grad fp32 T=256")


def test_layer_gradients_c2_bf16_sample(gpu):
    layer_case(gpu, "C2", 512, 2, "bf16", "C2 grad bf16 T=512 H=1024 E=16 K=2 I=2816")


def test_layer_gradients_c3_bf16_sample_with_shared(gpu):
    layer_case(gpu, "C3", 512, 8, "bf16", "C3 grad bf16 T=512 H=2048 E=64 K=8 I=1408 Ns=2")


def test_gradients_with_no_tokens(gpu):
    E, H, I, K = 4, 64, 64, 2
    z = lambda *s: torch.zeros(s, dtype=torch.bfloat16, device=gpu)
    rnd = lambda *s: torch.randn(s, device=gpu).to(torch.bfloat16)
    gate, up, down = rnd(E, H, I), rnd(E, H, I), rnd(E, I, H)
    plan = ops.dispatch(torch.zeros((0, K), dtype=torch.int32, device=gpu), E)
    res = grad.ExpertResiduals(z(0, I), z(0, I))
    got = grad.experts_backward(z(0, H), z(0, H), plan, z(0, K), gate, up, down, res)
    assert got.dx.shape == (0, H) and not got.d_gate.any() and not got.d_up.any() and not got.d_down.any()


def test_autograd_function_routes_cotangents_to_the_backward_entry(gpu):
    """torch.autograd over the layer gives what jtmoe_moe_backward gives for the same cotangents."""
    from research_amd import autograd

    inp = O.make_inputs("C2", seed=2, tokens=256)
    cfg = inp["cfg"]
    x2 = inp["x"].reshape(-1, cfg["H"])
    leaf = lambda a: dev(a, gpu, "bf16").requires_grad_(True)
    x, w, gate, up, down = (leaf(a) for a in (x2, inp["w_router"], inp["gate"], inp["up"], inp["down"]))
    bias = dev(inp["expert_bias"], gpu)
    y, scores, ids = autograd.moe_layer(x, w, bias, gate, up, down, 2, 1.0)
    assert not ids.requires_grad and y.requires_grad and scores.requires_grad
    rng = np.random.default_rng(23)
    dy = dev(rng.standard_normal(x2.shape).astype(np.float32), gpu, "bf16")
    d_scores = dev((rng.standard_normal(scores.shape) * 0.1).astype(np.float32), gpu)
    loss = (y.float() * dy.float()).sum() + (scores * d_scores).sum()
    loss.backward()
    result, residuals = grad.moe_forward_train(x.detach(), w.detach(), bias, gate.detach(), up.detach(),
                                               down.detach(), 2, 1.0)
    want = grad.moe_backward(x.detach(), dy, d_scores, w.detach(), gate.detach(), up.detach(), down.detach(), None,
                             result, residuals, 1.0)
    for got, ref in ((x.grad, want.dx), (w.grad, want.d_w_router), (gate.grad, want.d_gate), (up.grad, want.d_up),
                     (down.grad, want.d_down)):
        assert torch.equal(got, ref)


@pytest.mark.parametrize("batch,seq,experts,top_k", [(1, 5, 3, 2), (3, 70, 8, 2), (2, 300, 64, 8), (4, 129, 200, 16)])
def test_sequence_balance_loss_gradient_matches_oracle(gpu, batch, seq, experts, top_k):
    """d loss / d scores of the auxiliary loss (moe.py:828-840), alone and through torch autograd."""
    from research_amd import autograd

    rng = np.random.default_rng(batch * 1000 + seq)
    scores = (1.0 / (1.0 + np.exp(-rng.standard_normal((batch, seq, experts))))).astype(np.float32)
    ids = np.stack([[rng.permutation(experts)[:top_k] for _ in range(seq)] for _ in range(batch)]).astype(np.int32)
    want = G.sequence_balance_loss_backward(ids, scores, top_k, d_loss=1.0)
    sd, idd = dev(scores, gpu), dev(ids, gpu)
    got = ops.sequence_balance_loss_backward(idd, sd, top_k=top_k)
    scale = float(np.max(np.abs(want)))
    np.testing.assert_allclose(host(got) / scale, want / scale, rtol=1e-4, atol=2e-6)
    assert torch.equal(got, ops.sequence_balance_loss_backward(idd, sd, top_k=top_k))
    # through autograd, with a weight on the loss as the training objective applies it
    s_req = sd.clone().requires_grad_(True)
    loss = autograd.sequence_balance_loss(idd, s_req, top_k)
    assert float(loss.detach()) == pytest.approx(float(O.sequence_balance_loss(ids, scores, top_k)), rel=1e-5)
    (g,) = torch.autograd.grad(loss * 0.25, [s_req])
    np.testing.assert_allclose(host(g) / scale, 0.25 * want / scale, rtol=1e-4, atol=2e-6)


def test_training_step_replays_from_a_captured_graph(gpu):
    """Forward with residuals and the backward pass only enqueue kernels, so a training step can be captured
    once and replayed (the reference's step runs inside one compiled program, steps/train_step.py): every
    replay, with eager work and synchronisations between them, gives the eager call's gradients bit for bit."""
    tokens, hidden, experts, top_k, inter, shared_inter = 700, 256, 16, 2, 192, 128
    gen = torch.Generator(device=gpu).manual_seed(21)
    draw = lambda *shape, std=1.0: (torch.randn(*shape, device=gpu, generator=gen) * std).to(torch.bfloat16)
    w_router, gate, up = draw(hidden, experts, std=0.1), draw(experts, hidden, inter, std=0.05), draw(experts, hidden, inter, std=0.05)
    down = draw(experts, inter, hidden, std=0.05)
    shared = (draw(hidden, shared_inter, std=0.05), draw(hidden, shared_inter, std=0.05), draw(shared_inter, hidden, std=0.05))

    def step(x, dy):
        result, residuals = grad.moe_forward_train(x, w_router, None, gate, up, down, top_k, 1.0, shared=shared)
        return result, grad.moe_backward(x, dy, None, w_router, gate, up, down, shared, result, residuals, 1.0)

    x_in, dy_in = draw(tokens, hidden), draw(tokens, hidden)
    side = torch.cuda.Stream(device=gpu)
    side.wait_stream(torch.cuda.current_stream(gpu))
    with torch.cuda.stream(side):
        for _ in range(2):  # first calls set kernel attributes and size the workspaces
            step(x_in, dy_in)
    torch.cuda.current_stream(gpu).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured_result, captured = step(x_in, dy_in)
    for i in range(4):
        x, dy = draw(tokens, hidden), draw(tokens, hidden)
        eager_result, eager = step(x, dy)
        torch.cuda.synchronize()
        x_in.copy_(x)
        dy_in.copy_(dy)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured_result.y, eager_result.y), f"replay {i}: y"
        for name in ("dx", "d_w_router", "d_gate", "d_up", "d_down"):
            assert torch.equal(getattr(captured, name), getattr(eager, name)), f"replay {i}: {name}"
        for a, b in zip(captured.d_shared, eager.d_shared):
            assert torch.equal(a, b), f"replay {i}: shared gradient"
        (eager.dx.float() * 2).sum().item()  # unrelated eager work between the replays
