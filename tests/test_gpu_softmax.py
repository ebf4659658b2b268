"""The softmax score function of the router (the attribute the _sf entry points add) on the GPU.

The reference's router is a sigmoid (moe.py:133); the benchmark's second configuration names a softmax
router, which this library offers as an attribute of the same router.  PARITY UNPINNED against the
reference, which has nothing to compare with: the oracle's softmax is pinned by float64 closed forms
(tests/test_oracle_router.py) and its gradient by finite differences (tests/test_oracle_grad.py); the
kernels are held to the oracle at the bars of the sigmoid path: the routing decision bit-exact given
the logits, floating-point outputs within the bf16 / fp32 tolerances of test_gpu_parity.py.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import moe_grad_oracle as G
from oracle import moe_oracle as O
from research_amd import autograd, grad, ops
from research_amd.errors import ContractError
from test_gpu_parity import BF16_MAX_REL, dev, host, report

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize(
    "tokens,experts,top_k,dtype,scale,use_bias",
    [
        (1, 3, 2, "f32", 1.0, False),
        (65, 8, 2, "f32", 1.5, True),
        (300, 16, 2, "bf16", 1.0, False),
        (1000, 64, 8, "bf16", 2.5, True),
        (513, 128, 8, "bf16", 1.0, True),
        (130, 256, 16, "bf16", 1.0, False),
        (77, 5, 5, "f32", 1.0, False),
        (200, 30, 4, "bf16", 1.0, True),  # an expert count that the four runs of the sum do not divide
    ],
)
def test_softmax_routing_decision_is_bit_exact_given_logits(gpu, tokens, experts, top_k, dtype, scale, use_bias):
    rng = np.random.default_rng(tokens * 1000 + experts)
    logits = (rng.standard_normal((tokens, experts)) * 2.0).astype(np.float32)
    if dtype == "bf16":
        logits = O.bf16_round(logits)
    logits[0, :] = 0.0  # a fully tied row: every score 1/E
    if tokens > 2:
        logits[1, :] = 40.0
        logits[2, : experts // 2] = -100.0  # half of the experts at the clamp of the exponent
    bias = (rng.standard_normal(experts) * 0.05).astype(np.float32) if use_bias else None
    want = O.router_from_logits(logits, bias, top_k, scale, dtype, "softmax")
    got = ops.router_from_logits(dev(logits, gpu), None if bias is None else dev(bias, gpu), top_k, scale,
                                 dtype=torch.bfloat16 if dtype == "bf16" else torch.float32, score_func="softmax")
    assert np.array_equal(host(got.scores), want.scores)
    assert np.array_equal(host(got.expert_ids), want.expert_ids)
    assert np.array_equal(host(got.weights), want.weights)
    np.testing.assert_allclose(host(got.scores).sum(-1), 1.0, rtol=1e-5)
    stats = O.router_stats(want.expert_ids, want.weights, experts)
    assert np.array_equal(host(got.expert_counts), stats.expert_counts)
    np.testing.assert_allclose(host(got.importance), stats.importance, rtol=1e-5, atol=1e-5)
    # and the sigmoid entry point is untouched by the attribute
    plain = ops.router_from_logits(dev(logits, gpu), None if bias is None else dev(bias, gpu), top_k, scale,
                                   dtype=torch.bfloat16 if dtype == "bf16" else torch.float32)
    assert np.array_equal(host(plain.scores), O.router_from_logits(logits, bias, top_k, scale, dtype).scores)


@pytest.mark.parametrize(
    "tokens,hidden,experts,top_k,dtype",
    [(64, 32, 8, 2, "f32"), (300, 1024, 16, 2, "bf16"), (1024, 2048, 64, 8, "bf16"), (513, 2048, 128, 8, "bf16"),
     (100, 72, 24, 3, "bf16"), (64, 2048, 64, 8, "bf16"), (256, 1024, 128, 8, "bf16"), (64, 512, 256, 4, "bf16"),
     (255, 512, 256, 4, "bf16")],
)
def test_softmax_router_end_to_end(gpu, tokens, hidden, experts, top_k, dtype):
    """Every projection kernel (generic, 64-token matrix-core, k-split, k-sliced + finishing workgroup)
    ends in the same epilogue: the kernel's decision is the oracle's decision on the kernel's own logits."""
    rng = np.random.default_rng(hidden + experts)
    x = rng.standard_normal((tokens, hidden)).astype(np.float32)
    w = (rng.standard_normal((hidden, experts)) * 0.02).astype(np.float32)
    bias = (rng.standard_normal(experts) * 0.005).astype(np.float32)
    got = ops.router(dev(x, gpu, dtype), dev(w, gpu, dtype), dev(bias, gpu), top_k, 1.0, return_logits=True,
                     score_func="softmax")
    sig = ops.router(dev(x, gpu, dtype), dev(w, gpu, dtype), dev(bias, gpu), top_k, 1.0, return_logits=True)
    assert torch.equal(got.logits, sig.logits)  # the projection does not depend on the score function
    own = O.router_from_logits(host(got.logits), bias, top_k, 1.0, dtype, "softmax")
    assert np.array_equal(host(got.expert_ids), own.expert_ids)
    assert np.array_equal(host(got.weights), own.weights)
    assert np.array_equal(host(got.scores), own.scores)


@pytest.mark.parametrize("name,tokens,top_k,dtype", [("C1", 512, 2, "f32"), ("C2", 1024, 2, "bf16"),
                                                     ("C3", 300, 8, "bf16"), ("C5", None, 8, "bf16")])
def test_softmax_layer_matches_oracle_and_the_stand_alone_entry_points(gpu, name, tokens, top_k, dtype):
    inp = O.make_inputs(name, seed=0, tokens=tokens)
    cfg = inp["cfg"]
    T = inp["x"].shape[0] * inp["x"].shape[1]
    x2 = inp["x"].reshape(T, cfg["H"])
    E = inp["gate"].shape[0]
    shared = None if inp["shared"] is None else tuple(dev(m, gpu, dtype) for m in inp["shared"])
    xd, wr, bias = dev(x2, gpu, dtype), dev(inp["w_router"], gpu, dtype), dev(inp["expert_bias"], gpu)
    gate, up, down = (dev(inp[k], gpu, dtype) for k in ("gate", "up", "down"))
    layer = ops.moe_forward(xd, wr, bias, gate, up, down, top_k, 1.0, shared=shared, score_func="softmax")
    route = ops.router(xd, wr, bias, top_k, 1.0, score_func="softmax")
    plan = ops.dispatch(route.expert_ids, E)
    for field in ("expert_ids", "weights", "scores", "expert_counts", "importance"):
        assert torch.equal(getattr(layer, field), getattr(route, field)), field
    for field in ("group_sizes", "offsets", "source_order", "inverse"):
        assert torch.equal(getattr(layer, field), getattr(plan, field)), field
    sigmoid_layer = ops.moe_forward(xd, wr, bias, gate, up, down, top_k, 1.0, shared=shared)
    assert not torch.equal(sigmoid_layer.scores, layer.scores)
    # the experts and the combine on the kernel's own routing, as in test_gpu_parity.check_layer_against_oracle
    ids = host(layer.expert_ids)
    d = O.dispatch(ids, E, O.cast_compute(x2, dtype))
    packed_y = O.grouped_swiglu(d.packed_x, inp["gate"], inp["up"], inp["down"], d.group_sizes, dtype)
    shared_y = None if inp["shared"] is None else O.shared_swiglu(x2, *inp["shared"], dtype)
    want = O.combine(packed_y, d.inverse, host(layer.weights), dtype, shared_y)
    if dtype == "bf16":
        assert report(f"softmax layer {name}", host(layer.y), want) <= BF16_MAX_REL
    else:
        np.testing.assert_allclose(host(layer.y), want, rtol=1e-4, atol=2e-5)


@pytest.mark.parametrize("tokens,hidden,experts,top_k,dtype,with_scores",
                         [(6, 5, 7, 3, "f32", True), (300, 256, 64, 8, "bf16", True), (129, 72, 10, 2, "bf16", False),
                          (512, 2048, 128, 8, "bf16", True)])
def test_softmax_router_gradients_match_oracle(gpu, tokens, hidden, experts, top_k, dtype, with_scores):
    rng = np.random.default_rng(11)
    x = rng.standard_normal((tokens, hidden)).astype(np.float32)
    w = (rng.standard_normal((hidden, experts)) * (0.02 if hidden >= 256 else 0.3)).astype(np.float32)
    d_weights = rng.standard_normal((tokens, top_k)).astype(np.float32)
    d_scores = rng.standard_normal((tokens, experts)).astype(np.float32) if with_scores else None
    scale = 2.5
    xd, wd = dev(x, gpu, dtype), dev(w, gpu, dtype)
    fwd = ops.router(xd, wd, None, top_k, scale, score_func="softmax")
    cast = lambda a: O.cast_compute(a, dtype)
    want = G.router_backward(cast(x), cast(w), host(fwd.expert_ids), cast(d_weights), d_scores, scale,
                             scores=host(fwd.scores), score_func="softmax")
    dx, d_w = grad.router_backward(xd, wd, fwd.scores, fwd.expert_ids, dev(d_weights, gpu, dtype),
                                   None if d_scores is None else dev(d_scores, gpu), scale, score_func="softmax")
    tag = f"softmax router grad {dtype} T={tokens} H={hidden} E={experts} K={top_k}"
    if dtype == "bf16":
        assert report(tag + " dx", host(dx), want.dx.astype(np.float32)) <= BF16_MAX_REL
        assert report(tag + " d_w_router", host(d_w), want.d_w_router.astype(np.float32)) <= BF16_MAX_REL
    else:
        np.testing.assert_allclose(host(dx), want.dx, rtol=1e-4, atol=2e-5)
        np.testing.assert_allclose(host(d_w), want.d_w_router, rtol=1e-4, atol=2e-5)


def test_softmax_layer_gradients_through_autograd_fp32(gpu):
    rng = np.random.default_rng(23)
    T, H, E, K, I, Is = 40, 24, 6, 2, 32, 16
    f32 = lambda a: a.astype(np.float32)
    x = f32(rng.standard_normal((T, H)))
    w = f32(rng.standard_normal((H, E)) * 0.3)
    gate, up = f32(rng.standard_normal((E, H, I)) * 0.2), f32(rng.standard_normal((E, H, I)) * 0.2)
    down = f32(rng.standard_normal((E, I, H)) * 0.2)
    shared = tuple(f32(rng.standard_normal(s) * 0.2) for s in ((H, Is), (H, Is), (Is, H)))
    target = f32(rng.standard_normal((T, E)) * 0.1)
    leaves = [dev(a, gpu, "f32").requires_grad_(True) for a in (x, w, gate, up, down, *shared)]
    y, scores, ids = autograd.moe_layer(leaves[0], leaves[1], None, leaves[2], leaves[3], leaves[4], K, 1.5,
                                        shared=tuple(leaves[5:]), score_func="softmax")
    loss = (y * y).sum() / T + (scores * dev(target, gpu, "f32")).sum()
    grads = torch.autograd.grad(loss, leaves)
    ref_route = O.router(x, w, None, K, 1.5, "f32", "softmax")
    assert np.array_equal(host(ids), ref_route.expert_ids), "selection differs (a near-tie in the test inputs)"
    want = G.moe_backward(x, w, gate, up, down, shared, host(ids), ref_route.weights, 2.0 * host(y) / T, target, 1.5,
                          score_func="softmax")
    refs = (want.dx, want.d_w_router, want.d_gate, want.d_up, want.d_down, *want.d_shared)
    for name, g, ref in zip(("dx", "d_w_router", "d_gate", "d_up", "d_down", "sg", "su", "sd"), grads, refs):
        np.testing.assert_allclose(host(g), ref, rtol=2e-4, atol=2e-5, err_msg=name)


def test_unknown_score_function_is_refused(gpu):
    x = torch.zeros((4, 8), device=gpu)
    w = torch.zeros((8, 4), device=gpu)
    with pytest.raises(ContractError):
        ops.router(x, w, None, 2, 1.0, score_func="tanh")
    lib = ops._lib()
    ws = torch.empty((lib.jtmoe_router_workspace_bytes(4),), dtype=torch.uint8, device=gpu)
    out = [torch.empty((4, 2), dtype=torch.int32, device=gpu), torch.empty((4, 2), device=gpu),
           torch.empty((4, 4), device=gpu), torch.empty((4,), device=gpu), torch.empty((4,), device=gpu)]
    status = lib.jtmoe_router_sf(x.data_ptr(), w.data_ptr(), None, 4, 8, 4, 2, 1.0, 7, 1, *(t.data_ptr() for t in out),
                                 None, ws.data_ptr(), ws.numel(), None)
    assert status == -1 and b"score function" in lib.jtmoe_last_error()
