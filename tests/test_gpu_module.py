"""The host-side mirror of the reference layer, exercised the way the
reference's own tests exercise SparseMoE and its parts
(tests/jaxtitan/test_model.py:196-322, 873-910)."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from research_amd.errors import ContractError
from research_amd.moe import (ExpertSwiGLU, LocalExpertDispatcher, SigmoidTopKRouter, SparseMoE, TrinityMoeSpec)

pytestmark = pytest.mark.gpu
F32 = torch.float32


def t(a, gpu, dtype=F32):
    return torch.as_tensor(np.asarray(a), device=gpu).to(dtype)


def test_sigmoid_top_k_router_is_deterministic_and_normalizes_weights(gpu):
    router = SigmoidTopKRouter(hidden_size=2, num_experts=3, top_k=2, dtype=F32, param_dtype=F32, device=gpu)
    router.proj.kernel.set([[0.0, 1.0, 2.0], [0.0, 0.0, 0.0]])
    x = t([[[1.0, 0.0], [0.5, 0.0]]], gpu)
    first, second = router(x), router(x)
    assert torch.equal(first.expert_ids, second.expert_ids)
    assert first.expert_ids[0, 0].tolist() == [2, 1]
    assert first.expert_ids.dtype == torch.int32 and first.expert_ids.shape == (1, 2, 2)
    assert torch.allclose(first.weights.sum(-1), torch.ones((1, 2), device=gpu))
    assert bool((first.weights > 0).all())
    assert first.scores.shape == (1, 2, 3) and first.scores.dtype == F32


def test_sigmoid_top_k_router_uses_bias_for_selection_and_unbiased_scores_for_weights(gpu):
    router = SigmoidTopKRouter(hidden_size=2, num_experts=3, top_k=2, dtype=F32, param_dtype=F32, device=gpu,
                               route_scale=1.5)
    router.proj.kernel.set([[2.0, 0.0, -2.0], [0.0, 0.0, 0.0]])
    x = t([[[1.0, 0.0]]], gpu)
    routed = router(x, expert_bias=t([0.0, 0.0, 1.0], gpu))
    s = 1.0 / (1.0 + np.exp(-np.array([2.0, 0.0, -2.0])))
    assert routed.expert_ids.tolist() == [[[2, 0]]]
    expected = np.array([s[2], s[0]]) / (s[2] + s[0]) * 1.5
    np.testing.assert_allclose(routed.weights[0, 0].cpu().numpy(), expected, rtol=2e-6)
    np.testing.assert_allclose(routed.weights.sum(-1).cpu().numpy(), [[1.5]], rtol=1e-6)
    with pytest.raises(ContractError, match="expert_bias must have shape"):
        router(x, expert_bias=t([0.0, 1.0], gpu))


def test_expert_swiglu_matches_manual_selected_expert_calculation(gpu, kat):
    c = kat["expert_swiglu_manual"]
    experts = ExpertSwiGLU(hidden_size=2, intermediate_size=2, num_experts=2, dtype=F32, param_dtype=F32, device=gpu)
    experts.gate.set(c["gate"]); experts.up.set(c["up"]); experts.down.set(c["down"])
    x = t([c["x"]], gpu)
    ids = t([c["expert_ids"]], gpu, torch.int32)
    w = t([c["weights"]], gpu)
    actual = experts(x, ids, w)
    np.testing.assert_allclose(actual.cpu().numpy()[0], c["expected"]["out"], rtol=1e-5)
    # local_forward returns the unweighted per-assignment outputs [.., K, H]
    per = experts.local_forward(x, ids)
    assert per.shape == (1, 1, 2, 2)
    np.testing.assert_allclose((per * w[..., None]).sum(-2).cpu().numpy(), actual.cpu().numpy(), rtol=1e-6)
    with pytest.raises(ContractError, match="must equal weights shape"):
        experts(x, ids, w[..., :1])


def test_local_expert_dispatcher_matches_expert_swiglu_reference(gpu, kat):
    c = kat["local_dispatcher"]
    experts = ExpertSwiGLU(hidden_size=2, intermediate_size=2, num_experts=2, dtype=F32, param_dtype=F32, device=gpu)
    experts.gate.set(c["gate"]); experts.up.set(c["up"]); experts.down.set(c["down"])
    x, ids, w = t([c["x"]], gpu), t([c["expert_ids"]], gpu, torch.int32), t([c["weights"]], gpu)
    dispatched = LocalExpertDispatcher()(experts, x, ids, w)
    reference = experts(x, ids, w)
    assert torch.allclose(dispatched, reference)
    np.testing.assert_allclose(dispatched.cpu().numpy()[0], c["expected"]["out"], rtol=1e-5)


def test_sparse_moe_adds_shared_expert_output(gpu):
    spec = TrinityMoeSpec(num_experts=1, top_k=1, expert_intermediate_size=24, num_shared_experts=1)
    moe = SparseMoE(16, spec, compute_dtype="float32", device=gpu)
    assert moe.shared_experts is not None
    for p in (moe.experts.gate, moe.experts.up, moe.experts.down):
        p.set(torch.zeros_like(p.value))
    x = torch.ones((1, 1, 16), device=gpu)
    actual = moe(x)
    assert torch.allclose(actual, moe.shared_experts(x))
    assert float(actual.abs().max()) > 0


def test_forward_with_output_emits_router_stats_and_aux_loss_when_balanced(gpu):
    spec = TrinityMoeSpec(num_experts=3, top_k=2, expert_intermediate_size=32, balance={"name": "smebu"})
    moe = SparseMoE(16, spec, compute_dtype="float32", device=gpu, seed=0)
    x = torch.randn((2, 4, 16), generator=torch.Generator().manual_seed(1)).to(gpu)
    out, aux, stats = moe.forward_with_output(x, name="layer1.moe", layer_index=1)
    assert out.shape == x.shape and len(aux) == 1 and len(stats) == 1
    s = stats[0]
    assert s.name == "layer1.moe" and s.layer_index == 1
    assert s.expert_counts.shape == (3,) and s.importance.shape == (3,)
    assert float(s.expert_counts.sum()) == 2 * 4 * 2
    assert float(s.importance.sum()) == pytest.approx(2 * 4, abs=1e-2)
    assert s.max_vio.shape == () and float(s.total_assignments) == 16
    assert aux[0].name == "moe_sequence_balance" and float(aux[0].weight) == pytest.approx(1e-4)
    route = moe.route(x)
    want = O.sequence_balance_loss(route.expert_ids.cpu().numpy(), route.scores.cpu().numpy(), 2)
    assert float(aux[0].value) == pytest.approx(float(want), rel=1e-5)
    # __call__ is the same math without the records
    assert torch.equal(moe(x), out)
    plain = SparseMoE(16, TrinityMoeSpec(3, 2, expert_intermediate_size=32), compute_dtype="float32", device=gpu)
    assert plain.forward_with_output(x, name="m", layer_index=0)[1] == ()


def test_bf16_layer_with_fp32_params_matches_oracle(gpu):
    spec = TrinityMoeSpec(num_experts=8, top_k=2, expert_intermediate_size=128, num_shared_experts=1)
    moe = SparseMoE(64, spec, compute_dtype="bfloat16", param_dtype="float32", device=gpu, seed=3)
    x = torch.randn((2, 100, 64), generator=torch.Generator().manual_seed(2)).to(gpu)
    y = moe(x)
    assert y.dtype == torch.bfloat16 and y.shape == x.shape
    npy = lambda p: p.value.float().cpu().numpy()
    ref = O.moe_forward(x.cpu().numpy(), npy(moe.router.proj.kernel), None, npy(moe.experts.gate), npy(moe.experts.up),
                        npy(moe.experts.down), 2, 1.0, "bf16",
                        shared=tuple(npy(l.kernel) for l in (moe.shared_experts.gate, moe.shared_experts.up,
                                                             moe.shared_experts.down)))
    got = y.float().cpu().numpy()
    same = np.all(moe.route(x).expert_ids.cpu().numpy().reshape(-1, 2) == ref.route.expert_ids, axis=1)
    assert same.mean() > 0.98
    err = np.max(np.abs(got.reshape(-1, 64)[same] - ref.y.reshape(-1, 64)[same])) / np.max(np.abs(ref.y))
    assert err <= 2e-2


def test_graph_replay_matches_eager_on_every_replay(gpu):
    """The captured layer gives the eager result on each of several replays with fresh inputs, with
    eager work and synchronisations between the replays."""
    from oracle import moe_oracle as O
    from research_amd import ops
    from research_amd.graph import GraphedLayer

    inp = O.make_inputs("C5", seed=0)
    cfg = inp["cfg"]
    bf = lambda a: torch.from_numpy(a).to(gpu).to(torch.bfloat16).contiguous()
    params = (bf(inp["w_router"]), torch.from_numpy(inp["expert_bias"]).to(gpu), bf(inp["gate"]), bf(inp["up"]),
              bf(inp["down"]))
    x0 = bf(inp["x"].reshape(-1, cfg["H"]))
    layer = GraphedLayer(x0, *params, cfg["K"], 1.0)
    gen = torch.Generator(device=gpu).manual_seed(5)
    for i in range(4):
        x = torch.randn(x0.shape, device=gpu, generator=gen).to(torch.bfloat16) if i else x0
        eager = ops.moe_forward(x, *params, cfg["K"], 1.0)
        torch.cuda.synchronize()
        got = layer.replay(x)
        torch.cuda.synchronize()
        assert torch.equal(got.y, eager.y), f"replay {i}"
        assert torch.equal(got.expert_ids, eager.expert_ids) and torch.equal(got.weights, eager.weights)
        assert torch.equal(got.expert_counts, eager.expert_counts) and torch.equal(got.inverse, eager.inverse)
        (eager.y.float() * 2).sum().item()  # unrelated eager work between the replays


@pytest.mark.parametrize("tokens,hidden,experts,top_k,d_ff,shared_width",
                         [(600, 512, 16, 2, 256, 128),   # router, histogram, rank, four GEMMs, combine
                          (200, 256, 64, 8, 64, 0),      # the small-batch router with the plan in its last workgroup
                          (3000, 1024, 128, 8, 128, 0)])  # many short groups
def test_graph_replay_of_the_other_layer_paths(gpu, tokens, hidden, experts, top_k, d_ff, shared_width):
    """The same for the launches a call makes outside the decode path: every replay, with eager work and
    synchronisations between them, gives what the eager call gives on the same input."""
    from research_amd import ops
    from research_amd.graph import GraphedLayer

    gen = torch.Generator(device=gpu).manual_seed(tokens)
    draw = lambda *shape, std=1.0: (torch.randn(*shape, device=gpu, generator=gen) * std).to(torch.bfloat16)
    params = (draw(hidden, experts, std=0.1), None, draw(experts, hidden, d_ff, std=0.05),
              draw(experts, hidden, d_ff, std=0.05), draw(experts, d_ff, hidden, std=0.05))
    shared = None
    if shared_width:
        shared = (draw(hidden, shared_width, std=0.05), draw(hidden, shared_width, std=0.05),
                  draw(shared_width, hidden, std=0.05))
    layer = GraphedLayer(draw(tokens, hidden), *params, top_k, 1.0, shared=shared)
    for i in range(4):
        x = draw(tokens, hidden)
        eager = ops.moe_forward(x, *params, top_k, 1.0, shared=shared)
        torch.cuda.synchronize()
        got = layer.replay(x)
        torch.cuda.synchronize()
        for name in ("y", "expert_ids", "weights", "scores", "expert_counts", "importance", "group_sizes", "inverse"):
            assert torch.equal(getattr(got, name), getattr(eager, name)), f"replay {i}: {name}"
        (eager.y.float() * 2).sum().item()  # unrelated eager work between the replays
