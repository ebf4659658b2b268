"""Host-layer contract: spec validation and the operators' refusal to run
anywhere but on the GPU (there is no CPU path to fall back to)."""

from __future__ import annotations

import pytest
import torch

from research_amd import moe, ops
from research_amd.errors import ContractError


def test_spec_validation_follows_the_reference_contract():
    ok = moe.TrinityMoeSpec(num_experts=8, top_k=2, expert_intermediate_size=64)
    assert ok.balance.name == "none" and ok.route_scale == 1.0
    assert moe.TrinityMoeSpec(4, 2, balance={"name": "smebu"}).balance.name == "smebu"
    for kwargs in (
        dict(num_experts=0, top_k=1),
        dict(num_experts=4, top_k=5),
        dict(num_experts=4, top_k=True),
        dict(num_experts=4, top_k=2, expert_intermediate_size=0),
        dict(num_experts=4, top_k=2, num_shared_experts=-1),
        dict(num_experts=4, top_k=2, route_scale=0.0),
        dict(num_experts=4, top_k=2, balance={"name": "aux"}),
        dict(num_experts=4, top_k=2, balance={"name": "smebu", "sequence_aux_loss_weight": -1.0}),
        dict(num_experts=4, top_k=2, balance=3),
    ):
        with pytest.raises(ContractError):
            moe.TrinityMoeSpec(**kwargs)


def test_router_constructor_checks():
    for kw in (dict(num_experts=3, top_k=4), dict(num_experts=3, top_k=0), dict(num_experts=3, top_k=2, route_scale=0.0)):
        with pytest.raises(ContractError):
            moe.SigmoidTopKRouter(2, dtype=torch.float32, param_dtype=torch.float32, device="cpu", **kw)


def test_layer_requires_resolved_intermediate_size():
    with pytest.raises(ContractError, match="expert_intermediate_size"):
        moe.SparseMoE(8, moe.TrinityMoeSpec(4, 2), device="cpu")


def test_operators_refuse_cpu_tensors():
    x = torch.zeros((4, 8))
    w = torch.zeros((8, 4))
    with pytest.raises(ContractError, match="GPU"):
        ops.router(x, w, None, 2)
    with pytest.raises(ContractError, match="GPU"):
        ops.dispatch(torch.zeros((4, 2), dtype=torch.int32), 4)
    with pytest.raises(ContractError, match="GPU"):
        ops.combine(torch.zeros((8, 8)), torch.zeros(8, dtype=torch.int32), torch.zeros((4, 2)))
    layer = moe.SparseMoE(8, moe.TrinityMoeSpec(4, 2, expert_intermediate_size=16), compute_dtype="float32", device="cpu")
    with pytest.raises(ContractError, match="GPU"):
        layer(torch.zeros((1, 4, 8)))
    with pytest.raises(ContractError, match="one device"):
        layer(torch.zeros((1, 4, 8)), execution=object())


def test_dtype_names():
    assert moe.dtype_from_name("bfloat16") is torch.bfloat16
    with pytest.raises(ContractError):
        moe.dtype_from_name("float16")


def test_jax_ffi_stub_fails_loudly_without_jax():
    import importlib.util

    from research_amd import jax_ffi

    if importlib.util.find_spec("jax") is not None:
        pytest.skip("jax is installed here")
    with pytest.raises(ContractError, match="jax is not installed"):
        jax_ffi.register_moe()
    assert set(jax_ffi.TARGETS.values()) == {
        "JaxtitanMoeForward", "JaxtitanMoeRouter", "JaxtitanMoeDispatch", "JaxtitanMoeGroupedSwiglu",
        "JaxtitanMoeCombine", "JaxtitanMoeForwardTrain", "JaxtitanMoeBackward", "JaxtitanRmsnorm",
        "JaxtitanFfnBlockForward", "JaxtitanMoeSmebuUpdate"}
    with pytest.raises(ContractError, match="jax is not installed"):
        jax_ffi.moe_layer(None, None, None, None, None, None, top_k=1)


def test_training_and_block_operators_refuse_cpu_tensors_and_bad_shapes():
    from research_amd import grad

    x, dy = torch.zeros((4, 8)), torch.zeros((4, 8))
    gate = up = torch.zeros((2, 8, 16))
    down = torch.zeros((2, 16, 8))
    with pytest.raises(ContractError, match="GPU"):
        grad.shared_swiglu_train(x, gate[0], up[0], down[0])
    with pytest.raises(ContractError, match="GPU"):
        grad.router_backward(x, torch.zeros((8, 2)), torch.zeros((4, 2)), torch.zeros((4, 1), dtype=torch.int32),
                             torch.zeros((4, 1)))
    with pytest.raises(ContractError, match="GPU"):
        ops.rmsnorm(x, torch.ones(8))
    with pytest.raises(ContractError, match="GPU"):
        ops.ffn_block_forward(x, torch.ones(8), torch.ones(8), 1e-6, torch.zeros((8, 2)), None, gate, up, down, 1)
    with pytest.raises(ContractError, match="GPU"):
        grad.moe_forward_train(x, torch.zeros((8, 2)), None, gate, up, down, 1)


def test_balance_spec_and_state_contract():
    """The policy checks of the reference's MoeBalanceSpec (specs/model.py:25-42) and of
    initialize_moe_balance_state (steps/moe_balance.py:44-63), which need no GPU."""
    import torch

    from research_amd import balance as B

    assert B.MoeBalanceSpec().name == "none" and B.MoeBalanceSpec(name="smebu").load_lr == 5e-4
    with pytest.raises(ContractError, match="balance.name must be one of"):
        B.MoeBalanceSpec(name="aux_free")
    for field in ("load_lr", "momentum", "clamp"):
        with pytest.raises(ContractError, match=f"balance.{field} must be positive"):
            B.MoeBalanceSpec(name="smebu", **{field: 0.0})
        with pytest.raises(ContractError, match=f"balance.{field} must be positive"):
            B.MoeBalanceSpec(name="smebu", **{field: True})
    with pytest.raises(ContractError, match="sequence_aux_loss_weight must be non-negative"):
        B.MoeBalanceSpec(name="smebu", sequence_aux_loss_weight=-1.0)
    bias = torch.zeros((3, 8))
    assert B.initialize_moe_balance_state(bias, None) is None
    assert B.initialize_moe_balance_state(bias, B.MoeBalanceSpec()) is None
    state = B.initialize_moe_balance_state(bias, B.MoeBalanceSpec(name="smebu", momentum=0.25))
    assert state.num_layers == 3 and state.momentum_factor == 0.25 and state.momentum.shape == (3, 8)
    assert state.momentum.dtype == torch.float32 and not bool(state.momentum.any())
    with pytest.raises(ContractError, match="requires at least one MoE expert_bias parameter"):
        B.initialize_moe_balance_state(torch.zeros((0, 8)), B.MoeBalanceSpec(name="smebu"))
    assert B.zero_router_counts(None).shape == (0, 0)
    assert B.zero_router_counts(state).shape == (3, 8)
    # stacking the layers' statistics (moe_balance.py:73-94)
    from types import SimpleNamespace

    stats = tuple(SimpleNamespace(expert_counts=torch.full((8,), float(i)), importance=torch.full((8,), 0.5 * i))
                  for i in range(3))
    assert B.router_counts_from_stats(stats, state)[2].tolist() == [2.0] * 8
    assert B.router_importance_from_stats(stats, state).shape == (3, 8)
    assert B.router_counts_from_stats((), state).shape == (0, 0)
    with pytest.raises(ContractError, match="MoE balance expected 3 router stat entries, got 2"):
        B.router_counts_from_stats(stats[:2], state)


def test_default_initialiser_has_the_reference_distribution():
    """nnx.initializers.lecun_normal() on [E, H, I]: variance 1 / (E * H), truncated at two standard
    deviations of the underlying normal (moe.py:164-167; jax.nn.initializers.variance_scaling)."""
    import math

    import torch

    from research_amd.moe import lecun_normal

    gen = torch.Generator().manual_seed(0)
    E, H, I = 8, 96, 160
    w = lecun_normal((E, H, I), torch.float32, torch.device("cpu"), gen)
    want_std = math.sqrt(1.0 / (E * H))
    assert abs(float(w.std()) / want_std - 1.0) < 0.02
    assert abs(float(w.mean())) < 0.02 * want_std
    assert float(w.abs().max()) <= 2.0 * want_std / 0.87962566103423978 + 1e-9  # the truncation point
    assert float(w.abs().max()) > 1.9 * want_std / 0.87962566103423978           # and samples reach it
    k = lecun_normal((H, E), torch.float32, torch.device("cpu"), gen)             # a plain [in, out] kernel
    assert abs(float(k.std()) / math.sqrt(1.0 / H) - 1.0) < 0.05
