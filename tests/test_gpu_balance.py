"""The SMEBU balancing update on the GPU against the oracle, called the way the reference's train
step calls it (src/jaxtitan/steps/moe_balance.py:97-162; tests/jaxtitan/test_train_step.py:352-418).

All arithmetic is float32; the kernel and NumPy sum in different orders and use different tanh / log
routines, so results are held to rtol = atol = 1e-5 relative to the step size (load_lr), the bar of
the reference's fp32 dispatcher tests.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from research_amd import balance as B
from research_amd import ops
from research_amd.errors import ContractError
from test_gpu_parity import dev, host, random_problem

pytestmark = pytest.mark.gpu


def check_update(gpu, counts, momentum, bias, spec: B.MoeBalanceSpec):
    want = O.smebu_update(counts, momentum, bias, spec.load_lr, spec.momentum, spec.clamp)
    state = B.initialize_moe_balance_state(torch.as_tensor(bias, device=gpu), spec)
    state.momentum.copy_(torch.as_tensor(momentum, device=gpu))
    bias_d = torch.as_tensor(bias, device=gpu).clone()
    out_bias, next_state, metrics = B.apply_moe_balance_update(bias_d, state, torch.as_tensor(counts, device=gpu))
    assert out_bias.data_ptr() == bias_d.data_ptr()  # in place
    tol = dict(rtol=1e-5, atol=1e-5 * spec.load_lr)
    np.testing.assert_allclose(host(next_state.momentum), want.momentum, **tol)
    np.testing.assert_allclose(host(out_bias), want.expert_bias, rtol=1e-5, atol=1e-7)
    for name in ("max_vio", "load_min", "load_max", "load_entropy", "bias_norm", "momentum_norm"):
        np.testing.assert_allclose(float(getattr(metrics, name)), float(getattr(want, name)), rtol=2e-5, atol=1e-7,
                                   err_msg=name)
    return next_state, out_bias, metrics


@pytest.mark.parametrize("layers,experts", [(1, 2), (1, 3), (2, 8), (5, 64), (3, 128), (2, 256), (1, 300), (40, 64)])
def test_update_matches_oracle(gpu, layers, experts):
    rng = np.random.default_rng(layers * 1000 + experts)
    counts = rng.integers(0, 5000, size=(layers, experts)).astype(np.float32)
    counts[0, 0] = 0.0
    momentum = (rng.standard_normal((layers, experts)) * 2e-4).astype(np.float32)
    bias = (rng.standard_normal((layers, experts)) * 1e-2).astype(np.float32)
    check_update(gpu, counts, momentum, bias, B.MoeBalanceSpec(name="smebu"))
    check_update(gpu, counts, momentum, bias, B.MoeBalanceSpec(name="smebu", load_lr=1e-2, momentum=0.9, clamp=0.5))


def test_from_zero_state_and_repeated_steps(gpu):
    # test_train_step.py:382-384: after one step from zeros the bias equals the momentum
    rng = np.random.default_rng(5)
    counts = rng.integers(0, 50, size=(2, 3)).astype(np.float32)
    zeros = np.zeros_like(counts)
    spec = B.MoeBalanceSpec(name="smebu", load_lr=1e-2, momentum=0.5, clamp=2.0)
    state, bias, _ = check_update(gpu, counts, zeros, zeros, spec)
    assert bool(state.momentum.any())
    assert torch.allclose(bias, state.momentum, atol=1e-6)
    # a second step continues from the first one's state, as the train state carries it
    m1, b1 = host(state.momentum), host(bias)
    check_update(gpu, counts[::-1].copy(), m1, b1, spec)
    # doubled counts (two accumulated micro-batches) give the same momentum (:414-418)
    again, _, _ = check_update(gpu, counts * 2, zeros, zeros, spec)
    assert torch.allclose(again.momentum, state.momentum, rtol=1e-6, atol=1e-9)


def test_counts_go_from_the_layer_to_the_update_without_a_copy(gpu):
    """Rows of one [layers, experts] buffer are the layers' expert_counts outputs; the update reads it as is."""
    tokens, hidden, experts, top_k, inter = 96, 64, 8, 2, 64
    spec = B.MoeBalanceSpec(name="smebu", load_lr=1e-2)
    bias = torch.zeros((2, experts), dtype=torch.float32, device=gpu)
    state = B.initialize_moe_balance_state(bias, spec)
    counts = B.zero_router_counts(state)
    assert counts.shape == (2, experts) and not bool(counts.any())
    want_counts = []
    for layer in range(2):
        x, gate, up, down, _, _ = random_problem(40 + layer, tokens, hidden, experts, top_k, inter)
        w_router = np.random.default_rng(layer).standard_normal((hidden, experts)).astype(np.float32)
        res = ops.moe_forward(dev(x, gpu, "bf16"), dev(w_router, gpu, "bf16"), bias[layer], dev(gate, gpu, "bf16"),
                              dev(up, gpu, "bf16"), dev(down, gpu, "bf16"), top_k, expert_counts_out=counts[layer])
        assert res.expert_counts.data_ptr() == counts[layer].data_ptr()
        want_counts.append(np.bincount(host(res.expert_ids).reshape(-1), minlength=experts).astype(np.float32))
    assert np.array_equal(host(counts), np.stack(want_counts))
    want = O.smebu_update(np.stack(want_counts), np.zeros((2, experts), np.float32), np.zeros((2, experts), np.float32),
                          spec.load_lr, spec.momentum, spec.clamp)
    _, state, metrics = B.apply_moe_balance_update(bias, state, counts)
    np.testing.assert_allclose(host(bias), want.expert_bias, rtol=1e-5, atol=1e-9)
    np.testing.assert_allclose(float(metrics.max_vio), float(want.max_vio), rtol=1e-5)
    # the biased router of the next step sees the update: overloaded experts were pushed down
    heavy = int(np.argmax(want_counts[0]))
    assert float(bias[0, heavy]) < 0.0


def test_contract_errors(gpu):
    spec = B.MoeBalanceSpec(name="smebu")
    bias = torch.zeros((2, 4), dtype=torch.float32, device=gpu)
    state = B.initialize_moe_balance_state(bias, spec)
    with pytest.raises(ContractError, match="router count shape must match MoE balance state"):
        B.apply_moe_balance_update(bias, state, torch.zeros((1, 4), dtype=torch.float32, device=gpu))
    with pytest.raises(ContractError, match="must have dtype"):
        ops.smebu_update(torch.zeros((2, 4), dtype=torch.float64, device=gpu), state.momentum, bias, load_lr=1e-3,
                         momentum_factor=0.5, clamp=2.0)
    with pytest.raises(ContractError, match="must be positive"):
        ops.smebu_update(torch.zeros((2, 4), dtype=torch.float32, device=gpu), state.momentum, bias, load_lr=0.0,
                         momentum_factor=0.5, clamp=2.0)
    # no policy: nothing happens, zero metrics (moe_balance.py:104-106)
    same, none_state, metrics = B.apply_moe_balance_update(bias, None, torch.zeros((0, 0), device=gpu))
    assert same is bias and none_state is None and float(metrics.max_vio) == 0.0
    assert B.initialize_moe_balance_state(bias, B.MoeBalanceSpec()) is None
