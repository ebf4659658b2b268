"""MoE balancing state and update on the GPU: the consumer of the layer's expert_counts.

Host-side mirror of the reference's balancing helpers (src/jaxtitan/steps/moe_balance.py): the same
names, argument meaning and error behaviour, with the state held in torch tensors on the device
and the update itself one call of jtmoe_smebu_update.  Where the reference stacks the per-layer
counts it reads out of the model's router statistics (moe_balance.py:73-83), `zero_router_counts`
here hands out ONE [layers, experts] buffer whose rows are given to the layer calls as their
expert_counts output (`ops.moe_forward(..., expert_counts_out=counts[l])`, i.e. the
`expert_counts` pointer of `jtmoe_moe_forward`), so the
counts go from the router kernel to the update without a copy or a host round trip.
"""

from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any

import torch

from research_amd import ops
from research_amd.errors import ContractError

_POLICIES = ("none", "smebu")


@dataclass(frozen=True)
class MoeBalanceSpec:
    """The policy fields of the reference's MoeBalanceSpec (specs/model.py:15-42)."""

    name: str = "none"
    load_lr: float = 5e-4
    momentum: float = 0.5
    clamp: float = 2.0
    sequence_aux_loss_weight: float = 1e-4

    def __post_init__(self) -> None:
        if self.name not in _POLICIES:
            raise ContractError(
                f"model.trinity.moe.balance.name must be one of {sorted(_POLICIES)}, got {self.name!r}"
            )
        for field_name in ("load_lr", "momentum", "clamp"):
            value = getattr(self, field_name)
            if not isinstance(value, int | float) or isinstance(value, bool) or value <= 0.0:
                raise ContractError(f"model.trinity.moe.balance.{field_name} must be positive, got {value!r}")
        weight = self.sequence_aux_loss_weight
        if not isinstance(weight, int | float) or isinstance(weight, bool) or weight < 0.0:
            raise ContractError(
                f"model.trinity.moe.balance.sequence_aux_loss_weight must be non-negative, got {weight!r}"
            )


@dataclass(frozen=True)
class MoeBalanceState:
    """Non-gradient balancing state (moe_balance.py:22-30); momentum is [layers, experts] f32."""

    name: str
    load_lr: float
    momentum_factor: float
    clamp: float
    momentum: torch.Tensor

    @property
    def num_layers(self) -> int:
        return int(self.momentum.shape[0])


@dataclass(frozen=True)
class MoeBalanceMetrics:
    """Scalar diagnostics of one update (moe_balance.py:32-41), 0-d f32 tensors on the device."""

    max_vio: Any
    load_min: Any
    load_max: Any
    load_entropy: Any
    bias_norm: Any
    momentum_norm: Any


def initialize_moe_balance_state(expert_bias: torch.Tensor, balance: MoeBalanceSpec | None) -> MoeBalanceState | None:
    """Zero momentum shaped like the model's expert biases [layers, experts] (moe_balance.py:44-63)."""
    if balance is None or balance.name == "none":
        return None
    if balance.name != "smebu":
        raise ContractError(f"unsupported MoE balance policy {balance.name!r}")
    if not isinstance(expert_bias, torch.Tensor) or expert_bias.dim() != 2 or expert_bias.shape[0] == 0:
        raise ContractError("SMEBU balance requires at least one MoE expert_bias parameter")
    return MoeBalanceState(
        name=balance.name,
        load_lr=float(balance.load_lr),
        momentum_factor=float(balance.momentum),
        clamp=float(balance.clamp),
        momentum=torch.zeros_like(expert_bias, dtype=torch.float32),
    )


def zero_router_counts(balance: MoeBalanceState | None, device: torch.device | str | None = None) -> torch.Tensor:
    """A zero [layers, experts] f32 count buffer matching the state (moe_balance.py:66-71)."""
    if balance is None:
        return torch.zeros((0, 0), dtype=torch.float32, device=device)
    return torch.zeros_like(balance.momentum)


def _stack_stats(router_stats: tuple[Any, ...], balance: MoeBalanceState | None, field: str) -> torch.Tensor:
    if not router_stats:
        return torch.zeros((0, 0), dtype=torch.float32)
    if balance is not None and len(router_stats) != balance.num_layers:
        raise ContractError(f"MoE balance expected {balance.num_layers} router stat entries, got {len(router_stats)}")
    return torch.stack([getattr(stats, field).to(torch.float32) for stats in router_stats])


def router_counts_from_stats(router_stats: tuple[Any, ...], balance: MoeBalanceState | None) -> torch.Tensor:
    """Layer-major expert counts from the layers' RouterStats (moe_balance.py:73-83): the copying
    alternative to handing the layers rows of `zero_router_counts`."""
    return _stack_stats(router_stats, balance, "expert_counts")


def router_importance_from_stats(router_stats: tuple[Any, ...], balance: MoeBalanceState | None) -> torch.Tensor:
    """Layer-major selected-router-weight sums from the layers' RouterStats (moe_balance.py:86-94)."""
    return _stack_stats(router_stats, balance, "importance")


def apply_moe_balance_update(
    expert_bias: torch.Tensor,
    balance: MoeBalanceState | None,
    router_counts: torch.Tensor,
) -> tuple[torch.Tensor, MoeBalanceState | None, MoeBalanceMetrics]:
    """One non-gradient balancing update of the expert biases, in place (moe_balance.py:97-162).

    expert_bias [layers, experts] f32 on the GPU is updated in place and returned; the state's
    momentum tensor likewise.
    """
    if balance is None:
        zero = torch.zeros((), dtype=torch.float32, device=expert_bias.device)
        return expert_bias, None, MoeBalanceMetrics(zero, zero, zero, zero, zero, zero)
    if balance.name != "smebu":
        raise ContractError(f"unsupported MoE balance policy {balance.name!r}")
    if tuple(router_counts.shape) != tuple(balance.momentum.shape):
        raise ContractError(f"router count shape must match MoE balance state, got {tuple(router_counts.shape)}")
    metrics = ops.smebu_update(router_counts, balance.momentum, expert_bias, load_lr=balance.load_lr,
                               momentum_factor=balance.momentum_factor, clamp=balance.clamp)
    return expert_bias, replace(balance), MoeBalanceMetrics(*metrics.unbind(0))
