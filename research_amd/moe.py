"""Host-side mirror of the reference's MoE layer interface.

Class and method names, argument meaning and error behaviour follow
src/jaxtitan/models/components/moe.py (SigmoidTopKRouter :98-147, ExpertSwiGLU
:150-195, LocalExpertDispatcher :198-202, SharedSwiGLU :319-364, SparseMoE
:367-446), the output records of src/jaxtitan/models/output.py:8-38 and the
shape contract of src/jaxtitan/specs/model.py:16-91.  Parameters are torch
tensors on the GPU; all arithmetic of the forward pass is done by libjtmoe.

Differences that are part of the boundary: parameters are stored in
``param_dtype`` and cast to the compute dtype when they change (the reference
casts on every call, moe.py:182-184); the module is forward-only.
"""

from __future__ import annotations

from collections.abc import Mapping
from dataclasses import dataclass, field
import math
from typing import Any, Callable

import torch

from research_amd import ops
from research_amd.errors import ContractError

_MOE_BALANCE_POLICIES = {"none", "smebu"}
_DTYPE_NAMES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dtype_from_name(name: str | torch.dtype) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in _DTYPE_NAMES.values():
            raise ContractError(f"dtype must be float32 or bfloat16, got {name}")
        return name
    try:
        return _DTYPE_NAMES[name]
    except KeyError as exc:
        raise ContractError(f"dtype must be one of {sorted(_DTYPE_NAMES)}, got {name!r}") from exc


# ---------------------------------------------------------------------------
# specs (specs/model.py:16-91)
# ---------------------------------------------------------------------------
@dataclass(frozen=True)
class MoeBalanceSpec:
    name: str = "none"
    load_lr: float = 5e-4
    momentum: float = 0.5
    clamp: float = 2.0
    sequence_aux_loss_weight: float = 1e-4

    def __post_init__(self) -> None:
        if self.name not in _MOE_BALANCE_POLICIES:
            raise ContractError(
                f"model.trinity.moe.balance.name must be one of {sorted(_MOE_BALANCE_POLICIES)}, got {self.name!r}"
            )
        for field_name in ("load_lr", "momentum", "clamp"):
            value = getattr(self, field_name)
            if not isinstance(value, (int, float)) or isinstance(value, bool) or value <= 0.0:
                raise ContractError(f"model.trinity.moe.balance.{field_name} must be positive, got {value!r}")
        value = self.sequence_aux_loss_weight
        if not isinstance(value, (int, float)) or isinstance(value, bool) or value < 0.0:
            raise ContractError(
                f"model.trinity.moe.balance.sequence_aux_loss_weight must be non-negative, got {value!r}"
            )


@dataclass(frozen=True)
class TrinityMoeSpec:
    num_experts: int
    top_k: int
    expert_intermediate_size: int | None = None
    num_shared_experts: int = 0
    route_scale: float = 1.0
    balance: MoeBalanceSpec | Mapping[str, Any] = field(default_factory=MoeBalanceSpec)

    def __post_init__(self) -> None:
        balance = self.balance
        if isinstance(balance, Mapping):
            object.__setattr__(self, "balance", MoeBalanceSpec(**dict(balance)))
        elif not isinstance(balance, MoeBalanceSpec):
            raise ContractError("model.trinity.moe.balance must be a MoeBalanceSpec or mapping")
        for field_name in ("num_experts", "top_k"):
            value = getattr(self, field_name)
            if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
                raise ContractError(f"model.trinity.moe.{field_name} must be a positive integer, got {value!r}")
        if self.top_k > self.num_experts:
            raise ContractError("model.trinity.moe.top_k must be <= model.trinity.moe.num_experts")
        if self.expert_intermediate_size is not None:
            value = self.expert_intermediate_size
            if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
                raise ContractError(
                    f"model.trinity.moe.expert_intermediate_size must be a positive integer, got {value!r}"
                )
        value = self.num_shared_experts
        if not isinstance(value, int) or isinstance(value, bool) or value < 0:
            raise ContractError(f"model.trinity.moe.num_shared_experts must be a non-negative integer, got {value!r}")
        value = self.route_scale
        if not isinstance(value, (int, float)) or isinstance(value, bool) or value <= 0.0:
            raise ContractError(f"model.trinity.moe.route_scale must be positive, got {value!r}")


# ---------------------------------------------------------------------------
# output records (models/output.py:8-38)
# ---------------------------------------------------------------------------
@dataclass
class AuxLoss:
    name: str
    value: Any
    weight: Any = 1.0


@dataclass
class RouterStats:
    name: str
    layer_index: int
    expert_counts: Any
    importance: Any
    total_assignments: Any
    load_min: Any
    load_max: Any
    load_mean: Any
    max_vio: Any
    load_entropy: Any


@dataclass(frozen=True)
class RouterOutput:
    """Selected expert ids and normalized routing weights (moe.py:89-95)."""

    expert_ids: torch.Tensor
    weights: torch.Tensor
    scores: torch.Tensor
    expert_counts: torch.Tensor | None = None
    importance: torch.Tensor | None = None


# ---------------------------------------------------------------------------
# parameters
# ---------------------------------------------------------------------------
class Param:
    """A parameter stored in param_dtype with a cached compute-dtype view."""

    def __init__(self, value: torch.Tensor):
        self.value = value
        self._cast: torch.Tensor | None = None
        self._cast_key: tuple | None = None

    def set(self, value: torch.Tensor | Any) -> None:
        new = torch.as_tensor(value, dtype=self.value.dtype, device=self.value.device)
        if tuple(new.shape) != tuple(self.value.shape):
            raise ContractError(f"parameter shape {list(new.shape)} must equal {list(self.value.shape)}")
        self.value = new.contiguous()
        self._cast = None

    def as_dtype(self, dtype: torch.dtype) -> torch.Tensor:
        if self.value.dtype == dtype:
            return self.value
        key = (dtype, self.value.data_ptr(), self.value._version)
        if self._cast is None or self._cast_key != key:
            self._cast = self.value.to(dtype).contiguous()
            self._cast_key = key
        return self._cast


_TRUNCATED_NORMAL_STD = 0.87962566103423978  # standard deviation of N(0, 1) truncated to [-2, 2]


def lecun_normal(shape: tuple[int, ...], dtype: torch.dtype, device: torch.device, generator: torch.Generator) -> torch.Tensor:
    """The distribution of the reference's default initialiser, nnx.initializers.lecun_normal()
    (moe.py:164-167): variance scaling 1 / fan_in with a normal truncated at two standard deviations.

    Axis -2 is the input axis and -1 the output axis; every other axis counts into the receptive field,
    so for the expert tensors [E, H, I] fan_in = E * H (the product of all axes but the last), as JAX
    computes it.  Only the distribution can be matched, not JAX's random stream.
    """
    fan_in = 1
    for n in shape[:-1]:
        fan_in *= int(n)
    values = torch.empty(shape, dtype=torch.float32)
    torch.nn.init.trunc_normal_(values, mean=0.0, std=1.0, a=-2.0, b=2.0, generator=generator)
    values *= math.sqrt(1.0 / max(fan_in, 1)) / _TRUNCATED_NORMAL_STD
    return values.to(dtype).to(device)


KernelInit = Callable[[tuple[int, ...], torch.dtype, torch.device, torch.Generator], torch.Tensor]


def _flatten_tokens(x: torch.Tensor) -> tuple[torch.Tensor, tuple[int, ...]]:
    lead = tuple(x.shape[:-1])
    return x.reshape(-1, x.shape[-1]).contiguous(), lead


class Linear:
    """Bias-free linear layer holding ``kernel`` [in, out]."""

    def __init__(self, in_features, out_features, *, dtype, param_dtype, device, generator, kernel_init=None):
        init = lecun_normal if kernel_init is None else kernel_init
        self.kernel = Param(init((in_features, out_features), param_dtype, device, generator))
        self.dtype = dtype
        self.param_dtype = param_dtype


# ---------------------------------------------------------------------------
# router (moe.py:98-147)
# ---------------------------------------------------------------------------
class SigmoidTopKRouter:
    """Deterministic sigmoid top-k router."""

    def __init__(
        self,
        hidden_size: int,
        num_experts: int,
        top_k: int,
        *,
        dtype: torch.dtype,
        param_dtype: torch.dtype,
        device: torch.device | str = "cuda",
        generator: torch.Generator | None = None,
        route_scale: float = 1.0,
        kernel_init: KernelInit | None = None,
    ):
        if top_k <= 0 or num_experts <= 0 or top_k > num_experts:
            raise ContractError("router top_k must be positive and <= num_experts")
        if route_scale <= 0.0:
            raise ContractError(f"router route_scale must be positive, got {route_scale}")
        generator = generator or torch.Generator().manual_seed(0)
        self.proj = Linear(hidden_size, num_experts, dtype=dtype, param_dtype=param_dtype, device=torch.device(device),
                           generator=generator, kernel_init=kernel_init)
        self.num_experts = num_experts
        self.top_k = top_k
        self.route_scale = float(route_scale)
        self.dtype = dtype

    def __call__(self, x: torch.Tensor, expert_bias: torch.Tensor | None = None) -> RouterOutput:
        if expert_bias is not None:
            expert_bias = torch.as_tensor(expert_bias, dtype=torch.float32, device=x.device).contiguous()
            if tuple(expert_bias.shape) != (self.num_experts,):
                raise ContractError(
                    f"expert_bias must have shape [{self.num_experts}], got {tuple(expert_bias.shape)}"
                )
        flat, lead = _flatten_tokens(x.to(self.dtype))
        result = ops.router(flat, self.proj.kernel.as_dtype(self.dtype), expert_bias, self.top_k, self.route_scale)
        weights = result.weights if x.dtype == self.dtype else result.weights.to(x.dtype)
        return RouterOutput(
            expert_ids=result.expert_ids.reshape(*lead, self.top_k),
            weights=weights.reshape(*lead, self.top_k),
            scores=result.scores.reshape(*lead, self.num_experts),
            expert_counts=result.expert_counts,
            importance=result.importance,
        )


# ---------------------------------------------------------------------------
# routed experts (moe.py:150-202)
# ---------------------------------------------------------------------------
class ExpertSwiGLU:
    """Selected-expert SwiGLU feed-forward block."""

    def __init__(
        self,
        hidden_size: int,
        intermediate_size: int,
        num_experts: int,
        *,
        dtype: torch.dtype,
        param_dtype: torch.dtype,
        device: torch.device | str = "cuda",
        generator: torch.Generator | None = None,
        kernel_init: KernelInit | None = None,
    ):
        init = lecun_normal if kernel_init is None else kernel_init
        generator = generator or torch.Generator().manual_seed(0)
        device = torch.device(device)
        self.gate = Param(init((num_experts, hidden_size, intermediate_size), param_dtype, device, generator))
        self.up = Param(init((num_experts, hidden_size, intermediate_size), param_dtype, device, generator))
        self.down = Param(init((num_experts, intermediate_size, hidden_size), param_dtype, device, generator))
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.num_experts = num_experts
        self.dtype = dtype
        self.param_dtype = param_dtype

    def _packed_forward(self, x: torch.Tensor, expert_ids: torch.Tensor):
        if tuple(expert_ids.shape[:-1]) != tuple(x.shape[:-1]):
            raise ContractError("expert routing shape must match input batch and sequence dimensions")
        flat, lead = _flatten_tokens(x.to(self.dtype))
        ids = expert_ids.to(torch.int32).reshape(-1, expert_ids.shape[-1]).contiguous()
        disp = ops.dispatch(ids, self.num_experts, flat)
        packed_y = ops.grouped_swiglu(
            disp.packed_x, self.gate.as_dtype(self.dtype), self.up.as_dtype(self.dtype),
            self.down.as_dtype(self.dtype), disp.group_sizes, disp.offsets,
        )
        return packed_y, disp, lead

    def local_forward(self, x: torch.Tensor, expert_ids: torch.Tensor) -> torch.Tensor:
        """Selected expert outputs [..., K, H] without route weights (moe.py:174-188)."""
        packed_y, disp, lead = self._packed_forward(x, expert_ids)
        rows = packed_y.shape[0]
        ones = torch.ones((rows, 1), dtype=self.dtype, device=packed_y.device)
        per_assignment = ops.combine(packed_y, disp.inverse, ones)  # y[a] = packed_y[inverse[a]] * 1
        return per_assignment.reshape(*lead, expert_ids.shape[-1], self.hidden_size)

    def __call__(self, x: torch.Tensor, expert_ids: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
        if tuple(expert_ids.shape) != tuple(weights.shape):
            raise ContractError(
                f"expert_ids shape {tuple(expert_ids.shape)} must equal weights shape {tuple(weights.shape)}"
            )
        packed_y, disp, lead = self._packed_forward(x, expert_ids)
        w = weights.to(self.dtype).reshape(-1, weights.shape[-1]).contiguous()
        return ops.combine(packed_y, disp.inverse, w).reshape(*lead, self.hidden_size)


class LocalExpertDispatcher:
    """Expert dispatcher for local routed experts (moe.py:198-202)."""

    def __call__(self, experts: ExpertSwiGLU, x: torch.Tensor, expert_ids: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
        return experts(x, expert_ids, weights)


# ---------------------------------------------------------------------------
# shared experts (moe.py:319-364)
# ---------------------------------------------------------------------------
class SharedSwiGLU:
    """Always-on shared expert path with ordinary dense FFN matrices."""

    def __init__(self, hidden_size, intermediate_size, *, dtype, param_dtype, device="cuda", generator=None,
                 kernel_init=None):
        generator = generator or torch.Generator().manual_seed(0)
        kw = dict(dtype=dtype, param_dtype=param_dtype, device=torch.device(device), generator=generator,
                  kernel_init=kernel_init)
        self.gate = Linear(hidden_size, intermediate_size, **kw)
        self.up = Linear(hidden_size, intermediate_size, **kw)
        self.down = Linear(intermediate_size, hidden_size, **kw)
        self.dtype = dtype

    def matrices(self) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        return (self.gate.kernel.as_dtype(self.dtype), self.up.kernel.as_dtype(self.dtype),
                self.down.kernel.as_dtype(self.dtype))

    def __call__(self, x: torch.Tensor, execution: Any | None = None) -> torch.Tensor:
        if execution is not None:
            raise ContractError("this build runs on one device: execution must be None")
        flat, lead = _flatten_tokens(x.to(self.dtype))
        return ops.shared_swiglu(flat, *self.matrices()).reshape(*lead, flat.shape[-1])


# ---------------------------------------------------------------------------
# the layer (moe.py:367-446)
# ---------------------------------------------------------------------------
def _derive_stats(name: str, layer_index: int, counts: torch.Tensor, importance: torch.Tensor, num_experts: int) -> RouterStats:
    """The scalar fields of RouterStats from expert_counts (moe.py:806-813), computed on the device."""
    s = ops.router_stats(counts)
    return RouterStats(name, layer_index, counts, importance, total_assignments=s[0], load_min=s[1], load_max=s[2],
                       load_mean=s[3], max_vio=s[4], load_entropy=s[5])


class SparseMoE:
    """Sparse selected-expert feed-forward module."""

    def __init__(
        self,
        hidden_size: int,
        moe: TrinityMoeSpec,
        *,
        compute_dtype: str | torch.dtype = "bfloat16",
        param_dtype: str | torch.dtype = "float32",
        device: torch.device | str = "cuda",
        seed: int = 0,
        kernel_init: KernelInit | None = None,
    ):
        if moe.expert_intermediate_size is None:
            raise ContractError("model.trinity.moe.expert_intermediate_size must be resolved before model construction")
        dtype = dtype_from_name(compute_dtype)
        pdtype = dtype_from_name(param_dtype)
        device = torch.device(device)
        generator = torch.Generator().manual_seed(seed)
        self.hidden_size = hidden_size
        self.dtype = dtype
        self.router = SigmoidTopKRouter(hidden_size, moe.num_experts, moe.top_k, dtype=dtype, param_dtype=pdtype,
                                        device=device, generator=generator, route_scale=moe.route_scale,
                                        kernel_init=kernel_init)
        self.expert_bias = Param(torch.zeros((moe.num_experts,), dtype=torch.float32, device=device))
        self.balance_name = moe.balance.name
        self.sequence_aux_loss_weight = float(moe.balance.sequence_aux_loss_weight)
        self.experts = ExpertSwiGLU(hidden_size, moe.expert_intermediate_size, moe.num_experts, dtype=dtype,
                                    param_dtype=pdtype, device=device, generator=generator, kernel_init=kernel_init)
        self.dispatcher = LocalExpertDispatcher()
        self.shared_experts: SharedSwiGLU | None = None
        if moe.num_shared_experts > 0:
            self.shared_experts = SharedSwiGLU(hidden_size, moe.expert_intermediate_size * moe.num_shared_experts,
                                               dtype=dtype, param_dtype=pdtype, device=device, generator=generator,
                                               kernel_init=kernel_init)

    def route(self, x: torch.Tensor) -> RouterOutput:
        return self.router(x, expert_bias=self.expert_bias.value)

    def _layer(self, x: torch.Tensor, execution: Any | None) -> tuple[torch.Tensor, ops.LayerResult, tuple[int, ...]]:
        if execution is not None:
            raise ContractError("this build runs on one device: execution must be None")
        if x.shape[-1] != self.hidden_size:
            raise ContractError(f"input hidden size {x.shape[-1]} must equal {self.hidden_size}")
        flat, lead = _flatten_tokens(x.to(self.dtype))
        e = self.experts
        result = ops.moe_forward(
            flat, self.router.proj.kernel.as_dtype(self.dtype), self.expert_bias.value,
            e.gate.as_dtype(self.dtype), e.up.as_dtype(self.dtype), e.down.as_dtype(self.dtype),
            self.router.top_k, self.router.route_scale,
            shared=None if self.shared_experts is None else self.shared_experts.matrices(),
        )
        return result.y.reshape(*lead, self.hidden_size), result, lead

    def __call__(self, x: torch.Tensor, execution: Any | None = None) -> torch.Tensor:
        return self._layer(x, execution)[0]

    def forward_with_output(
        self,
        x: torch.Tensor,
        *,
        name: str,
        layer_index: int,
        execution: Any | None = None,
    ) -> tuple[torch.Tensor, tuple[AuxLoss, ...], tuple[RouterStats, ...]]:
        output, result, lead = self._layer(x, execution)
        stats = _derive_stats(name, layer_index, result.expert_counts, result.importance, self.experts.num_experts)
        aux_losses: tuple[AuxLoss, ...] = ()
        if self.balance_name == "smebu" and self.sequence_aux_loss_weight > 0.0:
            if len(lead) != 2:
                raise ContractError(f"router scores must have shape [batch, seq, experts], got {list(lead)} + [E]")
            batch, seq_len = lead
            loss = ops.sequence_balance_loss(
                result.expert_ids.reshape(batch, seq_len, self.router.top_k),
                result.scores.reshape(batch, seq_len, self.experts.num_experts),
                top_k=self.router.top_k,
            )
            aux_losses = (
                AuxLoss(
                    name="moe_sequence_balance",
                    value=loss,
                    weight=torch.tensor(self.sequence_aux_loss_weight, dtype=torch.float32, device=x.device),
                ),
            )
        return output, aux_losses, (stats,)
