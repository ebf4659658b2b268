"""Training-side operators: forward passes that keep residuals and the vector-Jacobian
products of the layer's operators, on torch tensors over the native library.

The reference trains ``SparseMoE`` through ``jax.grad`` and asks a forward-only kernel to
bring its own VJP before it may replace a training component
(docs/kernel_backend_design.md:120-128); the functions here are the host side of that VJP.
As in ``ops``, torch only holds device memory and the stream; there is no CPU path.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from research_amd import ops
from research_amd.errors import ContractError
from research_amd.ops import _check, _code, _lib, _ptr, _raise, _stream, _workspace


@dataclass
class ExpertResiduals:
    gate_pre: torch.Tensor  # [A,I] round(Xp Wg[e])
    up_pre: torch.Tensor  # [A,I] round(Xp Wu[e])


def _expert_shapes(x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor):
    _check(x, "x")
    if x.dim() != 2:
        raise ContractError(f"x must have shape [tokens, hidden], got {list(x.shape)}")
    tokens, hidden = x.shape
    _check(gate, "gate", x.dtype)
    if gate.dim() != 3 or gate.shape[1] != hidden:
        raise ContractError(f"expert gate matrix must have shape [experts, {hidden}, inter], got {list(gate.shape)}")
    experts, _, inter = gate.shape
    _check(up, "up", x.dtype, (experts, hidden, inter))
    _check(down, "down", x.dtype, (experts, inter, hidden))
    return tokens, hidden, experts, inter


def grouped_swiglu_train(x, source_order, top_k, gate, up, down, group_sizes, offsets):
    """x [T,H] + permutation (or packed rows with source_order=None) -> packed_y, act, ExpertResiduals."""
    tokens, hidden, experts, inter = _expert_shapes(x, gate, up, down)
    rows = tokens * top_k if source_order is not None else tokens
    if source_order is not None:
        _check(source_order, "source_order", torch.int32, (rows,))
    _check(group_sizes, "group_sizes", torch.int32, (experts,))
    _check(offsets, "offsets", torch.int32, (experts,))
    dev = x.device
    gate_pre = torch.empty((rows, inter), dtype=x.dtype, device=dev)
    up_pre = torch.empty_like(gate_pre)
    act = torch.empty_like(gate_pre)
    packed_y = torch.empty((rows, hidden), dtype=x.dtype, device=dev)
    status = _lib().jtmoe_grouped_swiglu_train(
        _ptr(x), _ptr(source_order), _ptr(gate), _ptr(up), _ptr(down), _ptr(group_sizes), _ptr(offsets),
        tokens, top_k, hidden, inter, experts, _code(x.dtype),
        _ptr(gate_pre), _ptr(up_pre), _ptr(act), _ptr(packed_y), _stream(dev),
    )
    _raise(status, "jtmoe_grouped_swiglu_train")
    return packed_y, act, ExpertResiduals(gate_pre, up_pre)


def _shared_shapes(x, gate, up, down):
    _check(x, "x")
    if x.dim() != 2:
        raise ContractError(f"x must have shape [tokens, hidden], got {list(x.shape)}")
    tokens, hidden = x.shape
    _check(gate, "shared gate", x.dtype)
    if gate.dim() != 2 or gate.shape[0] != hidden:
        raise ContractError(f"shared gate must have shape [{hidden}, inter], got {list(gate.shape)}")
    inter = gate.shape[1]
    _check(up, "shared up", x.dtype, (hidden, inter))
    _check(down, "shared down", x.dtype, (inter, hidden))
    return tokens, hidden, inter


def shared_swiglu_train(x, gate, up, down):
    """x [T,H] -> shared_y [T,H], ExpertResiduals ([T,Is] each)."""
    tokens, hidden, inter = _shared_shapes(x, gate, up, down)
    dev = x.device
    gate_pre = torch.empty((tokens, inter), dtype=x.dtype, device=dev)
    up_pre = torch.empty_like(gate_pre)
    act = torch.empty_like(gate_pre)
    out = torch.empty((tokens, hidden), dtype=x.dtype, device=dev)
    status = _lib().jtmoe_shared_swiglu_train(
        _ptr(x), _ptr(gate), _ptr(up), _ptr(down), tokens, hidden, inter, _code(x.dtype),
        _ptr(gate_pre), _ptr(up_pre), _ptr(act), _ptr(out), _stream(dev),
    )
    _raise(status, "jtmoe_shared_swiglu_train")
    return out, ExpertResiduals(gate_pre, up_pre)


@dataclass
class ExpertsGrad:
    dx: torch.Tensor  # [T,H]
    d_weights: torch.Tensor  # [T,K]
    d_gate: torch.Tensor  # [E,H,I]
    d_up: torch.Tensor  # [E,H,I]
    d_down: torch.Tensor  # [E,I,H]


def experts_backward(x, dy, plan: ops.DispatchResult, weights, gate, up, down, residuals: ExpertResiduals,
                     dx_extra=None) -> ExpertsGrad:
    """VJP of dispatch -> grouped SwiGLU -> combine for the cotangent dy [T,H]."""
    tokens, hidden, experts, inter = _expert_shapes(x, gate, up, down)
    _check(dy, "dy", x.dtype, (tokens, hidden))
    _check(weights, "weights", x.dtype)
    if weights.dim() != 2 or weights.shape[0] != tokens:
        raise ContractError(f"weights must have shape [{tokens}, top_k], got {list(weights.shape)}")
    top_k = weights.shape[1]
    rows = tokens * top_k
    _check(plan.source_order, "source_order", torch.int32, (rows,))
    _check(plan.inverse, "inverse", torch.int32, (rows,))
    _check(plan.group_sizes, "group_sizes", torch.int32, (experts,))
    _check(plan.offsets, "offsets", torch.int32, (experts,))
    _check(residuals.gate_pre, "gate_pre", x.dtype, (rows, inter))
    _check(residuals.up_pre, "up_pre", x.dtype, (rows, inter))
    if dx_extra is not None:
        _check(dx_extra, "dx_extra", x.dtype, (tokens, hidden))
    dev = x.device
    dx = torch.empty_like(x)
    d_weights = torch.empty_like(weights)
    d_gate, d_up, d_down = torch.empty_like(gate), torch.empty_like(up), torch.empty_like(down)
    lib = _lib()
    ws = _workspace(lib.jtmoe_experts_backward_workspace_bytes(tokens, top_k, hidden, inter, _code(x.dtype)), dev)
    status = lib.jtmoe_experts_backward(
        _ptr(x), _ptr(dy), _ptr(plan.source_order), _ptr(plan.inverse), _ptr(weights), _ptr(plan.group_sizes),
        _ptr(plan.offsets), _ptr(gate), _ptr(up), _ptr(down), _ptr(residuals.gate_pre), _ptr(residuals.up_pre),
        tokens, top_k, hidden, inter, experts, _code(x.dtype), _ptr(dx_extra),
        _ptr(dx), _ptr(d_weights), _ptr(d_gate), _ptr(d_up), _ptr(d_down),
        ws.data_ptr(), ws.numel(), _stream(dev),
    )
    _raise(status, "jtmoe_experts_backward")
    return ExpertsGrad(dx, d_weights, d_gate, d_up, d_down)


def shared_backward(x, dy, gate, up, down, residuals: ExpertResiduals):
    """VJP of the shared SwiGLU: (dx, d_gate, d_up, d_down)."""
    tokens, hidden, inter = _shared_shapes(x, gate, up, down)
    _check(dy, "dy", x.dtype, (tokens, hidden))
    _check(residuals.gate_pre, "gate_pre", x.dtype, (tokens, inter))
    _check(residuals.up_pre, "up_pre", x.dtype, (tokens, inter))
    dev = x.device
    dx = torch.empty_like(x)
    d_gate, d_up, d_down = torch.empty_like(gate), torch.empty_like(up), torch.empty_like(down)
    lib = _lib()
    ws = _workspace(lib.jtmoe_shared_backward_workspace_bytes(tokens, hidden, inter, _code(x.dtype)), dev)
    status = lib.jtmoe_shared_backward(
        _ptr(x), _ptr(dy), _ptr(gate), _ptr(up), _ptr(down), _ptr(residuals.gate_pre), _ptr(residuals.up_pre),
        tokens, hidden, inter, _code(x.dtype), _ptr(dx), _ptr(d_gate), _ptr(d_up), _ptr(d_down),
        ws.data_ptr(), ws.numel(), _stream(dev),
    )
    _raise(status, "jtmoe_shared_backward")
    return dx, d_gate, d_up, d_down


def router_backward(x, w_router, scores, expert_ids, d_weights, d_scores=None, route_scale: float = 1.0,
                    score_func: str = "sigmoid"):
    """VJP of the router for the cotangents d_weights [T,K] and (optionally) d_scores [T,E]: (dx, d_w_router)."""
    _check(x, "x")
    if x.dim() != 2:
        raise ContractError(f"x must have shape [tokens, hidden], got {list(x.shape)}")
    tokens, hidden = x.shape
    _check(w_router, "w_router", x.dtype)
    if w_router.dim() != 2 or w_router.shape[0] != hidden:
        raise ContractError(f"w_router must have shape [{hidden}, experts], got {list(w_router.shape)}")
    experts = w_router.shape[1]
    _check(scores, "scores", torch.float32, (tokens, experts))
    _check(expert_ids, "expert_ids", torch.int32)
    if expert_ids.dim() != 2 or expert_ids.shape[0] != tokens:
        raise ContractError(f"expert_ids must have shape [{tokens}, top_k], got {list(expert_ids.shape)}")
    top_k = expert_ids.shape[1]
    _check(d_weights, "d_weights", x.dtype, (tokens, top_k))
    if d_scores is not None:
        _check(d_scores, "d_scores", torch.float32, (tokens, experts))
    dev = x.device
    dx = torch.empty_like(x)
    d_w = torch.empty_like(w_router)
    lib = _lib()
    ws = _workspace(lib.jtmoe_router_backward_workspace_bytes(tokens, hidden, experts, _code(x.dtype)), dev)
    head = (_ptr(x), _ptr(w_router), _ptr(scores), _ptr(expert_ids), _ptr(d_weights), _ptr(d_scores),
            float(route_scale))
    tail = (tokens, hidden, experts, top_k, _code(x.dtype), _ptr(dx), _ptr(d_w), ws.data_ptr(), ws.numel(),
            _stream(dev))
    code = ops._score_code(score_func)
    status = lib.jtmoe_router_backward(*head, *tail) if code == 0 else lib.jtmoe_router_backward_sf(*head, code, *tail)
    _raise(status, "jtmoe_router_backward")
    return dx, d_w


@dataclass
class LayerResiduals:
    routed: ExpertResiduals
    shared: ExpertResiduals | None


@dataclass
class LayerGrad:
    dx: torch.Tensor
    d_w_router: torch.Tensor
    d_gate: torch.Tensor
    d_up: torch.Tensor
    d_down: torch.Tensor
    d_shared: tuple | None


def moe_forward_train(x, w_router, expert_bias, gate, up, down, top_k, route_scale: float = 1.0, shared=None,
                      score_func: str = "sigmoid"):
    """The layer forward through jtmoe_moe_forward_train: (ops.LayerResult, LayerResiduals)."""
    tokens, hidden, experts, inter = _expert_shapes(x, gate, up, down)
    _check(w_router, "w_router", x.dtype, (hidden, experts))
    ops._validate_router_attrs(experts, top_k, route_scale)
    if expert_bias is not None:
        _check(expert_bias, "expert_bias", torch.float32, (experts,))
    shared_inter = 0
    sg = su = sd = None
    if shared is not None:
        sg, su, sd = shared
        _, _, shared_inter = _shared_shapes(x, sg, su, sd)
    dev = x.device
    rows = tokens * top_k
    i32, f32 = torch.int32, torch.float32
    y = torch.empty_like(x)
    expert_ids = torch.empty((tokens, top_k), dtype=i32, device=dev)
    weights = torch.empty((tokens, top_k), dtype=x.dtype, device=dev)
    scores = torch.empty((tokens, experts), dtype=f32, device=dev)
    expert_counts = torch.empty((experts,), dtype=f32, device=dev)
    importance = torch.empty((experts,), dtype=f32, device=dev)
    group_sizes = torch.empty((experts,), dtype=i32, device=dev)
    offsets = torch.empty((experts,), dtype=i32, device=dev)
    source_order = torch.empty((rows,), dtype=i32, device=dev)
    inverse = torch.empty((rows,), dtype=i32, device=dev)
    routed = ExpertResiduals(torch.empty((rows, inter), dtype=x.dtype, device=dev),
                             torch.empty((rows, inter), dtype=x.dtype, device=dev))
    shared_res = None
    if shared is not None:
        shared_res = ExpertResiduals(torch.empty((tokens, shared_inter), dtype=x.dtype, device=dev),
                                     torch.empty((tokens, shared_inter), dtype=x.dtype, device=dev))
    lib = _lib()
    nbytes = lib.jtmoe_workspace_bytes(tokens, hidden, experts, top_k, inter, shared_inter, _code(x.dtype))
    ws = ops.layer_workspace(nbytes, dev)
    head = (_ptr(x), _ptr(w_router), _ptr(expert_bias), _ptr(gate), _ptr(up), _ptr(down), _ptr(sg), _ptr(su), _ptr(sd),
            tokens, hidden, experts, top_k, inter, shared_inter, float(route_scale))
    tail = (
        _code(x.dtype),
        _ptr(y), _ptr(expert_ids), _ptr(weights), _ptr(scores), _ptr(expert_counts), _ptr(importance),
        _ptr(group_sizes), _ptr(offsets), _ptr(source_order), _ptr(inverse),
        _ptr(routed.gate_pre), _ptr(routed.up_pre),
        _ptr(shared_res.gate_pre) if shared_res else None, _ptr(shared_res.up_pre) if shared_res else None,
        ws.data_ptr(), ws.numel(), _stream(dev),
    )
    code = ops._score_code(score_func)
    status = (lib.jtmoe_moe_forward_train(*head, *tail) if code == 0
              else lib.jtmoe_moe_forward_train_sf(*head, code, *tail))
    _raise(status, "jtmoe_moe_forward_train")
    result = ops.LayerResult(y, expert_ids, weights, scores, expert_counts, importance, group_sizes, offsets,
                             source_order, inverse)
    return result, LayerResiduals(routed, shared_res)


_BACKWARD_WORKSPACES: dict[tuple, torch.Tensor] = {}


def moe_backward(x, dy, d_scores, w_router, gate, up, down, shared, result: ops.LayerResult,
                 residuals: LayerResiduals, route_scale: float = 1.0, score_func: str = "sigmoid") -> LayerGrad:
    """VJP of the layer for the cotangents dy [T,H] and d_scores [T,E] (or None)."""
    tokens, hidden, experts, inter = _expert_shapes(x, gate, up, down)
    _check(dy, "dy", x.dtype, (tokens, hidden))
    _check(w_router, "w_router", x.dtype, (hidden, experts))
    top_k = result.expert_ids.shape[1]
    if d_scores is not None:
        _check(d_scores, "d_scores", torch.float32, (tokens, experts))
    shared_inter = 0
    sg = su = sd = None
    if shared is not None:
        sg, su, sd = shared
        _, _, shared_inter = _shared_shapes(x, sg, su, sd)
        if residuals.shared is None:
            raise ContractError("shared experts given but the residuals hold none")
    dev = x.device
    dx = torch.empty_like(x)
    d_w = torch.empty_like(w_router)
    d_gate, d_up, d_down = torch.empty_like(gate), torch.empty_like(up), torch.empty_like(down)
    d_shared = tuple(torch.empty_like(t) for t in shared) if shared is not None else None
    lib = _lib()
    nbytes = lib.jtmoe_moe_backward_workspace_bytes(tokens, hidden, experts, top_k, inter, shared_inter,
                                                    _code(x.dtype))
    key = (str(dev), _stream(dev))
    ws = _BACKWARD_WORKSPACES.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = _workspace(nbytes, dev)
        _BACKWARD_WORKSPACES[key] = ws
    sres = residuals.shared
    head = (
        _ptr(x), _ptr(dy), _ptr(d_scores), _ptr(w_router), _ptr(gate), _ptr(up), _ptr(down),
        _ptr(sg), _ptr(su), _ptr(sd), _ptr(result.scores), _ptr(result.expert_ids), _ptr(result.weights),
        _ptr(result.source_order), _ptr(result.inverse), _ptr(result.group_sizes), _ptr(result.offsets),
        _ptr(residuals.routed.gate_pre), _ptr(residuals.routed.up_pre),
        _ptr(sres.gate_pre) if sres else None, _ptr(sres.up_pre) if sres else None,
        float(route_scale),
    )
    tail = (
        tokens, hidden, experts, top_k, inter, shared_inter, _code(x.dtype),
        _ptr(dx), _ptr(d_w), _ptr(d_gate), _ptr(d_up), _ptr(d_down),
        _ptr(d_shared[0]) if d_shared else None, _ptr(d_shared[1]) if d_shared else None,
        _ptr(d_shared[2]) if d_shared else None,
        ws.data_ptr(), ws.numel(), _stream(dev),
    )
    code = ops._score_code(score_func)
    status = lib.jtmoe_moe_backward(*head, *tail) if code == 0 else lib.jtmoe_moe_backward_sf(*head, code, *tail)
    _raise(status, "jtmoe_moe_backward")
    return LayerGrad(dx, d_w, d_gate, d_up, d_down, d_shared)
