"""Stage-level operators: torch tensors in, libjtmoe launchers underneath.

torch is used only for device memory and the current HIP stream; every
computation is done by the native library.  Each function validates what the
reference's wrappers validate (dtype / shape / device, cf.
src/jaxtitan/kernels/rmsnorm.py:55-65) and raises ContractError before calling
into C; a negative status from the library is raised with its message.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from research_amd import _ffi
from research_amd.errors import ContractError, KernelLaunchError

_DTYPES = {torch.bfloat16: _ffi.JTMOE_BF16, torch.float32: _ffi.JTMOE_F32}


def _lib():
    return _ffi.load_library()


def _code(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError as exc:
        raise ContractError(f"compute dtype must be bfloat16 or float32, got {dtype}") from exc


def _check(tensor: torch.Tensor, name: str, dtype: torch.dtype | None = None, shape: tuple | None = None) -> torch.Tensor:
    if not isinstance(tensor, torch.Tensor):
        raise ContractError(f"{name} must be a torch.Tensor")
    if not tensor.is_cuda:
        raise ContractError(f"{name} must live on the GPU (got device {tensor.device}); there is no CPU path")
    if dtype is not None and tensor.dtype != dtype:
        raise ContractError(f"{name} must have dtype {dtype}, got {tensor.dtype}")
    if shape is not None and tuple(tensor.shape) != tuple(shape):
        raise ContractError(f"{name} must have shape {list(shape)}, got {list(tensor.shape)}")
    if not tensor.is_contiguous():
        raise ContractError(f"{name} must be dense row-major (contiguous)")
    return tensor


def _ptr(tensor: torch.Tensor | None) -> int | None:
    if tensor is None:
        return None
    return tensor.data_ptr() if tensor.numel() else None


def _stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _raise(status: int, what: str) -> None:
    if status == 0:
        return
    message = _ffi.last_error(_lib())
    if status == -4:
        raise KernelLaunchError(f"{what}: {message}")
    raise ContractError(f"{what}: {message} (status {status})")


def _workspace(nbytes: int, device: torch.device) -> torch.Tensor:
    return torch.empty((max(int(nbytes), 256),), dtype=torch.uint8, device=device)


@dataclass
class RouterResult:
    expert_ids: torch.Tensor  # [T,K] int32
    weights: torch.Tensor  # [T,K] compute dtype
    scores: torch.Tensor  # [T,E] float32
    expert_counts: torch.Tensor  # [E] float32
    importance: torch.Tensor  # [E] float32
    logits: torch.Tensor | None  # [T,E] float32 when requested


SCORE_FUNCS = {"sigmoid": 0, "softmax": 1}  # JTMOE_SCORE_SIGMOID / JTMOE_SCORE_SOFTMAX of include/jtmoe.h


def _score_code(score_func: str) -> int:
    """"sigmoid" is the reference's router (moe.py:133); "softmax" is the attribute this library adds."""
    if score_func not in SCORE_FUNCS:
        raise ContractError(f"router score_func must be one of {sorted(SCORE_FUNCS)}, got {score_func!r}")
    return SCORE_FUNCS[score_func]


def _validate_router_attrs(num_experts: int, top_k: int, route_scale: float) -> None:
    if top_k <= 0 or num_experts <= 0 or top_k > num_experts:
        raise ContractError("router top_k must be positive and <= num_experts")
    if route_scale <= 0.0:
        raise ContractError(f"router route_scale must be positive, got {route_scale}")


def router(
    x: torch.Tensor,
    w_router: torch.Tensor,
    expert_bias: torch.Tensor | None,
    top_k: int,
    route_scale: float = 1.0,
    *,
    return_logits: bool = False,
    score_func: str = "sigmoid",
) -> RouterResult:
    """x [T,H], w_router [H,E] -> ids, weights, scores, counts, importance."""
    _check(x, "x")
    if x.dim() != 2:
        raise ContractError(f"router x must have shape [tokens, hidden], got {list(x.shape)}")
    tokens, hidden = x.shape
    _check(w_router, "w_router", x.dtype)
    if w_router.dim() != 2 or w_router.shape[0] != hidden:
        raise ContractError(f"w_router must have shape [{hidden}, experts], got {list(w_router.shape)}")
    experts = w_router.shape[1]
    _validate_router_attrs(experts, top_k, route_scale)
    if expert_bias is not None:
        _check(expert_bias, "expert_bias", torch.float32)
        if tuple(expert_bias.shape) != (experts,):
            raise ContractError(f"expert_bias must have shape [{experts}], got {tuple(expert_bias.shape)}")
    dev = x.device
    ids = torch.empty((tokens, top_k), dtype=torch.int32, device=dev)
    weights = torch.empty((tokens, top_k), dtype=x.dtype, device=dev)
    scores = torch.empty((tokens, experts), dtype=torch.float32, device=dev)
    counts = torch.empty((experts,), dtype=torch.float32, device=dev)
    importance = torch.empty((experts,), dtype=torch.float32, device=dev)
    logits = torch.empty((tokens, experts), dtype=torch.float32, device=dev) if return_logits else None
    lib = _lib()
    ws_bytes = lib.jtmoe_router_workspace_bytes(experts)
    ws = _workspace(ws_bytes, dev)
    head = (_ptr(x), _ptr(w_router), _ptr(expert_bias), tokens, hidden, experts, top_k, float(route_scale))
    tail = (_code(x.dtype), _ptr(ids), _ptr(weights), _ptr(scores), _ptr(counts), _ptr(importance), _ptr(logits),
            _ptr(ws), ws.numel(), _stream(dev))
    if _score_code(score_func) == 0:  # the reference's router: the entry point that replaces it
        status = lib.jtmoe_router(*head, *tail)
    else:
        status = lib.jtmoe_router_sf(*head, _score_code(score_func), *tail)
    _raise(status, "jtmoe_router")
    return RouterResult(ids, weights, scores, counts, importance, logits)


def router_from_logits(
    logits: torch.Tensor,
    expert_bias: torch.Tensor | None,
    top_k: int,
    route_scale: float = 1.0,
    *,
    dtype: torch.dtype = torch.float32,
    score_func: str = "sigmoid",
) -> RouterResult:
    """Routing decision from given fp32 logits [T,E]; weights are cast to ``dtype``."""
    _check(logits, "logits", torch.float32)
    if logits.dim() != 2:
        raise ContractError(f"logits must have shape [tokens, experts], got {list(logits.shape)}")
    tokens, experts = logits.shape
    _validate_router_attrs(experts, top_k, route_scale)
    if expert_bias is not None:
        _check(expert_bias, "expert_bias", torch.float32)
        if tuple(expert_bias.shape) != (experts,):
            raise ContractError(f"expert_bias must have shape [{experts}], got {tuple(expert_bias.shape)}")
    dev = logits.device
    ids = torch.empty((tokens, top_k), dtype=torch.int32, device=dev)
    weights = torch.empty((tokens, top_k), dtype=dtype, device=dev)
    scores = torch.empty((tokens, experts), dtype=torch.float32, device=dev)
    counts = torch.empty((experts,), dtype=torch.float32, device=dev)
    importance = torch.empty((experts,), dtype=torch.float32, device=dev)
    lib = _lib()
    ws = _workspace(lib.jtmoe_router_workspace_bytes(experts), dev)
    head = (_ptr(logits), _ptr(expert_bias), tokens, experts, top_k, float(route_scale))
    tail = (_code(dtype), _ptr(ids), _ptr(weights), _ptr(scores), _ptr(counts), _ptr(importance), _ptr(ws), ws.numel(),
            _stream(dev))
    if _score_code(score_func) == 0:
        status = lib.jtmoe_router_from_logits(*head, *tail)
    else:
        status = lib.jtmoe_router_from_logits_sf(*head, _score_code(score_func), *tail)
    _raise(status, "jtmoe_router_from_logits")
    return RouterResult(ids, weights, scores, counts, importance, None)


@dataclass
class DispatchResult:
    group_sizes: torch.Tensor  # [E] int32
    offsets: torch.Tensor  # [E] int32
    source_order: torch.Tensor  # [A] int32
    inverse: torch.Tensor  # [A] int32
    packed_x: torch.Tensor | None  # [A,H]


def dispatch(expert_ids: torch.Tensor, num_experts: int, x: torch.Tensor | None = None) -> DispatchResult:
    """expert_ids [T,K] int32 (+ x [T,H]) -> histogram, offsets, permutation, packed rows."""
    _check(expert_ids, "expert_ids", torch.int32)
    if expert_ids.dim() != 2:
        raise ContractError(f"expert_ids must have shape [tokens, top_k], got {list(expert_ids.shape)}")
    tokens, top_k = expert_ids.shape
    if num_experts <= 0 or top_k <= 0:
        raise ContractError("dispatch needs num_experts > 0 and top_k > 0")
    dev = expert_ids.device
    hidden = 0
    dtype = torch.bfloat16
    packed_x = None
    if x is not None:
        _check(x, "x")
        if x.dim() != 2 or x.shape[0] != tokens:
            raise ContractError(f"x must have shape [{tokens}, hidden], got {list(x.shape)}")
        hidden = x.shape[1]
        dtype = x.dtype
        packed_x = torch.empty((tokens * top_k, hidden), dtype=dtype, device=dev)
    n_assign = tokens * top_k
    group_sizes = torch.empty((num_experts,), dtype=torch.int32, device=dev)
    offsets = torch.empty((num_experts,), dtype=torch.int32, device=dev)
    source_order = torch.empty((n_assign,), dtype=torch.int32, device=dev)
    inverse = torch.empty((n_assign,), dtype=torch.int32, device=dev)
    lib = _lib()
    ws = _workspace(lib.jtmoe_dispatch_workspace_bytes(n_assign, num_experts), dev)
    status = lib.jtmoe_dispatch(
        _ptr(expert_ids), _ptr(x), tokens, hidden, num_experts, top_k, _code(dtype),
        _ptr(group_sizes), _ptr(offsets), _ptr(source_order), _ptr(inverse), _ptr(packed_x),
        _ptr(ws), ws.numel(), _stream(dev),
    )
    _raise(status, "jtmoe_dispatch")
    return DispatchResult(group_sizes, offsets, source_order, inverse, packed_x)


def grouped_swiglu(
    packed_x: torch.Tensor,
    gate: torch.Tensor,
    up: torch.Tensor,
    down: torch.Tensor,
    group_sizes: torch.Tensor,
    offsets: torch.Tensor,
    *,
    return_act: bool = False,
):
    """packed_x [A,H]; gate, up [E,H,I]; down [E,I,H] -> packed_y [A,H]."""
    _check(packed_x, "packed_x")
    if packed_x.dim() != 2:
        raise ContractError(f"packed_x must have shape [rows, hidden], got {list(packed_x.shape)}")
    rows, hidden = packed_x.shape
    _check(gate, "gate", packed_x.dtype)
    if gate.dim() != 3 or gate.shape[1] != hidden:
        raise ContractError(f"expert gate matrix must have shape [experts, {hidden}, inter], got {list(gate.shape)}")
    experts, _, inter = gate.shape
    _check(up, "up", packed_x.dtype, (experts, hidden, inter))
    _check(down, "down", packed_x.dtype, (experts, inter, hidden))
    _check(group_sizes, "group_sizes", torch.int32, (experts,))
    _check(offsets, "offsets", torch.int32, (experts,))
    dev = packed_x.device
    act = torch.empty((rows, inter), dtype=packed_x.dtype, device=dev)
    packed_y = torch.empty((rows, hidden), dtype=packed_x.dtype, device=dev)
    status = _lib().jtmoe_grouped_swiglu(
        _ptr(packed_x), _ptr(gate), _ptr(up), _ptr(down), _ptr(group_sizes), _ptr(offsets),
        rows, hidden, inter, experts, _code(packed_x.dtype), _ptr(act), _ptr(packed_y), _stream(dev),
    )
    _raise(status, "jtmoe_grouped_swiglu")
    return (packed_y, act) if return_act else packed_y


def grouped_swiglu_gather(
    x: torch.Tensor,
    source_order: torch.Tensor,
    top_k: int,
    gate: torch.Tensor,
    up: torch.Tensor,
    down: torch.Tensor,
    group_sizes: torch.Tensor,
    offsets: torch.Tensor,
) -> torch.Tensor:
    """x [T,H] and the permutation -> packed_y [T*K,H] without materialising packed_x."""
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
    _check(source_order, "source_order", torch.int32, (tokens * top_k,))
    _check(group_sizes, "group_sizes", torch.int32, (experts,))
    _check(offsets, "offsets", torch.int32, (experts,))
    dev = x.device
    act = torch.empty((tokens * top_k, inter), dtype=x.dtype, device=dev)
    packed_y = torch.empty((tokens * top_k, hidden), dtype=x.dtype, device=dev)
    status = _lib().jtmoe_grouped_swiglu_gather(
        _ptr(x), _ptr(source_order), _ptr(gate), _ptr(up), _ptr(down), _ptr(group_sizes), _ptr(offsets),
        tokens, top_k, hidden, inter, experts, _code(x.dtype), _ptr(act), _ptr(packed_y), _stream(dev),
    )
    _raise(status, "jtmoe_grouped_swiglu_gather")
    return packed_y


def shared_swiglu(x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    """x [T,H]; gate, up [H,Is]; down [Is,H] -> [T,H]."""
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
    dev = x.device
    act = torch.empty((tokens, inter), dtype=x.dtype, device=dev)
    out = torch.empty((tokens, hidden), dtype=x.dtype, device=dev)
    status = _lib().jtmoe_shared_swiglu(
        _ptr(x), _ptr(gate), _ptr(up), _ptr(down), tokens, hidden, inter, _code(x.dtype),
        _ptr(act), _ptr(out), _stream(dev),
    )
    _raise(status, "jtmoe_shared_swiglu")
    return out


def combine(
    packed_y: torch.Tensor,
    inverse: torch.Tensor,
    weights: torch.Tensor,
    shared_y: torch.Tensor | None = None,
) -> torch.Tensor:
    """packed_y [A,H], inverse [A], weights [T,K] (+ shared_y [T,H]) -> y [T,H]."""
    _check(packed_y, "packed_y")
    _check(weights, "weights", packed_y.dtype)
    if packed_y.dim() != 2 or weights.dim() != 2:
        raise ContractError("combine expects packed_y [rows, hidden] and weights [tokens, top_k]")
    tokens, top_k = weights.shape
    rows, hidden = packed_y.shape
    if rows != tokens * top_k:
        raise ContractError(f"packed_y has {rows} rows, expected tokens*top_k = {tokens * top_k}")
    _check(inverse, "inverse", torch.int32, (rows,))
    if shared_y is not None:
        _check(shared_y, "shared_y", packed_y.dtype, (tokens, hidden))
    dev = packed_y.device
    y = torch.empty((tokens, hidden), dtype=packed_y.dtype, device=dev)
    status = _lib().jtmoe_combine(
        _ptr(packed_y), _ptr(inverse), _ptr(weights), _ptr(shared_y), tokens, hidden, top_k,
        _code(packed_y.dtype), _ptr(y), _stream(dev),
    )
    _raise(status, "jtmoe_combine")
    return y


def rmsnorm(x: torch.Tensor, scale: torch.Tensor, eps: float = 1.0e-6) -> torch.Tensor:
    """RMSNorm over the last axis of x [..., H] with a float32 scale [H]."""
    _check(x, "x")
    if x.dim() < 2:
        raise ContractError("rmsnorm input rank must be at least 2")
    hidden = x.shape[-1]
    _check(scale, "scale", torch.float32, (hidden,))
    if eps < 0:
        raise ContractError("eps must not be negative")
    rows = x.numel() // hidden
    y = torch.empty_like(x)
    status = _lib().jtmoe_rmsnorm(_ptr(x), _ptr(scale), rows, hidden, float(eps), _code(x.dtype), _ptr(y),
                                  _stream(x.device))
    _raise(status, "jtmoe_rmsnorm")
    return y


def combine_norm_residual(
    packed_y: torch.Tensor,
    inverse: torch.Tensor,
    weights: torch.Tensor,
    residual: torch.Tensor,
    post_scale: torch.Tensor,
    eps: float = 1.0e-6,
    shared_y: torch.Tensor | None = None,
) -> torch.Tensor:
    """residual + rmsnorm(combine(packed_y, inverse, weights, shared_y); post_scale) in one kernel."""
    _check(packed_y, "packed_y")
    _check(weights, "weights", packed_y.dtype)
    if packed_y.dim() != 2 or weights.dim() != 2:
        raise ContractError("combine expects packed_y [rows, hidden] and weights [tokens, top_k]")
    tokens, top_k = weights.shape
    rows, hidden = packed_y.shape
    if rows != tokens * top_k:
        raise ContractError(f"packed_y has {rows} rows, expected tokens*top_k = {tokens * top_k}")
    _check(inverse, "inverse", torch.int32, (rows,))
    _check(residual, "residual", packed_y.dtype, (tokens, hidden))
    _check(post_scale, "post_scale", torch.float32, (hidden,))
    if shared_y is not None:
        _check(shared_y, "shared_y", packed_y.dtype, (tokens, hidden))
    dev = packed_y.device
    out = torch.empty((tokens, hidden), dtype=packed_y.dtype, device=dev)
    status = _lib().jtmoe_combine_norm_residual(
        _ptr(packed_y), _ptr(inverse), _ptr(weights), _ptr(shared_y), _ptr(residual), _ptr(post_scale), float(eps),
        tokens, hidden, top_k, _code(packed_y.dtype), _ptr(out), _stream(dev),
    )
    _raise(status, "jtmoe_combine_norm_residual")
    return out


def router_stats(expert_counts: torch.Tensor) -> torch.Tensor:
    """expert_counts [E] f32 -> [6] f32: total, min, max, mean, max_vio, entropy."""
    _check(expert_counts, "expert_counts", torch.float32)
    if expert_counts.dim() != 1 or expert_counts.numel() == 0:
        raise ContractError(f"expert_counts must have shape [experts], got {list(expert_counts.shape)}")
    out = torch.empty((6,), dtype=torch.float32, device=expert_counts.device)
    status = _lib().jtmoe_router_stats(_ptr(expert_counts), expert_counts.numel(), _ptr(out), _stream(out.device))
    _raise(status, "jtmoe_router_stats")
    return out


def smebu_update(router_counts: torch.Tensor, momentum: torch.Tensor, expert_bias: torch.Tensor, *, load_lr: float,
                 momentum_factor: float, clamp: float) -> torch.Tensor:
    """One SMEBU step on device: router_counts [L,E] f32 -> momentum, expert_bias [L,E] f32 updated in place.

    Returns [6] f32: max_vio, load_min, load_max, load_entropy, bias_norm, momentum_norm
    (steps/moe_balance.py:97-162).
    """
    _check(router_counts, "router_counts", torch.float32)
    if router_counts.dim() != 2 or router_counts.numel() == 0:
        raise ContractError(f"router_counts must have shape [layers, experts], got {list(router_counts.shape)}")
    layers, experts = router_counts.shape
    _check(momentum, "momentum", torch.float32, (layers, experts))
    _check(expert_bias, "expert_bias", torch.float32, (layers, experts))
    out = torch.empty((6,), dtype=torch.float32, device=router_counts.device)
    status = _lib().jtmoe_smebu_update(_ptr(router_counts), _ptr(momentum), _ptr(expert_bias), layers, experts,
                                       float(load_lr), float(momentum_factor), float(clamp), _ptr(out),
                                       _stream(out.device))
    _raise(status, "jtmoe_smebu_update")
    return out


def sequence_balance_loss(expert_ids: torch.Tensor, scores: torch.Tensor, *, top_k: int) -> torch.Tensor:
    """expert_ids [B,S,K] int32, scores [B,S,E] f32 -> scalar f32 tensor."""
    if not isinstance(scores, torch.Tensor) or scores.dim() != 3:
        shape = list(scores.shape) if isinstance(scores, torch.Tensor) else None
        raise ContractError(f"router scores must have shape [batch, seq, experts], got {shape}")
    _check(scores, "scores", torch.float32)
    batch, seq_len, experts = scores.shape
    _check(expert_ids, "expert_ids", torch.int32, (batch, seq_len, top_k))
    dev = scores.device
    loss = torch.empty((1,), dtype=torch.float32, device=dev)
    lib = _lib()
    ws = _workspace(lib.jtmoe_balance_workspace_bytes(batch, experts), dev)
    status = lib.jtmoe_sequence_balance_loss(
        _ptr(expert_ids), _ptr(scores), batch, seq_len, experts, top_k, _ptr(loss), _ptr(ws), ws.numel(), _stream(dev),
    )
    _raise(status, "jtmoe_sequence_balance_loss")
    return loss.reshape(())


def sequence_balance_loss_backward(expert_ids: torch.Tensor, scores: torch.Tensor, *, top_k: int,
                                   d_loss: torch.Tensor | None = None) -> torch.Tensor:
    """Gradient of sequence_balance_loss with respect to the scores [B,S,E] (d_loss: scalar f32 tensor or None = 1)."""
    if not isinstance(scores, torch.Tensor) or scores.dim() != 3:
        shape = list(scores.shape) if isinstance(scores, torch.Tensor) else None
        raise ContractError(f"router scores must have shape [batch, seq, experts], got {shape}")
    _check(scores, "scores", torch.float32)
    batch, seq_len, experts = scores.shape
    _check(expert_ids, "expert_ids", torch.int32, (batch, seq_len, top_k))
    if d_loss is not None:
        _check(d_loss, "d_loss", torch.float32)
        if d_loss.numel() != 1:
            raise ContractError(f"d_loss must hold one value, got shape {list(d_loss.shape)}")
    dev = scores.device
    d_scores = torch.empty_like(scores)
    status = _lib().jtmoe_sequence_balance_loss_backward(
        _ptr(expert_ids), _ptr(scores), _ptr(d_loss), batch, seq_len, experts, top_k, _ptr(d_scores), _stream(dev),
    )
    _raise(status, "jtmoe_sequence_balance_loss_backward")
    return d_scores


@dataclass
class LayerResult:
    y: torch.Tensor  # [T,H]
    expert_ids: torch.Tensor  # [T,K] int32
    weights: torch.Tensor  # [T,K]
    scores: torch.Tensor  # [T,E] f32
    expert_counts: torch.Tensor  # [E] f32
    importance: torch.Tensor  # [E] f32
    group_sizes: torch.Tensor  # [E] int32
    offsets: torch.Tensor  # [E] int32
    source_order: torch.Tensor  # [A] int32
    inverse: torch.Tensor  # [A] int32


_WORKSPACES: dict[tuple, torch.Tensor] = {}


def layer_workspace(nbytes: int, device: torch.device) -> torch.Tensor:
    """Scratch of the whole-layer call, cached per (device, stream) and grown on demand.

    Calls on one stream are ordered, so they can share one scratch allocation.
    """
    key = (str(device), _stream(device))
    ws = _WORKSPACES.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty((max(int(nbytes), 256),), dtype=torch.uint8, device=device)
        _WORKSPACES[key] = ws
    return ws


def moe_forward(
    x: torch.Tensor,
    w_router: torch.Tensor,
    expert_bias: torch.Tensor | None,
    gate: torch.Tensor,
    up: torch.Tensor,
    down: torch.Tensor,
    top_k: int,
    route_scale: float = 1.0,
    shared: tuple[torch.Tensor, torch.Tensor, torch.Tensor] | None = None,
    workspace: torch.Tensor | None = None,
    stage_ms: list | None = None,
    expert_counts_out: torch.Tensor | None = None,
    score_func: str = "sigmoid",
) -> LayerResult:
    """The whole layer on x [T,H] through the single C entry point jtmoe_moe_forward
    (jtmoe_moe_forward_sf for a score function other than the reference's sigmoid).

    ``expert_counts_out`` ([experts] f32, contiguous — e.g. one row of the [layers, experts] buffer
    the balancing update reads) receives the expert counts instead of a fresh tensor.

    With ``stage_ms`` (a list) the measuring variant jtmoe_moe_forward_timed is
    used instead: it synchronises the stream and the list receives the elapsed
    milliseconds of each stage in the order of ``_ffi.STAGE_NAMES``.
    """
    _check(x, "x")
    if x.dim() != 2:
        raise ContractError(f"x must have shape [tokens, hidden], got {list(x.shape)}")
    tokens, hidden = x.shape
    _check(w_router, "w_router", x.dtype)
    if w_router.dim() != 2 or w_router.shape[0] != hidden:
        raise ContractError(f"w_router must have shape [{hidden}, experts], got {list(w_router.shape)}")
    experts = w_router.shape[1]
    _validate_router_attrs(experts, top_k, route_scale)
    if expert_bias is not None:
        _check(expert_bias, "expert_bias", torch.float32)
        if tuple(expert_bias.shape) != (experts,):
            raise ContractError(f"expert_bias must have shape [{experts}], got {tuple(expert_bias.shape)}")
    _check(gate, "gate", x.dtype)
    if gate.dim() != 3 or gate.shape[0] != experts or gate.shape[1] != hidden:
        raise ContractError(f"expert gate must have shape [{experts}, {hidden}, inter], got {list(gate.shape)}")
    inter = gate.shape[2]
    _check(up, "up", x.dtype, (experts, hidden, inter))
    _check(down, "down", x.dtype, (experts, inter, hidden))
    shared_inter = 0
    sg = su = sd = None
    if shared is not None:
        sg, su, sd = shared
        _check(sg, "shared gate", x.dtype)
        if sg.dim() != 2 or sg.shape[0] != hidden:
            raise ContractError(f"shared gate must have shape [{hidden}, inter], got {list(sg.shape)}")
        shared_inter = sg.shape[1]
        _check(su, "shared up", x.dtype, (hidden, shared_inter))
        _check(sd, "shared down", x.dtype, (shared_inter, hidden))
    dev = x.device
    n_assign = tokens * top_k
    i32, f32 = torch.int32, torch.float32
    y = torch.empty((tokens, hidden), dtype=x.dtype, device=dev)
    expert_ids = torch.empty((tokens, top_k), dtype=i32, device=dev)
    weights = torch.empty((tokens, top_k), dtype=x.dtype, device=dev)
    scores = torch.empty((tokens, experts), dtype=f32, device=dev)
    if expert_counts_out is None:
        expert_counts = torch.empty((experts,), dtype=f32, device=dev)
    else:
        _check(expert_counts_out, "expert_counts_out", f32, (experts,))
        expert_counts = expert_counts_out
    importance = torch.empty((experts,), dtype=f32, device=dev)
    group_sizes = torch.empty((experts,), dtype=i32, device=dev)
    offsets = torch.empty((experts,), dtype=i32, device=dev)
    source_order = torch.empty((n_assign,), dtype=i32, device=dev)
    inverse = torch.empty((n_assign,), dtype=i32, device=dev)
    lib = _lib()
    nbytes = lib.jtmoe_workspace_bytes(tokens, hidden, experts, top_k, inter, shared_inter, _code(x.dtype))
    if workspace is None:
        workspace = layer_workspace(nbytes, dev)
    else:
        _check(workspace, "workspace", torch.uint8)
        if workspace.numel() < nbytes or workspace.data_ptr() % 256:
            raise ContractError(f"workspace must hold {nbytes} bytes and be 256-byte aligned")
    args = (
        _ptr(x), _ptr(w_router), _ptr(expert_bias), _ptr(gate), _ptr(up), _ptr(down), _ptr(sg), _ptr(su), _ptr(sd),
        tokens, hidden, experts, top_k, inter, shared_inter, float(route_scale), _code(x.dtype),
        _ptr(y), _ptr(expert_ids), _ptr(weights), _ptr(scores), _ptr(expert_counts), _ptr(importance),
        _ptr(group_sizes), _ptr(offsets), _ptr(source_order), _ptr(inverse),
        workspace.data_ptr(), workspace.numel(), _stream(dev),
    )
    if _score_code(score_func) != 0:
        if stage_ms is not None:
            raise ContractError("the per-stage timing entry point runs the reference's sigmoid router only")
        status = lib.jtmoe_moe_forward_sf(*args[:16], _score_code(score_func), *args[16:])
    elif stage_ms is None:
        status = lib.jtmoe_moe_forward(*args)
    else:
        import ctypes

        buf = (ctypes.c_float * _ffi.NUM_STAGES)()
        status = lib.jtmoe_moe_forward_timed(*args, buf)
        stage_ms[:] = list(buf)
    _raise(status, "jtmoe_moe_forward")
    return LayerResult(y, expert_ids, weights, scores, expert_counts, importance,
                       group_sizes, offsets, source_order, inverse)


def ffn_block_forward(
    x: torch.Tensor,
    pre_scale: torch.Tensor,
    post_scale: torch.Tensor,
    eps: float,
    w_router: torch.Tensor,
    expert_bias: torch.Tensor | None,
    gate: torch.Tensor,
    up: torch.Tensor,
    down: torch.Tensor,
    top_k: int,
    route_scale: float = 1.0,
    shared: tuple[torch.Tensor, torch.Tensor, torch.Tensor] | None = None,
) -> LayerResult:
    """x + post_norm(moe(pre_norm(x))) on x [T,H] through jtmoe_ffn_block_forward; ``y`` of the result is the block output."""
    _check(x, "x")
    if x.dim() != 2:
        raise ContractError(f"x must have shape [tokens, hidden], got {list(x.shape)}")
    tokens, hidden = x.shape
    _check(pre_scale, "pre_scale", torch.float32, (hidden,))
    _check(post_scale, "post_scale", torch.float32, (hidden,))
    _check(w_router, "w_router", x.dtype)
    if w_router.dim() != 2 or w_router.shape[0] != hidden:
        raise ContractError(f"w_router must have shape [{hidden}, experts], got {list(w_router.shape)}")
    experts = w_router.shape[1]
    _validate_router_attrs(experts, top_k, route_scale)
    if expert_bias is not None:
        _check(expert_bias, "expert_bias", torch.float32, (experts,))
    _check(gate, "gate", x.dtype)
    if gate.dim() != 3 or gate.shape[0] != experts or gate.shape[1] != hidden:
        raise ContractError(f"expert gate must have shape [{experts}, {hidden}, inter], got {list(gate.shape)}")
    inter = gate.shape[2]
    _check(up, "up", x.dtype, (experts, hidden, inter))
    _check(down, "down", x.dtype, (experts, inter, hidden))
    shared_inter = 0
    sg = su = sd = None
    if shared is not None:
        sg, su, sd = shared
        _check(sg, "shared gate", x.dtype)
        if sg.dim() != 2 or sg.shape[0] != hidden:
            raise ContractError(f"shared gate must have shape [{hidden}, inter], got {list(sg.shape)}")
        shared_inter = sg.shape[1]
        _check(su, "shared up", x.dtype, (hidden, shared_inter))
        _check(sd, "shared down", x.dtype, (shared_inter, hidden))
    dev = x.device
    n_assign = tokens * top_k
    i32, f32 = torch.int32, torch.float32
    out = torch.empty_like(x)
    expert_ids = torch.empty((tokens, top_k), dtype=i32, device=dev)
    weights = torch.empty((tokens, top_k), dtype=x.dtype, device=dev)
    scores = torch.empty((tokens, experts), dtype=f32, device=dev)
    expert_counts = torch.empty((experts,), dtype=f32, device=dev)
    importance = torch.empty((experts,), dtype=f32, device=dev)
    group_sizes = torch.empty((experts,), dtype=i32, device=dev)
    offsets = torch.empty((experts,), dtype=i32, device=dev)
    source_order = torch.empty((n_assign,), dtype=i32, device=dev)
    inverse = torch.empty((n_assign,), dtype=i32, device=dev)
    lib = _lib()
    nbytes = lib.jtmoe_ffn_block_workspace_bytes(tokens, hidden, experts, top_k, inter, shared_inter, _code(x.dtype))
    workspace = layer_workspace(nbytes, dev)
    status = lib.jtmoe_ffn_block_forward(
        _ptr(x), _ptr(pre_scale), _ptr(post_scale), float(eps), _ptr(w_router), _ptr(expert_bias),
        _ptr(gate), _ptr(up), _ptr(down), _ptr(sg), _ptr(su), _ptr(sd),
        tokens, hidden, experts, top_k, inter, shared_inter, float(route_scale), _code(x.dtype),
        _ptr(out), _ptr(expert_ids), _ptr(weights), _ptr(scores), _ptr(expert_counts), _ptr(importance),
        _ptr(group_sizes), _ptr(offsets), _ptr(source_order), _ptr(inverse),
        workspace.data_ptr(), workspace.numel(), _stream(dev),
    )
    _raise(status, "jtmoe_ffn_block_forward")
    return LayerResult(out, expert_ids, weights, scores, expert_counts, importance,
                       group_sizes, offsets, source_order, inverse)
