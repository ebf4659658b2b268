"""jax.ffi registration of the MoE custom calls (the reference's plugin mechanism).

Mirrors src/jaxtitan/kernels/_ffi.py:19-45 and src/jaxtitan/kernels/rmsnorm.py:23-52 with
platform="ROCM": the FFI shared object (libjtmoe_ffi.so, `make ffi`) is located through the
checksum manifest, opened with ctypes, and its handler symbols are registered once.

JAX and the XLA FFI headers are not part of this build's environment, so this module is the
integration stub a JAX host would use; without JAX every entry point raises ContractError.
"""

from __future__ import annotations

import ctypes
from pathlib import Path
from typing import Any

from research_amd.build import cache_dir
from research_amd.errors import ContractError

FFI_LIBRARY_NAME = "libjtmoe_ffi.so"
TARGETS = {
    "jaxtitan_moe_forward": "JaxtitanMoeForward",
    "jaxtitan_moe_router": "JaxtitanMoeRouter",
    "jaxtitan_moe_dispatch": "JaxtitanMoeDispatch",
    "jaxtitan_moe_grouped_swiglu": "JaxtitanMoeGroupedSwiglu",
    "jaxtitan_moe_combine": "JaxtitanMoeCombine",
    "jaxtitan_moe_forward_train": "JaxtitanMoeForwardTrain",
    "jaxtitan_moe_backward": "JaxtitanMoeBackward",
    "jaxtitan_rmsnorm": "JaxtitanRmsnorm",
    "jaxtitan_ffn_block_forward": "JaxtitanFfnBlockForward",
    "jaxtitan_moe_smebu_update": "JaxtitanMoeSmebuUpdate",
}

_REGISTERED: set[str] = set()
_LOADED_LIBS: dict[str, ctypes.CDLL] = {}


def _jax():
    try:
        import jax  # noqa: PLC0415
    except ImportError as exc:
        raise ContractError("jax is not installed: the jax.ffi custom calls cannot be registered") from exc
    return jax


def register_moe(cache_root: str | Path | None = None) -> dict[str, str]:
    """Register every MoE FFI target; returns {target name: symbol}."""
    jax = _jax()
    if set(TARGETS) <= _REGISTERED:
        return dict(TARGETS)
    path = cache_dir(cache_root) / FFI_LIBRARY_NAME
    if not path.exists():
        raise ContractError(f"MoE FFI shared object is missing: {path} (build it with `make ffi`)")
    try:
        library = ctypes.CDLL(path.as_posix())
    except OSError as exc:
        raise ContractError(f"failed to load MoE FFI shared object {path}: {exc}") from exc
    for target, symbol_name in TARGETS.items():
        try:
            symbol = getattr(library, symbol_name)
        except AttributeError as exc:
            raise ContractError(f"MoE FFI shared object {path} is missing symbol {symbol_name}") from exc
        jax.ffi.register_ffi_target(target, jax.ffi.pycapsule(symbol), platform="ROCM", api_version=1)
        _REGISTERED.add(target)
    _LOADED_LIBS[path.as_posix()] = library
    return dict(TARGETS)


def moe_forward(x: Any, router_kernel: Any, expert_bias: Any, gate: Any, up: Any, down: Any, *, top_k: int,
                route_scale: float = 1.0, shared: tuple[Any, Any, Any] | None = None,
                cache_root: str | Path | None = None):
    """SparseMoE forward as one jax.ffi custom call: returns (y, ids, weights, scores, counts, importance)."""
    jax = _jax()
    import jax.numpy as jnp  # noqa: PLC0415

    register_moe(cache_root)
    from research_amd import _ffi  # noqa: PLC0415

    lead, hidden = x.shape[:-1], x.shape[-1]
    tokens = 1
    for n in lead:
        tokens *= n
    experts, _, inter = gate.shape
    if shared is None:
        shared = (jnp.zeros((hidden, 0), x.dtype), jnp.zeros((hidden, 0), x.dtype), jnp.zeros((0, hidden), x.dtype))
    shared_inter = shared[0].shape[1]
    code = _ffi.JTMOE_BF16 if x.dtype == jnp.bfloat16 else _ffi.JTMOE_F32
    ws_bytes = _ffi.load_library(cache_root).jtmoe_workspace_bytes(tokens, hidden, experts, top_k, inter,
                                                                   shared_inter, code)
    sds = jax.ShapeDtypeStruct
    assignments = tokens * top_k
    call = jax.ffi.ffi_call(
        "jaxtitan_moe_forward",
        (
            sds(x.shape, x.dtype), sds((*lead, top_k), jnp.int32), sds((*lead, top_k), x.dtype),
            sds((*lead, experts), jnp.float32), sds((experts,), jnp.float32), sds((experts,), jnp.float32),
            sds((experts,), jnp.int32), sds((experts,), jnp.int32), sds((assignments,), jnp.int32),
            sds((assignments,), jnp.int32), sds((max(int(ws_bytes), 256),), jnp.uint8),
        ),
        vmap_method="sequential",
    )
    out = call(x, router_kernel, expert_bias, gate, up, down, *shared, top_k=int(top_k),
               route_scale=float(route_scale))
    return out[:6]


def smebu_update(router_counts: Any, momentum: Any, expert_bias: Any, *, load_lr: float, momentum_factor: float,
                 clamp: float, cache_root: str | Path | None = None):
    """The per-layer arithmetic of apply_moe_balance_update (steps/moe_balance.py:123-161) on stacked
    [layers, experts] f32 arrays: returns (next_momentum, next_expert_bias, metrics[6]).  The state
    operands are aliased to the results, so under jit with donated state nothing is copied."""
    jax = _jax()
    import jax.numpy as jnp  # noqa: PLC0415

    register_moe(cache_root)
    if router_counts.ndim != 2 or router_counts.shape != momentum.shape or router_counts.shape != expert_bias.shape:
        raise ContractError(f"router count shape must match MoE balance state, got {router_counts.shape}")
    sds = jax.ShapeDtypeStruct
    call = jax.ffi.ffi_call(
        "jaxtitan_moe_smebu_update",
        (sds(momentum.shape, jnp.float32), sds(expert_bias.shape, jnp.float32), sds((6,), jnp.float32)),
        input_output_aliases={1: 0, 2: 1},
        vmap_method="sequential",
    )
    return call(router_counts.astype(jnp.float32), momentum.astype(jnp.float32), expert_bias.astype(jnp.float32),
                load_lr=float(load_lr), momentum_factor=float(momentum_factor), clamp=float(clamp))


def moe_layer(x: Any, router_kernel: Any, expert_bias: Any, gate: Any, up: Any, down: Any, *, top_k: int,
              route_scale: float = 1.0, shared: tuple[Any, Any, Any] | None = None,
              cache_root: str | Path | None = None):
    """The layer with its custom VJP (docs/kernel_backend_design.md:120-128 of the reference):
    returns (y, scores, expert_ids); differentiable in x, the router kernel, the expert matrices and
    the shared-expert matrices, with cotangents on y and on the scores."""
    jax = _jax()
    import jax.numpy as jnp  # noqa: PLC0415

    register_moe(cache_root)
    from research_amd import _ffi  # noqa: PLC0415

    lead, hidden = x.shape[:-1], x.shape[-1]
    tokens = 1
    for n in lead:
        tokens *= n
    experts, _, inter = gate.shape
    if shared is None:
        shared = (jnp.zeros((hidden, 0), x.dtype), jnp.zeros((hidden, 0), x.dtype), jnp.zeros((0, hidden), x.dtype))
    shared_inter = shared[0].shape[1]
    code = _ffi.JTMOE_BF16 if x.dtype == jnp.bfloat16 else _ffi.JTMOE_F32
    lib = _ffi.load_library(cache_root)
    fwd_ws = max(int(lib.jtmoe_workspace_bytes(tokens, hidden, experts, top_k, inter, shared_inter, code)), 256)
    bwd_ws = max(int(lib.jtmoe_moe_backward_workspace_bytes(tokens, hidden, experts, top_k, inter, shared_inter,
                                                            code)), 256)
    sds = jax.ShapeDtypeStruct
    rows = tokens * top_k
    i32, f32 = jnp.int32, jnp.float32

    def forward_call(x, router_kernel, gate, up, down, shared):
        out = jax.ffi.ffi_call(
            "jaxtitan_moe_forward_train",
            (
                sds(x.shape, x.dtype), sds((*lead, top_k), i32), sds((*lead, top_k), x.dtype),
                sds((*lead, experts), f32), sds((experts,), f32), sds((experts,), f32), sds((experts,), i32),
                sds((experts,), i32), sds((rows,), i32), sds((rows,), i32),
                sds((rows, inter), x.dtype), sds((rows, inter), x.dtype),
                sds((tokens, shared_inter), x.dtype), sds((tokens, shared_inter), x.dtype),
                sds((fwd_ws,), jnp.uint8),
            ),
            vmap_method="sequential",
        )(x, router_kernel, jax.lax.stop_gradient(expert_bias), gate, up, down, *shared, top_k=int(top_k),
          route_scale=float(route_scale))
        return out[:-1]

    @jax.custom_vjp
    def layer(x, router_kernel, gate, up, down, shared):
        y, ids, _, scores = forward_call(x, router_kernel, gate, up, down, shared)[:4]
        return y, scores, ids

    def layer_fwd(x, router_kernel, gate, up, down, shared):
        out = forward_call(x, router_kernel, gate, up, down, shared)
        y, ids, weights, scores = out[:4]
        plan, residuals = out[6:10], out[10:14]
        return (y, scores, ids), (x, router_kernel, gate, up, down, shared, scores, ids, weights, plan, residuals)

    def layer_bwd(saved, cotangents):
        x, router_kernel, gate, up, down, shared, scores, ids, weights, plan, residuals = saved
        dy, d_scores, _ = cotangents
        group_sizes, offsets, source_order, inverse = plan
        grads = jax.ffi.ffi_call(
            "jaxtitan_moe_backward",
            (
                sds(x.shape, x.dtype), sds(router_kernel.shape, x.dtype), sds(gate.shape, x.dtype),
                sds(up.shape, x.dtype), sds(down.shape, x.dtype), sds(shared[0].shape, x.dtype),
                sds(shared[1].shape, x.dtype), sds(shared[2].shape, x.dtype), sds((bwd_ws,), jnp.uint8),
            ),
            vmap_method="sequential",
        )(x, dy, d_scores.astype(f32), router_kernel, gate, up, down, *shared, scores, ids, weights, source_order,
          inverse, group_sizes, offsets, *residuals, route_scale=float(route_scale))
        dx, d_router, d_gate, d_up, d_down, dsg, dsu, dsd = grads[:8]
        return dx, d_router, d_gate, d_up, d_down, (dsg, dsu, dsd)

    layer.defvjp(layer_fwd, layer_bwd)
    return layer(x, router_kernel, gate, up, down, shared)
