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
