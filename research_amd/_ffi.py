"""ctypes binding of libjtmoe.so and (when JAX is present) jax.ffi registration.

Follows the reference's loader (src/jaxtitan/kernels/_ffi.py:19-76): the shared
object is located through the cache manifest, its sha256 is verified, it is
opened with ctypes.CDLL and kept alive in a module-level table.  There is no
fallback: if the library is missing, stale or lacks a symbol, a ContractError is
raised.
"""

from __future__ import annotations

import ctypes
from pathlib import Path

from research_amd.build import _sha256, cache_dir, load_cache_manifest
from research_amd.errors import ContractError

c_i64 = ctypes.c_int64
c_ptr = ctypes.c_void_p
c_size = ctypes.c_size_t
c_int = ctypes.c_int
c_dbl = ctypes.c_double
c_float = ctypes.c_float

# symbol -> (restype, argtypes); exactly the entry points of include/jtmoe.h
PROTOTYPES: dict[str, tuple] = {
    "jtmoe_version": (c_int, []),
    "jtmoe_last_error": (ctypes.c_char_p, []),
    "jtmoe_router_workspace_bytes": (c_size, [c_i64]),
    "jtmoe_router": (
        c_int,
        [c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_i64, c_i64, c_dbl, c_int,
         c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_size, c_ptr],
    ),
    "jtmoe_router_sf": (
        c_int,
        [c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_i64, c_i64, c_dbl, c_int, c_int,
         c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_size, c_ptr],
    ),
    "jtmoe_router_from_logits": (
        c_int,
        [c_ptr, c_ptr, c_i64, c_i64, c_i64, c_dbl, c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_size, c_ptr],
    ),
    "jtmoe_router_from_logits_sf": (
        c_int,
        [c_ptr, c_ptr, c_i64, c_i64, c_i64, c_dbl, c_int, c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_size,
         c_ptr],
    ),
    "jtmoe_dispatch_workspace_bytes": (c_size, [c_i64, c_i64]),
    "jtmoe_dispatch": (
        c_int,
        [c_ptr, c_ptr, c_i64, c_i64, c_i64, c_i64, c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_size, c_ptr],
    ),
    "jtmoe_dispatch_static": (
        c_int,
        [c_ptr, c_ptr, c_i64, c_i64, c_i64, c_i64, c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr],
    ),
    "jtmoe_grouped_swiglu": (
        c_int,
        [c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_i64, c_i64, c_int, c_ptr, c_ptr, c_ptr],
    ),
    "jtmoe_grouped_swiglu_gather_supported": (c_int, [c_i64, c_i64, c_i64, c_int]),
    "jtmoe_moe_forward_takes_decode_path": (c_int, [c_i64, c_i64, c_i64, c_i64, c_i64, c_int]),
    "jtmoe_grouped_swiglu_gather": (
        c_int,
        [c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_i64, c_i64, c_i64, c_int, c_ptr, c_ptr, c_ptr],
    ),
    "jtmoe_shared_swiglu": (c_int, [c_ptr, c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_i64, c_int, c_ptr, c_ptr, c_ptr]),
    "jtmoe_combine": (c_int, [c_ptr, c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_i64, c_int, c_ptr, c_ptr]),
    "jtmoe_router_stats": (c_int, [c_ptr, c_i64, c_ptr, c_ptr]),
    "jtmoe_smebu_update": (c_int, [c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_float, c_float, c_float, c_ptr, c_ptr]),
    "jtmoe_balance_workspace_bytes": (c_size, [c_i64, c_i64]),
    "jtmoe_sequence_balance_loss": (c_int, [c_ptr, c_ptr, c_i64, c_i64, c_i64, c_i64, c_ptr, c_ptr, c_size, c_ptr]),
    "jtmoe_sequence_balance_loss_backward": (c_int, [c_ptr, c_ptr, c_ptr, c_i64, c_i64, c_i64, c_i64, c_ptr, c_ptr]),
    "jtmoe_workspace_bytes": (c_size, [c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_int]),
    "jtmoe_moe_forward": (
        c_int,
        [c_ptr] * 9 + [c_i64] * 6 + [c_dbl, c_int] + [c_ptr] * 10 + [c_ptr, c_size, c_ptr],
    ),
    "jtmoe_moe_forward_sf": (
        c_int,
        [c_ptr] * 9 + [c_i64] * 6 + [c_dbl, c_int, c_int] + [c_ptr] * 10 + [c_ptr, c_size, c_ptr],
    ),
    "jtmoe_rmsnorm": (c_int, [c_ptr, c_ptr, c_i64, c_i64, c_dbl, c_int, c_ptr, c_ptr]),
    "jtmoe_combine_norm_residual": (
        c_int,
        [c_ptr] * 6 + [c_dbl] + [c_i64] * 3 + [c_int, c_ptr, c_ptr],
    ),
    "jtmoe_ffn_block_workspace_bytes": (c_size, [c_i64] * 6 + [c_int]),
    "jtmoe_ffn_block_forward": (
        c_int,
        [c_ptr] * 3 + [c_dbl] + [c_ptr] * 8 + [c_i64] * 6 + [c_dbl, c_int] + [c_ptr] * 10 + [c_ptr, c_size, c_ptr],
    ),
    "jtmoe_grouped_swiglu_train": (
        c_int,
        [c_ptr] * 7 + [c_i64] * 5 + [c_int] + [c_ptr] * 5,
    ),
    "jtmoe_shared_swiglu_train": (c_int, [c_ptr] * 4 + [c_i64] * 3 + [c_int] + [c_ptr] * 5),
    "jtmoe_experts_backward_workspace_bytes": (c_size, [c_i64, c_i64, c_i64, c_i64, c_int]),
    "jtmoe_experts_backward": (
        c_int,
        [c_ptr] * 12 + [c_i64] * 5 + [c_int] + [c_ptr] * 6 + [c_ptr, c_size, c_ptr],
    ),
    "jtmoe_shared_backward_workspace_bytes": (c_size, [c_i64, c_i64, c_i64, c_int]),
    "jtmoe_shared_backward": (c_int, [c_ptr] * 7 + [c_i64] * 3 + [c_int] + [c_ptr] * 4 + [c_ptr, c_size, c_ptr]),
    "jtmoe_router_backward_workspace_bytes": (c_size, [c_i64, c_i64, c_i64, c_int]),
    "jtmoe_router_backward": (
        c_int,
        [c_ptr] * 6 + [c_dbl] + [c_i64] * 4 + [c_int] + [c_ptr] * 2 + [c_ptr, c_size, c_ptr],
    ),
    "jtmoe_router_backward_sf": (
        c_int,
        [c_ptr] * 6 + [c_dbl, c_int] + [c_i64] * 4 + [c_int] + [c_ptr] * 2 + [c_ptr, c_size, c_ptr],
    ),
    "jtmoe_moe_forward_train": (
        c_int,
        [c_ptr] * 9 + [c_i64] * 6 + [c_dbl, c_int] + [c_ptr] * 14 + [c_ptr, c_size, c_ptr],
    ),
    "jtmoe_moe_forward_train_sf": (
        c_int,
        [c_ptr] * 9 + [c_i64] * 6 + [c_dbl, c_int, c_int] + [c_ptr] * 14 + [c_ptr, c_size, c_ptr],
    ),
    "jtmoe_moe_backward_workspace_bytes": (c_size, [c_i64] * 6 + [c_int]),
    "jtmoe_moe_backward": (
        c_int,
        [c_ptr] * 21 + [c_dbl] + [c_i64] * 6 + [c_int] + [c_ptr] * 8 + [c_ptr, c_size, c_ptr],
    ),
    "jtmoe_moe_backward_sf": (
        c_int,
        [c_ptr] * 21 + [c_dbl, c_int] + [c_i64] * 6 + [c_int] + [c_ptr] * 8 + [c_ptr, c_size, c_ptr],
    ),
    "jtmoe_moe_forward_timed": (
        c_int,
        [c_ptr] * 9 + [c_i64] * 6 + [c_dbl, c_int] + [c_ptr] * 10 + [c_ptr, c_size, c_ptr]
        + [ctypes.POINTER(ctypes.c_float)],
    ),
}

NUM_STAGES = 8
STAGE_NAMES = (
    "router",
    "dispatch_meta",
    "dispatch_rows",
    "gate_up",
    "down",
    "shared_gate_up",
    "shared_down",
    "combine",
)

JTMOE_BF16 = 0
JTMOE_F32 = 1

_LOADED_LIBS: dict[str, ctypes.CDLL] = {}  # by path of the shared object
_LIBS_BY_ROOT: dict[str, ctypes.CDLL] = {}  # by cache root, once its manifest and checksum have been validated


def shared_object_path(cache_root: str | Path | None = None) -> Path:
    """Path of libjtmoe.so after manifest and checksum validation."""
    manifest = load_cache_manifest(cache_root)
    if manifest is None:
        raise ContractError(
            "kernel cache manifest is missing; run `python -m research_amd.build` "
            "(or __graft_entry__.build()) first"
        )
    artifacts = manifest.get("artifacts", {})
    if not isinstance(artifacts, dict) or not isinstance(artifacts.get("moe"), dict):
        raise ContractError("kernel cache manifest does not contain a MoE artifact")
    ffi_artifact = artifacts["moe"].get("ffi")
    if not isinstance(ffi_artifact, dict):
        raise ContractError("kernel cache manifest does not contain a MoE FFI artifact")
    rel_path = ffi_artifact.get("path")
    expected_sha = ffi_artifact.get("sha256")
    if not isinstance(rel_path, str) or not isinstance(expected_sha, str):
        raise ContractError("MoE FFI artifact must record path and sha256")
    path = cache_dir(cache_root) / rel_path
    if not path.exists():
        raise ContractError(f"MoE shared object is missing: {path}")
    if _sha256(path) != expected_sha:
        raise ContractError(f"MoE shared object checksum mismatch: {path}")
    return path


def load_library(cache_root: str | Path | None = None) -> ctypes.CDLL:
    """Open libjtmoe.so and attach the prototypes.

    The manifest and the checksum are validated when a cache root is first used in the process, as the
    reference does at registration (_ffi.py:19-45); later calls return the library already opened
    (hashing the file again on every operator call would cost more than a small layer call itself).
    """
    root_key = "" if cache_root is None else Path(cache_root).as_posix()
    cached = _LIBS_BY_ROOT.get(root_key)
    if cached is not None:
        return cached
    path = shared_object_path(cache_root)
    key = path.as_posix()
    if key in _LOADED_LIBS:
        _LIBS_BY_ROOT[root_key] = _LOADED_LIBS[key]
        return _LOADED_LIBS[key]
    try:
        library = ctypes.CDLL(key)
    except OSError as exc:
        raise ContractError(f"failed to load MoE shared object {path}: {exc}") from exc
    for name, (restype, argtypes) in PROTOTYPES.items():
        try:
            fn = getattr(library, name)
        except AttributeError as exc:
            raise ContractError(f"MoE shared object {path} is missing symbol {name}") from exc
        fn.restype = restype
        fn.argtypes = argtypes
    _LOADED_LIBS[key] = library
    _LIBS_BY_ROOT[root_key] = library
    return library


def last_error(library: ctypes.CDLL) -> str:
    message = library.jtmoe_last_error()
    return message.decode("utf-8", "replace") if message else ""


def reset_registrations_for_tests() -> None:
    _LOADED_LIBS.clear()
    _LIBS_BY_ROOT.clear()
