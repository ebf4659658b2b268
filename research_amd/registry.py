"""Kernel registry and plan resolution for the operations libjtmoe.so implements.

Host-side mirror of the reference's kernel registry (src/jaxtitan/kernels/registry.py:16-124)
and of its cache enrichment (src/jaxtitan/kernels/build.py:93-143), with the same payload
fields, so that the reference's `kernels list / plan` output and its run diagnostics can carry
these entries unchanged.  The difference is the one the reference leaves open: there every
target operation falls back to XLA ("no_jax_ffi_implementation", registry.py:123); here the
two MoE operations and the FFN norm resolve to this library when

  * kernels are enabled in the request,
  * the device is a gfx950 part,
  * the built library is present and its checksum matches the manifest, and
  * the run mode (train / eval / inference) is one the entry is validated for.

Anything else resolves to "xla" with an explicit reason, and strict mode refuses such a plan
(registry.py:160-176).  Nothing here loads the shared object or touches a GPU.
"""

from __future__ import annotations

from dataclasses import asdict, dataclass
import json
from pathlib import Path
from typing import Any

from research_amd.build import ARCH, MANIFEST_NAME, _sha256, cache_dir, load_cache_manifest
from research_amd.errors import ContractError

REGISTRY_VERSION = 1
IMPLEMENTATION = "hip_gfx950"
BACKEND = "jtmoe"
MODES = ("train", "eval", "inference")
# substrings of the device kind (jax.devices()[0].device_kind / torch.cuda.get_device_name) that
# identify a gfx950 part
_GFX950_DEVICE_MARKS = ("gfx950", "mi355", "mi350")


@dataclass(frozen=True)
class KernelRegistration:
    """Static metadata of one operation (field list of registry.py:16-27) plus the entry points behind it."""

    op: str
    implementation: str
    status: str
    train_capable: bool
    eval_capable: bool
    inference_capable: bool
    notes: str
    entry_points: tuple[str, ...] = ()


_REGISTRY: tuple[KernelRegistration, ...] = (
    KernelRegistration(
        op="moe_dispatch_combine",
        implementation=IMPLEMENTATION,
        status="validated",
        train_capable=True,
        eval_capable=True,
        inference_capable=True,
        notes="Sigmoid top-k router, histogram / offsets / stable permutation, gate-weighted combine; "
        "indices, counts and permutation bit-exact against the CPU restatement; backward included.",
        entry_points=("jtmoe_router", "jtmoe_dispatch", "jtmoe_combine", "jtmoe_router_backward"),
    ),
    KernelRegistration(
        op="routed_expert_ffn",
        implementation=IMPLEMENTATION,
        status="validated",
        train_capable=True,
        eval_capable=True,
        inference_capable=True,
        notes="Grouped SwiGLU expert FFN (bf16 MFMA grouped GEMM over ragged groups) and the dense shared "
        "experts; forward, data- and weight-gradient products.",
        entry_points=(
            "jtmoe_grouped_swiglu", "jtmoe_grouped_swiglu_gather", "jtmoe_shared_swiglu", "jtmoe_moe_forward",
            "jtmoe_moe_forward_train", "jtmoe_moe_backward",
        ),
    ),
    KernelRegistration(
        op="rmsnorm",
        implementation=IMPLEMENTATION,
        status="validated",
        train_capable=False,
        eval_capable=True,
        inference_capable=True,
        notes="RMSNorm of the FFN sub-block (pre-norm stand-alone, post-norm and residual fused into the "
        "combine); forward only, so it does not replace the norm in a training step.",
        entry_points=("jtmoe_rmsnorm", "jtmoe_combine_norm_residual", "jtmoe_ffn_block_forward"),
    ),
)

@dataclass(frozen=True)
class KernelRequest:
    """What a run asks of the kernel backend: the `kernels` section of the reference's run spec
    (enabled / strict / compile), whether the model has MoE layers, and the run mode."""

    enabled: bool = True
    strict: bool = False
    compile: bool = False
    moe: bool = True
    mode: str = "inference"
    optimizer: str | None = None

    def __post_init__(self) -> None:
        if self.mode not in MODES:
            raise ContractError(f"kernel request mode must be one of {MODES}, got {self.mode!r}")

    @classmethod
    def from_run_spec(cls, spec: Any, *, mode: str = "train") -> "KernelRequest":
        """Read the fields `kernel_plan` uses from a reference RunSpec-shaped object
        (spec.kernels.{enabled,strict,compile}, spec.model.name / .trinity.moe, spec.optimizer.name;
        registry.py:230-237)."""
        kernels = getattr(spec, "kernels", None)
        if kernels is None:
            raise ContractError("run spec has no `kernels` section")
        model = getattr(spec, "model", None)
        trinity = getattr(model, "trinity", None)
        has_moe = getattr(model, "name", None) == "trinity" and getattr(trinity, "moe", None) is not None
        optimizer = getattr(getattr(spec, "optimizer", None), "name", None)
        return cls(
            enabled=bool(kernels.enabled), strict=bool(kernels.strict), compile=bool(kernels.compile), moe=has_moe,
            mode=mode, optimizer=optimizer,
        )


def kernel_registry() -> tuple[KernelRegistration, ...]:
    return _REGISTRY


def _registration_payload(registration: KernelRegistration) -> dict[str, Any]:
    payload = asdict(registration)
    payload["entry_points"] = list(registration.entry_points)
    return payload


def kernel_registry_payload() -> dict[str, Any]:
    """JSON-safe registry summary (registry.py:92-98)."""
    return {"schema_version": REGISTRY_VERSION, "kernels": [_registration_payload(item) for item in _REGISTRY]}


def is_gfx950_device(device_kind: str | None) -> bool:
    if not device_kind:
        return False
    lowered = device_kind.lower()
    return any(mark in lowered for mark in _GFX950_DEVICE_MARKS)


def library_cache_status(root: str | Path | None = None) -> tuple[str, str]:
    """('cached' | 'stale' | 'missing', detail) of the built library, by manifest and checksum
    (the three states of build.py:297-306)."""
    manifest = load_cache_manifest(root)
    if manifest is None:
        return "missing", "not_compiled"
    try:
        artifact = manifest["artifacts"]["moe"]["ffi"]
        rel_path, expected = artifact["path"], artifact["sha256"]
    except (KeyError, TypeError):
        return "missing", "manifest_without_library"
    if not isinstance(rel_path, str) or not isinstance(expected, str):
        return "missing", "manifest_without_library"
    path = cache_dir(root) / rel_path
    if not path.exists():
        return "missing", rel_path
    if artifact.get("arch") != ARCH:
        return "stale", rel_path
    return ("cached" if _sha256(path) == expected else "stale"), rel_path


# Stable names of how the routed experts run, for artifacts that must not change silently between a
# run and its resumption: the reference records `expert_execution` and `grouped_gemm_lowering` in
# the dispatcher payload that enters its diagnostics and its resume fingerprint
# (src/jaxtitan/models/execution.py:29-33, 136-138; src/jaxtitan/runtime/resume.py:87-97, 115).
EXPERT_EXECUTION = "expert_major_jtmoe_grouped_gemm"
GROUPED_GEMM_LOWERING = "hip_gfx950_lds_dma_mfma"


def expert_execution_payload(root: str | Path | None = None) -> dict[str, Any]:
    """The fields a run's diagnostics and resume metadata carry when this library runs the experts.

    `library_sha256` is the manifest's checksum of the shared object (None unless the cache is
    intact): two runs with the same value execute the same machine code, so a resumed run can
    insist on it, or on the two names alone if a rebuilt library is acceptable.
    """
    status, _ = library_cache_status(root)
    sha = None
    if status == "cached":
        manifest = load_cache_manifest(root)
        sha = manifest["artifacts"]["moe"]["ffi"]["sha256"]
    return {
        "expert_execution": EXPERT_EXECUTION,
        "grouped_gemm_lowering": GROUPED_GEMM_LOWERING,
        "implementation": IMPLEMENTATION,
        "arch": ARCH,
        "library_cache": status,
        "library_sha256": sha,
    }


def _requested_ops(request: KernelRequest) -> tuple[str, ...]:
    # the order of registry.py:230-237
    ops = ["rmsnorm", "attention", "swiglu"]
    if request.moe:
        ops.extend(["moe_dispatch_combine", "routed_expert_ffn"])
    if request.optimizer == "muon":
        ops.append("optimizer_matrix_update")
    return tuple(dict.fromkeys(ops))


def _mode_capable(registration: KernelRegistration, mode: str) -> bool:
    return {"train": registration.train_capable, "eval": registration.eval_capable,
            "inference": registration.inference_capable}[mode]


def _decision(op: str, backend: str, reason: str, registration: KernelRegistration | None, cache_status: str) -> dict[str, Any]:
    return {
        "op": op,
        "backend": backend,
        "reason": reason,
        "implementation": None if registration is None else registration.implementation,
        "status": None if registration is None else registration.status,
        "train_capable": False if registration is None else registration.train_capable,
        "eval_capable": False if registration is None else registration.eval_capable,
        "inference_capable": False if registration is None else registration.inference_capable,
        "cache_status": cache_status,
    }


def kernel_plan(request: KernelRequest, *, device_kind: str | None = None,
                cache_root: str | Path | None = None) -> dict[str, Any]:
    """Resolve which requested operations run on this library (field list of registry.py:126-146,
    with the cache fields of build.py:134-143 already attached)."""
    registry = {item.op: item for item in _REGISTRY}
    library_state, library_detail = library_cache_status(cache_root)
    decisions: list[dict[str, Any]] = []
    active: dict[str, str] = {}
    fallback: dict[str, str] = {}
    unavailable: dict[str, str] = {}
    disabled: dict[str, str] = {}
    cached: dict[str, str] = {}
    missing: dict[str, str] = {}
    stale: dict[str, str] = {}

    for op in _requested_ops(request):
        registration = registry.get(op)
        if registration is None:
            decisions.append(_decision(op, "xla", "not_registered", None, "not_buildable"))
            fallback[op] = unavailable[op] = "not_registered"
            continue
        cache_status = {"cached": "ffi_cached", "stale": "stale", "missing": "missing"}[library_state]
        {"cached": cached, "stale": stale, "missing": missing}[library_state][op] = library_detail
        if not request.enabled:
            reason = "kernels_disabled"
            disabled[op] = reason
        elif not is_gfx950_device(device_kind):
            reason = "unsupported_device"
            unavailable[op] = reason
        elif library_state == "missing":
            reason = "library_not_built"
            unavailable[op] = reason
        elif library_state == "stale":
            reason = "stale_library"
            unavailable[op] = reason
        elif not _mode_capable(registration, request.mode):
            reason = f"not_{request.mode}_capable"
            unavailable[op] = reason
        else:
            decisions.append(_decision(op, BACKEND, "validated", registration, cache_status))
            active[op] = registration.implementation
            continue
        decisions.append(_decision(op, "xla", reason, registration, cache_status))
        fallback[op] = reason

    root = cache_dir(cache_root)
    return {
        "schema_version": REGISTRY_VERSION,
        "enabled": request.enabled,
        "strict": request.strict,
        "compile": request.compile,
        "mode": "auto" if request.enabled else "xla",
        "run_mode": request.mode,
        "device_kind": device_kind,
        "registry_version": REGISTRY_VERSION,
        "target_ops": list(_requested_ops(request)),
        "active": active,
        "fallback": fallback,
        "disabled": disabled,
        "unavailable": unavailable,
        "active_count": len(active),
        "fallback_count": len(fallback),
        "disabled_count": len(disabled),
        "unavailable_count": len(unavailable),
        "cache_dir": root.as_posix(),
        "cache_manifest": (root / MANIFEST_NAME).as_posix() if (root / MANIFEST_NAME).exists() else None,
        "cached": cached,
        "missing_cache": missing,
        "stale_cache": stale,
        "cached_count": len(cached),
        "missing_cache_count": len(missing),
        "stale_cache_count": len(stale),
        "decisions": decisions,
    }


def kernel_plan_to_json(plan: dict[str, Any]) -> str:
    """Canonical JSON (registry.py:154-157): the form the reference stores in run diagnostics."""
    return json.dumps(plan, sort_keys=True, separators=(",", ":"))


def require_kernel_plan_supported(plan: dict[str, Any], *, ops: tuple[str, ...] | None = None) -> None:
    """Strict mode refuses a plan in which a target operation falls back (registry.py:160-176).

    `ops` narrows the check to the operations the caller needs from this library; by default every
    target operation counts, as in the reference, so a strict plan that includes the operations this
    library does not cover is refused.
    """
    if not plan.get("enabled") or not plan.get("strict"):
        return
    fallback = plan.get("fallback", {})
    if not isinstance(fallback, dict):
        fallback = {}
    failing = sorted(op for op in fallback if ops is None or op in ops)
    if not failing:
        return
    raise ContractError(
        "kernels.strict=true requires validated kernels for all target ops; "
        "unavailable ops: " + ", ".join(f"{op} ({fallback[op]})" for op in failing)
    )


def format_kernel_registry(payload: dict[str, Any]) -> str:
    lines = ["kernels:"]
    kernels = payload.get("kernels", [])
    if not kernels:
        lines.append("  none")
    for item in kernels:
        lines.append(
            f"  {item['op']}: impl={item['implementation']} status={item['status']} "
            f"train={item['train_capable']} eval={item['eval_capable']} infer={item['inference_capable']}"
        )
    return "\n".join(lines)


def format_kernel_plan(plan: dict[str, Any]) -> str:
    lines = [
        f"kernels: enabled={plan['enabled']} strict={plan['strict']} compile={plan['compile']} "
        f"active={plan['active_count']} fallback={plan['fallback_count']} "
        f"unavailable={plan['unavailable_count']} device={plan['device_kind']} "
        f"cache={plan['cache_dir']} cached={plan['cached_count']} "
        f"missing_cache={plan['missing_cache_count']} stale_cache={plan['stale_cache_count']}"
    ]
    for decision in plan["decisions"]:
        lines.append(
            f"  {decision['op']}: backend={decision['backend']} reason={decision['reason']} "
            f"status={decision['status']} cache={decision['cache_status']}"
        )
    return "\n".join(lines)


def main(argv: list[str] | None = None) -> int:
    """`python -m research_amd.registry [list|plan] ...`: the two read-only sub-commands."""
    import argparse

    parser = argparse.ArgumentParser(prog="python -m research_amd.registry")
    sub = parser.add_subparsers(dest="command", required=True)
    sub.add_parser("list").add_argument("--json", action="store_true")
    plan_parser = sub.add_parser("plan")
    plan_parser.add_argument("--json", action="store_true")
    plan_parser.add_argument("--device-kind", default=None, help="device name; default: ask torch for cuda:0")
    plan_parser.add_argument("--mode", choices=MODES, default="inference")
    plan_parser.add_argument("--strict", action="store_true")
    plan_parser.add_argument("--disabled", action="store_true")
    args = parser.parse_args(argv)
    if args.command == "list":
        payload = kernel_registry_payload()
        print(json.dumps(payload, sort_keys=True) if args.json else format_kernel_registry(payload))
        return 0
    device_kind = args.device_kind
    if device_kind is None:
        import torch

        if torch.cuda.is_available():
            props = torch.cuda.get_device_properties(0)
            device_kind = f"{props.name} ({getattr(props, 'gcnArchName', '')})"
    plan = kernel_plan(KernelRequest(enabled=not args.disabled, strict=args.strict, mode=args.mode),
                       device_kind=device_kind)
    print(kernel_plan_to_json(plan) if args.json else format_kernel_plan(plan))
    try:
        require_kernel_plan_supported(plan, ops=tuple(item.op for item in _REGISTRY))
    except ContractError as exc:
        print(f"error: {exc}")
        return 1
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
