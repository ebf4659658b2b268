"""Kernel benchmark of the MoE layer: libjtmoe.so against a plain composition of library routines.

The counterpart, for the MoE operations, of the reference's kernel benchmark helper
(src/jaxtitan/kernels/bench.py:29-77, `jaxtitan kernels bench rmsnorm`): the same protocol —
a first call timed apart (:192-195), warm-up calls, then `perf_counter` around calls that block
until the result is ready (:203-209), latency summary min / p50 / p90 / p99 / max (:212-220) —
and the same payload layout (cache directory, manifest and shared-object checksums, one entry
per shape with both latency summaries, their ratio and the largest absolute difference), written
as a JSON artifact when a directory is given.

The side it is measured against is what a framework does without a kernel of its own: the
expert-major formulation of the layer (moe.py:577-671) written with torch tensor routines on the
same GPU — `torch.topk`, a stable `argsort`, one vendor-BLAS `matmul` triple per expert, an indexed
sum.  It is a comparison partner for this report only; the parity tests use the CPU restatement.
"""

from __future__ import annotations

from dataclasses import dataclass
from datetime import datetime, timezone
import json
from pathlib import Path
import statistics
import time
from typing import Any

from research_amd._ffi import shared_object_path
from research_amd.build import MANIFEST_NAME, _sha256, cache_dir, load_cache_manifest
from research_amd.errors import ContractError
from research_amd.synthetic import CONFIGS, DESCRIPTIONS, make_inputs


@dataclass(frozen=True)
class MoeBenchmarkConfig:
    configs: tuple[str, ...] = ("C5", "C2")
    warmup: int = 3
    iters: int = 10


def parse_configs(value: str) -> tuple[str, ...]:
    """Comma-separated configuration names (the `--rows` parser of bench.py:112-121, for names)."""
    names = tuple(part.strip() for part in value.split(",") if part.strip())
    if not names:
        raise ContractError("configs must contain at least one configuration name")
    unknown = [name for name in names if name not in CONFIGS]
    if unknown:
        raise ContractError(f"unknown configuration(s) {unknown}; known: {sorted(CONFIGS)}")
    return names


def _validate_benchmark_config(config: MoeBenchmarkConfig) -> None:
    parse_configs(",".join(config.configs))
    if config.warmup < 0:
        raise ContractError("MoE benchmark warmup must be non-negative")
    if config.iters <= 0:
        raise ContractError("MoE benchmark iters must be positive")


def _percentile(values: list[float], q: float) -> float:
    if len(values) == 1:
        return values[0]
    position = q * (len(values) - 1)
    lower = int(position)
    upper = min(lower + 1, len(values) - 1)
    return values[lower] + (values[upper] - values[lower]) * (position - lower)


def _latency_stats(times: list[float]) -> dict[str, float]:
    values = sorted(times)
    return {"min": values[0], "p50": statistics.median(values), "p90": _percentile(values, 0.90),
            "p99": _percentile(values, 0.99), "max": values[-1]}


def torch_layer(x, w_router, expert_bias, gate, up, down, top_k: int, route_scale: float, shared):
    """The layer with torch routines only (expert-major, moe.py:131-147 and :577-671).  Returns (y, ids)."""
    import torch

    tokens, hidden = x.shape
    experts = w_router.shape[1]
    scores = torch.sigmoid((x @ w_router).float())
    _, ids = torch.topk(scores + expert_bias, top_k, dim=-1)
    top = torch.gather(scores, 1, ids)
    weights = (top / (top.sum(-1, keepdim=True) + 1e-20) * route_scale).to(x.dtype)
    flat = ids.reshape(-1)
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=experts).tolist()
    packed = x[order // top_k]
    out = torch.empty((tokens * top_k, hidden), dtype=x.dtype, device=x.device)
    start = 0
    for e, n in enumerate(counts):
        if n:
            rows = packed[start:start + n]
            act = torch.nn.functional.silu(rows @ gate[e]) * (rows @ up[e])
            out[start:start + n] = act @ down[e]
        start += n
    inverse = torch.empty_like(order)
    inverse[order] = torch.arange(order.numel(), device=order.device)
    y = (out[inverse].reshape(tokens, top_k, hidden) * weights[..., None]).float().sum(1).to(x.dtype)
    if shared is not None:
        y = y + (torch.nn.functional.silu(x @ shared[0]) * (x @ shared[1])) @ shared[2]
    return y, ids.to(torch.int32)


def _timed_calls(fn, count: int) -> list[float]:
    import torch

    times = []
    for _ in range(count):
        torch.cuda.synchronize()
        start = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        times.append((time.perf_counter() - start) * 1e3)
    return times


def _benchmark_config(name: str, config: MoeBenchmarkConfig) -> dict[str, Any]:
    import torch

    from research_amd import ops

    dev = torch.device("cuda:0")
    inp = make_inputs(name, seed=0)
    cfg = inp["cfg"]
    dtype = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float32
    tokens = cfg["batch"] * cfg["seq"]

    def put(a):
        return torch.from_numpy(a).to(dev).to(dtype).contiguous()

    x = put(inp["x"].reshape(tokens, cfg["H"]))
    w_router, gate, up, down = (put(inp[k]) for k in ("w_router", "gate", "up", "down"))
    bias = torch.from_numpy(inp["expert_bias"]).to(dev)
    shared = None if inp["shared"] is None else tuple(put(m) for m in inp["shared"])
    del inp

    def run_library():
        return ops.moe_forward(x, w_router, bias, gate, up, down, cfg["K"], 1.0, shared=shared)

    def run_torch():
        return torch_layer(x, w_router, bias, gate, up, down, cfg["K"], 1.0, shared)

    torch_first_ms = _timed_calls(run_torch, 1)[0]
    library_first_ms = _timed_calls(run_library, 1)[0]
    _timed_calls(run_torch, config.warmup)
    _timed_calls(run_library, config.warmup)
    torch_ms = _latency_stats(_timed_calls(run_torch, config.iters))
    library_ms = _latency_stats(_timed_calls(run_library, config.iters))

    want, want_ids = run_torch()
    got = run_library()
    same_routing = (got.expert_ids.sort(-1).values == want_ids.sort(-1).values).all(-1)
    diff = (got.y.float() - want.float()).abs()[same_routing]
    scale = float(want.float().abs().max())
    return {
        "config": name,
        "description": DESCRIPTIONS[name],
        "shape": {k: cfg[k] for k in ("batch", "seq", "H", "E", "K", "I", "Ns")},
        "dtype": "bfloat16" if dtype is torch.bfloat16 else "float32",
        "torch_first_call_ms": torch_first_ms,
        "jtmoe_first_call_ms": library_first_ms,
        "torch_ms": torch_ms,
        "jtmoe_ms": library_ms,
        "speedup_p50": None if library_ms["p50"] <= 0.0 else torch_ms["p50"] / library_ms["p50"],
        "tokens_per_s_p50": tokens / (library_ms["p50"] * 1e-3),
        # rows both sides routed to the same experts (the two top-k routines may order a rounding-level
        # near-tie differently; the parity tests pin the selection against the CPU restatement)
        "same_routing_fraction": float(same_routing.float().mean()),
        "max_abs_error": float(diff.max()) if diff.numel() else 0.0,
        "max_abs_error_over_max_abs": (float(diff.max()) / scale) if diff.numel() and scale > 0 else 0.0,
    }


def benchmark_moe(
    *,
    cache_root: str | Path | None = None,
    configs: tuple[str, ...] = ("C5", "C2"),
    warmup: int = 3,
    iters: int = 10,
    artifact_dir: str | Path | None = None,
) -> dict[str, Any]:
    """Benchmark the library's layer against the torch composition on cuda:0 (bench.py:29-77)."""
    config = MoeBenchmarkConfig(configs=tuple(configs), warmup=warmup, iters=iters)
    _validate_benchmark_config(config)
    shared_object = shared_object_path(cache_root)
    manifest = load_cache_manifest(cache_root)
    if manifest is None:
        raise ContractError("kernel cache manifest is missing")
    manifest_path = cache_dir(cache_root) / MANIFEST_NAME

    import torch

    if not torch.cuda.is_available():
        raise ContractError("the MoE kernel benchmark needs a GPU (there is no CPU path)")
    props = torch.cuda.get_device_properties(0)

    rows = [_benchmark_config(name, config) for name in config.configs]
    payload: dict[str, Any] = {
        "schema_version": 1,
        "created_at": datetime.now(timezone.utc).strftime("%Y-%m-%dT%H:%M:%SZ"),
        "op": "moe",
        "kind": "forward_only_benchmark",
        "torch_version": torch.__version__,
        "backend": "rocm",
        "devices": [f"{props.name} ({getattr(props, 'gcnArchName', '')})"],
        "warmup": warmup,
        "iters": iters,
        "cache_dir": cache_dir(cache_root).as_posix(),
        "cache_manifest": manifest_path.as_posix(),
        "cache_manifest_sha256": _sha256(manifest_path),
        "shared_object": shared_object.relative_to(cache_dir(cache_root)).as_posix(),
        "shared_object_sha256": _sha256(shared_object),
        "rows": rows,
    }
    if artifact_dir is not None:
        artifact_path = Path(artifact_dir) / "diagnostics" / "kernel_benchmarks" / "moe.json"
        artifact_path.parent.mkdir(parents=True, exist_ok=True)
        payload["artifact_path"] = artifact_path.as_posix()
        artifact_path.write_text(json.dumps(payload, indent=2, sort_keys=True))
    return payload


def benchmark_to_json(payload: dict[str, Any]) -> str:
    return json.dumps(payload, sort_keys=True, separators=(",", ":"))


def format_moe_benchmark(payload: dict[str, Any]) -> str:
    lines = [f"moe benchmark: backend={payload['backend']} device={payload['devices'][0]} "
             f"warmup={payload['warmup']} iters={payload['iters']}"]
    for row in payload["rows"]:
        lines.append(
            f"  {row['config']} ({row['dtype']}): torch_p50={row['torch_ms']['p50']:.4f}ms "
            f"jtmoe_p50={row['jtmoe_ms']['p50']:.4f}ms speedup={row['speedup_p50']:.2f}x "
            f"tokens/s={row['tokens_per_s_p50']:.4g} same_routing={row['same_routing_fraction']:.4f} "
            f"max_abs_error={row['max_abs_error']:.6f}"
        )
    if "artifact_path" in payload:
        lines.append(f"artifact: {payload['artifact_path']}")
    return "\n".join(lines)


def main(argv: list[str] | None = None) -> int:
    import argparse

    parser = argparse.ArgumentParser(prog="python -m research_amd.kernel_bench")
    parser.add_argument("--configs", default="C5,C2", help="comma-separated names out of " + ",".join(sorted(CONFIGS)))
    parser.add_argument("--warmup", type=int, default=3)
    parser.add_argument("--iters", type=int, default=10)
    parser.add_argument("--artifact-dir", default=None)
    parser.add_argument("--json", action="store_true")
    args = parser.parse_args(argv)
    try:
        payload = benchmark_moe(configs=parse_configs(args.configs), warmup=args.warmup, iters=args.iters,
                                artifact_dir=args.artifact_dir)
    except ContractError as exc:
        print(f"error: {exc}")
        return 2
    print(benchmark_to_json(payload) if args.json else format_moe_benchmark(payload))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
