"""The kernel benchmark and the plan resolution on the real device."""

from __future__ import annotations

import json

import numpy as np
import pytest
import torch

from research_amd import kernel_bench, registry

pytestmark = pytest.mark.gpu


def test_plan_resolves_to_the_library_on_this_device():
    props = torch.cuda.get_device_properties(0)
    device_kind = f"{props.name} ({getattr(props, 'gcnArchName', '')})"
    plan = registry.kernel_plan(registry.KernelRequest(strict=True, mode="train"), device_kind=device_kind)
    assert set(plan["active"]) == {"moe_dispatch_combine", "routed_expert_ffn"}, plan
    registry.require_kernel_plan_supported(plan, ops=("moe_dispatch_combine", "routed_expert_ffn"))
    assert registry.main(["plan", "--mode", "inference"]) == 0  # asks torch for the device itself


def test_benchmark_of_the_decode_shape_writes_its_artifact(tmp_path):
    print("kernel benchmark C5", flush=True)
    payload = kernel_bench.benchmark_moe(configs=("C5",), warmup=1, iters=3, artifact_dir=tmp_path)
    row = payload["rows"][0]
    assert row["config"] == "C5" and row["shape"]["E"] == 64 and row["dtype"] == "bfloat16"
    assert payload["op"] == "moe" and payload["backend"] == "rocm" and payload["iters"] == 3
    assert len(payload["shared_object_sha256"]) == 64 and payload["shared_object"] == "libjtmoe.so"
    # both sides select the same experts except at rounding-level near-ties, and agree on those rows
    assert row["same_routing_fraction"] >= 0.95, row
    assert row["max_abs_error_over_max_abs"] <= 2e-2, row  # the stated bf16 tolerance
    assert row["jtmoe_ms"]["min"] > 0 and row["jtmoe_ms"]["min"] <= row["jtmoe_ms"]["p50"] <= row["jtmoe_ms"]["max"]
    assert np.isfinite(row["speedup_p50"])  # a reported figure: a timing ratio is no correctness property
    stored = json.loads((tmp_path / "diagnostics" / "kernel_benchmarks" / "moe.json").read_text())
    assert stored["rows"][0]["config"] == "C5" and stored["artifact_path"] == payload["artifact_path"]
    assert "C5 (bfloat16)" in kernel_bench.format_moe_benchmark(payload)
    assert json.loads(kernel_bench.benchmark_to_json(payload))["rows"][0]["jtmoe_ms"] == row["jtmoe_ms"]
