"""Kernel registry, plan resolution and the kernel benchmark's host logic (no GPU needed).

The expectations follow the reference's tests of its own registry and cache enrichment
(tests/jaxtitan/test_kernels.py: plan fields, strict-mode refusal, cached / missing / stale
artifacts), applied to a registry whose MoE entries are validated rather than planned.
"""

from __future__ import annotations

import json
import shutil
from types import SimpleNamespace

import pytest

from research_amd import kernel_bench, registry
from research_amd.build import LIBRARY_NAME, MANIFEST_NAME, cache_dir, load_cache_manifest
from research_amd.errors import ContractError

MI355X = "AMD Instinct MI355X (gfx950:sramecc+:xnack-)"


def test_registry_lists_the_operations_of_the_library_with_existing_entry_points():
    from research_amd._ffi import PROTOTYPES

    payload = registry.kernel_registry_payload()
    assert payload["schema_version"] == 1
    by_op = {item["op"]: item for item in payload["kernels"]}
    assert set(by_op) == {"moe_dispatch_combine", "routed_expert_ffn", "rmsnorm"}
    assert by_op["routed_expert_ffn"]["train_capable"] and by_op["moe_dispatch_combine"]["train_capable"]
    assert not by_op["rmsnorm"]["train_capable"] and by_op["rmsnorm"]["inference_capable"]
    for item in payload["kernels"]:
        assert item["status"] == "validated" and item["implementation"] == "hip_gfx950"
        assert item["entry_points"] and all(name in PROTOTYPES for name in item["entry_points"])
    text = registry.format_kernel_registry(payload)
    assert "routed_expert_ffn: impl=hip_gfx950 status=validated train=True eval=True infer=True" in text
    json.dumps(payload)  # JSON-safe


def test_plan_activates_the_moe_operations_on_gfx950_with_a_built_library():
    if load_cache_manifest() is None:
        pytest.skip("library not built")
    plan = registry.kernel_plan(registry.KernelRequest(mode="inference"), device_kind=MI355X)
    assert plan["target_ops"] == ["rmsnorm", "attention", "swiglu", "moe_dispatch_combine", "routed_expert_ffn"]
    assert plan["active"] == {op: "hip_gfx950" for op in ("rmsnorm", "moe_dispatch_combine", "routed_expert_ffn")}
    assert plan["fallback"] == {"attention": "not_registered", "swiglu": "not_registered"}
    assert plan["active_count"] == 3 and plan["fallback_count"] == 2 and plan["unavailable_count"] == 2
    assert plan["cached_count"] == 3 and plan["missing_cache_count"] == 0 and plan["stale_cache_count"] == 0
    by_op = {d["op"]: d for d in plan["decisions"]}
    assert by_op["routed_expert_ffn"]["backend"] == "jtmoe" and by_op["routed_expert_ffn"]["cache_status"] == "ffi_cached"
    assert by_op["attention"]["backend"] == "xla" and by_op["attention"]["cache_status"] == "not_buildable"
    assert plan["mode"] == "auto" and plan["device_kind"] == MI355X and plan["registry_version"] == 1
    # canonical JSON round-trips and is key-sorted
    text = registry.kernel_plan_to_json(plan)
    assert json.loads(text) == plan and " " not in text.split('"cache_dir"')[0]
    assert "routed_expert_ffn: backend=jtmoe reason=validated status=validated cache=ffi_cached" in (
        registry.format_kernel_plan(plan))


def test_training_keeps_the_forward_only_norm_on_xla():
    if load_cache_manifest() is None:
        pytest.skip("library not built")
    plan = registry.kernel_plan(registry.KernelRequest(mode="train"), device_kind=MI355X)
    assert set(plan["active"]) == {"moe_dispatch_combine", "routed_expert_ffn"}
    assert plan["fallback"]["rmsnorm"] == "not_train_capable"


@pytest.mark.parametrize("device_kind", [None, "", "NVIDIA A100-SXM4-80GB", "AMD Instinct MI300X (gfx942)"])
def test_other_devices_fall_back_with_a_reason(device_kind):
    plan = registry.kernel_plan(registry.KernelRequest(), device_kind=device_kind)
    assert plan["active"] == {}
    assert plan["fallback"]["routed_expert_ffn"] == "unsupported_device"
    assert registry.is_gfx950_device("gfx950:sramecc+:xnack-") and registry.is_gfx950_device("AMD Instinct MI355X")


def test_disabled_kernels_resolve_to_xla():
    plan = registry.kernel_plan(registry.KernelRequest(enabled=False, strict=True), device_kind=MI355X)
    assert plan["mode"] == "xla" and plan["active"] == {}
    assert plan["disabled"] == {op: "kernels_disabled" for op in ("rmsnorm", "moe_dispatch_combine", "routed_expert_ffn")}
    registry.require_kernel_plan_supported(plan)  # strict does not apply to a disabled backend


def test_missing_and_stale_libraries_are_reported_and_never_active(tmp_path):
    plan = registry.kernel_plan(registry.KernelRequest(), device_kind=MI355X, cache_root=tmp_path)
    assert plan["active"] == {} and plan["fallback"]["routed_expert_ffn"] == "library_not_built"
    assert plan["missing_cache"]["routed_expert_ffn"] == "not_compiled" and plan["cache_manifest"] is None
    assert {d["cache_status"] for d in plan["decisions"] if d["status"]} == {"missing"}

    if load_cache_manifest() is None:
        pytest.skip("library not built")
    shutil.copy(cache_dir() / MANIFEST_NAME, tmp_path / MANIFEST_NAME)
    assert registry.library_cache_status(tmp_path) == ("missing", LIBRARY_NAME)  # manifest without the file
    (tmp_path / LIBRARY_NAME).write_bytes(b"not the library the manifest describes")
    assert registry.library_cache_status(tmp_path) == ("stale", LIBRARY_NAME)
    plan = registry.kernel_plan(registry.KernelRequest(), device_kind=MI355X, cache_root=tmp_path)
    assert plan["active"] == {} and plan["fallback"]["moe_dispatch_combine"] == "stale_library"
    assert plan["stale_cache_count"] == 3 and plan["cache_manifest"] == (tmp_path / MANIFEST_NAME).as_posix()

    shutil.copy(cache_dir() / LIBRARY_NAME, tmp_path / LIBRARY_NAME)
    assert registry.library_cache_status(tmp_path) == ("cached", LIBRARY_NAME)
    manifest = json.loads((tmp_path / MANIFEST_NAME).read_text())
    manifest["artifacts"]["moe"]["ffi"]["arch"] = "gfx942"
    (tmp_path / MANIFEST_NAME).write_text(json.dumps(manifest))
    assert registry.library_cache_status(tmp_path)[0] == "stale"  # built for another part
    (tmp_path / MANIFEST_NAME).write_text("{ not json")
    with pytest.raises(ContractError, match="failed to parse"):
        registry.kernel_plan(registry.KernelRequest(), device_kind=MI355X, cache_root=tmp_path)


def test_strict_mode_refuses_fallbacks_and_can_be_narrowed_to_the_library_operations(tmp_path):
    request = registry.KernelRequest(strict=True, mode="inference")
    if load_cache_manifest() is not None:
        plan = registry.kernel_plan(request, device_kind=MI355X)
        with pytest.raises(ContractError, match=r"attention \(not_registered\), swiglu \(not_registered\)"):
            registry.require_kernel_plan_supported(plan)  # the reference's rule: every target op counts
        registry.require_kernel_plan_supported(plan, ops=("moe_dispatch_combine", "routed_expert_ffn", "rmsnorm"))
    plan = registry.kernel_plan(request, device_kind=MI355X, cache_root=tmp_path)
    with pytest.raises(ContractError, match=r"routed_expert_ffn \(library_not_built\)"):
        registry.require_kernel_plan_supported(plan, ops=("routed_expert_ffn",))
    relaxed = registry.kernel_plan(registry.KernelRequest(strict=False), device_kind=None, cache_root=tmp_path)
    registry.require_kernel_plan_supported(relaxed)


def test_request_from_a_run_spec_shaped_object():
    kernels = SimpleNamespace(enabled=True, strict=False, compile=True)
    moe_spec = SimpleNamespace(kernels=kernels, model=SimpleNamespace(name="trinity", trinity=SimpleNamespace(moe=object())),
                               optimizer=SimpleNamespace(name="muon"))
    request = registry.KernelRequest.from_run_spec(moe_spec)
    assert request == registry.KernelRequest(enabled=True, strict=False, compile=True, moe=True, mode="train",
                                             optimizer="muon")
    plan = registry.kernel_plan(request, device_kind=None)
    assert plan["target_ops"][-1] == "optimizer_matrix_update" and plan["compile"] is True
    assert plan["fallback"]["optimizer_matrix_update"] == "not_registered"
    dense = SimpleNamespace(kernels=kernels, model=SimpleNamespace(name="qwen3", trinity=None), optimizer=None)
    assert registry.kernel_plan(registry.KernelRequest.from_run_spec(dense), device_kind=None)["target_ops"] == [
        "rmsnorm", "attention", "swiglu"]
    with pytest.raises(ContractError, match="kernels"):
        registry.KernelRequest.from_run_spec(SimpleNamespace())
    with pytest.raises(ContractError, match="mode"):
        registry.KernelRequest(mode="serve")


def test_registry_command_line(capsys):
    assert registry.main(["list"]) == 0
    assert "moe_dispatch_combine" in capsys.readouterr().out
    assert registry.main(["list", "--json"]) == 0
    assert json.loads(capsys.readouterr().out)["kernels"][0]["op"] == "moe_dispatch_combine"
    assert registry.main(["plan", "--device-kind", "NVIDIA H100", "--json"]) == 0
    assert json.loads(capsys.readouterr().out)["active_count"] == 0
    assert registry.main(["plan", "--device-kind", "NVIDIA H100", "--strict"]) == 1
    assert "unsupported_device" in capsys.readouterr().out


def test_kernel_benchmark_host_logic():
    assert kernel_bench.parse_configs(" C5, C2 ,") == ("C5", "C2")
    for bad in ("", ",", "C9", "C2,nope"):
        with pytest.raises(ContractError):
            kernel_bench.parse_configs(bad)
    with pytest.raises(ContractError, match="warmup"):
        kernel_bench.benchmark_moe(configs=("C5",), warmup=-1)
    with pytest.raises(ContractError, match="iters"):
        kernel_bench.benchmark_moe(configs=("C5",), iters=0)
    stats = kernel_bench._latency_stats([4.0, 1.0, 3.0, 2.0])
    assert stats == {"min": 1.0, "p50": 2.5, "p90": pytest.approx(3.7), "p99": pytest.approx(3.97), "max": 4.0}
    assert kernel_bench._latency_stats([7.0])["p99"] == 7.0

    import torch

    if not torch.cuda.is_available() and load_cache_manifest() is not None:
        with pytest.raises(ContractError, match="GPU"):
            kernel_bench.benchmark_moe(configs=("C5",))
        assert kernel_bench.main(["--configs", "C5"]) == 2


def test_torch_composition_matches_a_dense_evaluation_on_cpu():
    """The benchmark's comparison partner is itself checked: against the dense per-assignment form
    (gather the selected matrices, three einsums, weighted sum) on a small fp32 case."""
    import torch

    g = torch.Generator().manual_seed(0)
    T, H, E, K, I = 9, 6, 5, 2, 4
    x = torch.randn((T, H), generator=g)
    w_r, bias = torch.randn((H, E), generator=g), torch.zeros(E)
    gate, up = torch.randn((E, H, I), generator=g) * 0.3, torch.randn((E, H, I), generator=g) * 0.3
    down = torch.randn((E, I, H), generator=g) * 0.3
    shared = tuple(torch.randn(s, generator=g) * 0.3 for s in ((H, 3), (H, 3), (3, H)))
    y, ids = kernel_bench.torch_layer(x, w_r, bias, gate, up, down, K, 1.5, shared)
    scores = torch.sigmoid(x @ w_r)
    top = torch.gather(scores, 1, ids.long())
    weights = top / top.sum(-1, keepdim=True) * 1.5
    act = torch.nn.functional.silu(torch.einsum("th,tkhi->tki", x, gate[ids.long()])) * torch.einsum(
        "th,tkhi->tki", x, up[ids.long()])
    want = (torch.einsum("tki,tkih->tkh", act, down[ids.long()]) * weights[..., None]).sum(1)
    want = want + (torch.nn.functional.silu(x @ shared[0]) * (x @ shared[1])) @ shared[2]
    assert ids.dtype == torch.int32 and (ids.long() == torch.topk(scores, K).indices).all()
    torch.testing.assert_close(y, want, rtol=1e-5, atol=1e-5)


def test_expert_execution_payload_names_the_lowering_and_the_library(tmp_path):
    """The counterpart of the reference's `expert_execution` / `grouped_gemm_lowering` fields
    (execution.py:136-138), which enter its resume fingerprint (resume.py:87-97, 115)."""
    missing = registry.expert_execution_payload(tmp_path)
    assert missing["expert_execution"] == "expert_major_jtmoe_grouped_gemm"
    assert missing["grouped_gemm_lowering"] == "hip_gfx950_lds_dma_mfma"
    assert missing["library_cache"] == "missing" and missing["library_sha256"] is None
    built = registry.expert_execution_payload()
    status, _ = registry.library_cache_status()
    assert built["library_cache"] == status
    if status == "cached":
        assert isinstance(built["library_sha256"], str) and len(built["library_sha256"]) == 64
    # the payload is plain JSON and stable between calls
    assert json.dumps(built, sort_keys=True) == json.dumps(registry.expert_execution_payload(), sort_keys=True)
