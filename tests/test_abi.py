"""CPU-side checks of the drop-in boundary: the library loads, exports every
symbol the header declares, its pure host functions answer, and the loader /
wrappers fail loudly (no fallback) on a bad artefact or bad arguments."""

from __future__ import annotations

import json
from pathlib import Path
import re
import shutil

import pytest

from research_amd import _ffi, build
from research_amd.errors import ContractError

ROOT = Path(__file__).resolve().parents[1]


def header_symbols() -> set[str]:
    text = (ROOT / "include" / "jtmoe.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(jtmoe_[a-z0-9_]+)\s*\(", text))


def test_header_and_binding_agree():
    assert header_symbols() == set(_ffi.PROTOTYPES)


def test_library_exports_every_declared_symbol():
    lib = _ffi.load_library()
    for name in header_symbols():
        assert hasattr(lib, name), name
    assert lib.jtmoe_version() == 1
    assert _ffi.last_error(lib) == ""


def test_workspace_sizing_is_pure_host_arithmetic():
    lib = _ffi.load_library()
    T, H, E, K, I, Is = 16384, 2048, 64, 8, 1408, 2816
    total = lib.jtmoe_workspace_bytes(T, H, E, K, I, Is, _ffi.JTMOE_BF16)
    A = T * K
    # bf16 at these sizes: the grouped GEMM gathers its rows through the permutation, so the workspace
    # holds the activation, the expert outputs and the shared experts' buffers, but no permuted copy of x
    assert lib.jtmoe_grouped_swiglu_gather_supported(T, H, I, _ffi.JTMOE_BF16) == 1
    payload = 2 * (A * I + A * H + T * Is + T * H)
    assert payload <= total <= payload + 2**21  # + metadata, alignment and the router's partial sums (0.5 MiB at E=64)
    assert total < 1.14e9  # 1.67e9 with the permuted copy
    assert total % 256 == 0
    # fp32 (and any shape the gathering GEMM does not take, e.g. H not a multiple of 64) keeps the copy
    assert lib.jtmoe_grouped_swiglu_gather_supported(T, H, I, _ffi.JTMOE_F32) == 0
    assert lib.jtmoe_workspace_bytes(T, H, E, K, I, Is, _ffi.JTMOE_F32) >= 2 * (payload + 2 * A * H)
    odd = lib.jtmoe_workspace_bytes(T, H + 8, E, K, I, Is, _ffi.JTMOE_BF16)
    assert odd >= 2 * (A * (H + 8) + A * I + A * (H + 8) + T * Is + T * (H + 8))
    assert lib.jtmoe_workspace_bytes(0, H, E, K, I, 0, _ffi.JTMOE_BF16) > 0
    assert lib.jtmoe_workspace_bytes(T, H, E, K, I, Is, 7) == 0  # unknown dtype
    # the decode path (activations of all tokens through every expert) and its workspace
    bf = _ffi.JTMOE_BF16
    assert lib.jtmoe_moe_forward_takes_decode_path(64, H, E, K, I, bf) == 1
    assert lib.jtmoe_moe_forward_takes_decode_path(16, H, E, K, I, bf) == 1   # T * K = 2 * E
    assert lib.jtmoe_moe_forward_takes_decode_path(15, H, E, K, I, bf) == 0
    assert lib.jtmoe_moe_forward_takes_decode_path(65, H, E, K, I, bf) == 0
    assert lib.jtmoe_moe_forward_takes_decode_path(T, H, E, K, I, bf) == 0
    assert lib.jtmoe_moe_forward_takes_decode_path(64, H, E, K, I, _ffi.JTMOE_F32) == 0
    assert lib.jtmoe_workspace_bytes(64, H, E, K, I, 0, bf) >= 2 * (E * 64 * I + 64 * K * H)
    assert lib.jtmoe_router_workspace_bytes(E) >= 12 * E
    assert lib.jtmoe_dispatch_workspace_bytes(A, E) >= 4 * E * ((A + 1023) // 1024)
    assert lib.jtmoe_balance_workspace_bytes(8, E) >= 32


def test_argument_errors_return_status_and_message_without_a_gpu():
    lib = _ffi.load_library()
    # validation happens before any launch: null pointers / bad attributes are reported, nothing runs
    rc = lib.jtmoe_combine(None, None, None, None, 4, 8, 2, 9, None, None)
    assert rc == -1 and "dtype" in _ffi.last_error(lib)
    rc = lib.jtmoe_router(None, None, None, 4, 8, 4, 5, 1.0, _ffi.JTMOE_BF16, None, None, None, None, None, None,
                          None, 0, None)
    assert rc == -1 and "top_k" in _ffi.last_error(lib)
    rc = lib.jtmoe_router(None, None, None, 4, 8, 4, 2, 0.0, _ffi.JTMOE_BF16, None, None, None, None, None, None,
                          None, 0, None)
    assert rc == -1 and "route_scale" in _ffi.last_error(lib)
    rc = lib.jtmoe_router(None, None, None, 4, 8, 1024, 2, 1.0, _ffi.JTMOE_BF16, None, None, None, None, None, None,
                          None, 0, None)
    assert rc == -2
    rc = lib.jtmoe_grouped_swiglu(None, None, None, None, None, None, 16, 8, 8, 2, _ffi.JTMOE_BF16, None, None, None)
    assert rc == -1 and "null" in _ffi.last_error(lib)
    rc = lib.jtmoe_moe_forward(*([None] * 9), 4, 8, 2, 1, 8, 0, 1.0, _ffi.JTMOE_BF16, *([None] * 10), None, 0, None)
    assert rc == -1 and "workspace" in _ffi.last_error(lib)


def test_training_and_block_entry_points_validate_before_launching():
    lib = _ffi.load_library()
    bf = _ffi.JTMOE_BF16
    T, H, E, K, I, Is = 16384, 2048, 64, 8, 1408, 2816
    b = 2
    # workspace sizes: pure host arithmetic, at least the buffers they are documented to hold
    experts = lib.jtmoe_experts_backward_workspace_bytes(T, K, H, I, bf)
    assert experts >= b * (3 * T * K * I + T * K * H + T * K) and experts % 256 == 0
    shared = lib.jtmoe_shared_backward_workspace_bytes(T, H, Is, bf)
    assert shared >= b * 3 * T * Is
    router = lib.jtmoe_router_backward_workspace_bytes(T, H, E, bf)
    assert router >= b * T * E
    whole = lib.jtmoe_moe_backward_workspace_bytes(T, H, E, K, I, Is, bf)
    assert whole >= experts + shared + router
    assert lib.jtmoe_moe_backward_workspace_bytes(T, H, E, K, I, Is, 9) == 0
    assert lib.jtmoe_ffn_block_workspace_bytes(T, H, E, K, I, Is, bf) == \
        lib.jtmoe_workspace_bytes(T, H, E, K, I, Is, bf) + b * T * H
    # argument errors come back as a status and a message; nothing is launched
    rc = lib.jtmoe_rmsnorm(None, None, 4, 8, 1e-6, 9, None, None)
    assert rc == -1 and "dtype" in _ffi.last_error(lib)
    rc = lib.jtmoe_rmsnorm(None, None, 4, 8, -1.0, bf, None, None)
    assert rc == -1 and "eps" in _ffi.last_error(lib)
    rc = lib.jtmoe_rmsnorm(None, None, 4, 8, 1e-6, bf, None, None)
    assert rc == -1 and "null" in _ffi.last_error(lib)
    rc = lib.jtmoe_combine_norm_residual(*([None] * 6), 1e-6, 4, 8, 2, bf, None, None)
    assert rc == -1 and "null" in _ffi.last_error(lib)
    rc = lib.jtmoe_experts_backward(*([None] * 12), 4, 2, 8, 8, 300, bf, *([None] * 6), None, 0, None)
    assert rc == -2 and "exceeds" in _ffi.last_error(lib)
    rc = lib.jtmoe_experts_backward(*([None] * 12), 4, 2, 8, 8, 4, bf, *([None] * 6), None, 0, None)
    assert rc == -1 and "null" in _ffi.last_error(lib)
    rc = lib.jtmoe_shared_backward(*([None] * 7), 4, 8, 8, 9, *([None] * 4), None, 0, None)
    assert rc == -1 and "dtype" in _ffi.last_error(lib)
    rc = lib.jtmoe_router_backward(*([None] * 6), 1.0, 4, 8, 4, 17, bf, None, None, None, 0, None)
    assert rc == -2 and "exceeds" in _ffi.last_error(lib)
    rc = lib.jtmoe_moe_backward(*([None] * 21), 1.0, 4, 8, 4, 2, 8, 0, bf, *([None] * 8), None, 0, None)
    assert rc == -1 and "null" in _ffi.last_error(lib)
    rc = lib.jtmoe_ffn_block_forward(None, None, None, 1e-6, *([None] * 8), 4, 8, 4, 2, 8, 0, 1.0, bf, *([None] * 10),
                                     None, 0, None)
    assert rc == -1 and "norm scale" in _ffi.last_error(lib)
    rc = lib.jtmoe_moe_forward_train(*([None] * 9), 4, 8, 4, 2, 8, 0, 1.0, bf, *([None] * 14), None, 0, None)
    assert rc == -1 and "residual" in _ffi.last_error(lib)


def test_loader_refuses_missing_or_stale_artifacts(tmp_path):
    with pytest.raises(ContractError, match="manifest is missing"):
        _ffi.shared_object_path(tmp_path)
    src = build.cache_dir()
    shutil.copy(src / build.LIBRARY_NAME, tmp_path / build.LIBRARY_NAME)
    shutil.copy(src / build.MANIFEST_NAME, tmp_path / build.MANIFEST_NAME)
    assert _ffi.shared_object_path(tmp_path).name == build.LIBRARY_NAME
    with (tmp_path / build.LIBRARY_NAME).open("ab") as handle:
        handle.write(b"\0")
    with pytest.raises(ContractError, match="checksum mismatch"):
        _ffi.shared_object_path(tmp_path)
    (tmp_path / build.LIBRARY_NAME).unlink()
    with pytest.raises(ContractError, match="is missing"):
        _ffi.shared_object_path(tmp_path)
    (tmp_path / build.MANIFEST_NAME).write_text("{not json")
    with pytest.raises(ContractError, match="failed to parse"):
        _ffi.shared_object_path(tmp_path)
    (tmp_path / build.MANIFEST_NAME).write_text(json.dumps({"artifacts": {}}))
    with pytest.raises(ContractError, match="does not contain"):
        _ffi.shared_object_path(tmp_path)


def test_library_is_validated_once_per_process_not_per_call(monkeypatch):
    _ffi.reset_registrations_for_tests()
    calls = []
    real = _ffi._sha256
    monkeypatch.setattr(_ffi, "_sha256", lambda path: (calls.append(path), real(path))[1])
    first = _ffi.load_library()
    assert len(calls) == 1
    for _ in range(3):
        assert _ffi.load_library() is first
    assert len(calls) == 1  # operator calls after the first do not hash the file again
    assert _ffi.load_library(build.cache_dir()) is first and len(calls) == 2  # another spelling of the root: checked, same handle


def test_manifest_records_the_build():
    manifest = build.load_cache_manifest()
    art = manifest["artifacts"]["moe"]["ffi"]
    assert art["arch"] == "gfx950" and art["kind"] == "ffi"
    assert set(art["sources"]) == set(build.SOURCE_FILES)
    assert len(art["sha256"]) == 64 and art["bytes"] > 0
