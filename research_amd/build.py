"""Compile libjtmoe.so for gfx950 and record it in a checksum manifest.

Mirrors the reference's kernel build driver
(src/jaxtitan/kernels/build.py:146-220): ``make`` is run in the kernel source
directory with ARCH / OUTDIR overridden, and every artefact is recorded with
path, sha256, size, kind, arch and compiler version in ``manifest.json`` next
to it.  The loader refuses an artefact whose checksum no longer matches.
"""

from __future__ import annotations

from datetime import datetime, timezone
from hashlib import sha256
import json
import os
from pathlib import Path
import shutil
import subprocess
from typing import Any

from research_amd.errors import ContractError

CACHE_SCHEMA_VERSION = 1
MANIFEST_NAME = "manifest.json"
LIBRARY_NAME = "libjtmoe.so"
NATIVE_TEST_NAME = "gemm_check"
ARCH = "gfx950"
SOURCE_FILES = (
    "api.hip", "router.hip", "dispatch.hip", "combine.hip", "norm.hip", "grouped_gemm.hip", "grouped_gemm_bwd.hip",
    "backward.hip", "common.hpp", "gemm_common.hpp", "gemm_launch.hpp", "grouped_gemm_dma.hpp",
    "grouped_gemm_stream.hpp", "grouped_gemm_bwd.hpp", "dispatch_small.hpp", "native/gemm_check.hip",
)


def package_root() -> Path:
    return Path(__file__).resolve().parent


def source_dir() -> Path:
    return package_root() / "csrc"


def cache_dir(root: str | Path | None = None) -> Path:
    """Directory holding the built library and its manifest."""
    return package_root() / "_build" if root is None else Path(root)


def _sha256(path: Path) -> str:
    digest = sha256()
    with path.open("rb") as handle:
        for block in iter(lambda: handle.read(1 << 20), b""):
            digest.update(block)
    return digest.hexdigest()


def _compiler_version(hipcc: str) -> str:
    try:
        out = subprocess.run([hipcc, "--version"], capture_output=True, text=True, check=False).stdout
    except OSError:
        return "unknown"
    return " | ".join(line.strip() for line in out.splitlines()[:2])


def load_cache_manifest(root: str | Path | None = None) -> dict[str, Any] | None:
    path = cache_dir(root) / MANIFEST_NAME
    if not path.exists():
        return None
    try:
        payload = json.loads(path.read_text())
    except json.JSONDecodeError as exc:
        raise ContractError(f"failed to parse kernel cache manifest {path}: {exc}") from exc
    if not isinstance(payload, dict):
        raise ContractError(f"kernel cache manifest must be a JSON object: {path}")
    return payload


def compile_kernels(root: str | Path | None = None, *, jobs: int = 8, clean: bool = True) -> dict[str, Any]:
    """Run make for libjtmoe.so and write the manifest.  Returns the manifest."""
    hipcc = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if shutil.which(hipcc) is None and not Path(hipcc).exists():
        raise ContractError("hipcc is required to build libjtmoe.so")
    out_dir = cache_dir(root)
    out_dir.mkdir(parents=True, exist_ok=True)
    make_vars = [f"ARCH={ARCH}", f"HIPCC={hipcc}", f"OUTDIR={out_dir.as_posix()}"]
    if clean:
        subprocess.run(["make", "clean", *make_vars], cwd=source_dir(), check=False, capture_output=True)
    proc = subprocess.run(
        ["make", f"-j{jobs}", "all", *make_vars],
        cwd=source_dir(),
        capture_output=True,
        text=True,
        check=False,
    )
    if proc.returncode != 0:
        raise ContractError(f"libjtmoe build failed:\n{proc.stdout[-4000:]}\n{proc.stderr[-4000:]}")
    library = out_dir / LIBRARY_NAME
    if not library.exists():
        raise ContractError(f"build finished without producing {library}")
    manifest = {
        "schema_version": CACHE_SCHEMA_VERSION,
        "created_at": datetime.now(timezone.utc).isoformat(),
        "artifacts": {
            "moe": {
                "ffi": {
                    "path": LIBRARY_NAME,
                    "sha256": _sha256(library),
                    "bytes": library.stat().st_size,
                    "kind": "ffi",
                    "arch": ARCH,
                    "compiler": _compiler_version(hipcc),
                    "sources": {name: _sha256(source_dir() / name) for name in SOURCE_FILES},
                },
                "standalone_test": {
                    "path": NATIVE_TEST_NAME,
                    "sha256": _sha256(out_dir / NATIVE_TEST_NAME),
                    "bytes": (out_dir / NATIVE_TEST_NAME).stat().st_size,
                    "kind": "standalone_test",
                    "arch": ARCH,
                },
            }
        },
    }
    (out_dir / MANIFEST_NAME).write_text(json.dumps(manifest, indent=2, sort_keys=True) + "\n")
    return manifest


if __name__ == "__main__":
    print(json.dumps(compile_kernels(), indent=2, sort_keys=True))
