"""Runs the stand-alone native check of the grouped GEMM kernels (its own reference,
no Python in the loop), the way the reference keeps a test binary per kernel
(src/jaxtitan/kernels/cuda/rmsnorm/rmsnorm_test.cu)."""

from __future__ import annotations

import subprocess

import pytest

from research_amd import build

pytestmark = pytest.mark.gpu


def test_native_gemm_check_passes(gpu):
    binary = build.cache_dir() / build.NATIVE_TEST_NAME
    assert binary.exists(), "run __graft_entry__.build() first"
    proc = subprocess.run([binary.as_posix()], capture_output=True, text=True, timeout=110)
    print(proc.stdout, flush=True)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert proc.stdout.strip().endswith("PASS")
    assert proc.stdout.count("bad=0") == proc.stdout.count("case ") >= 8
