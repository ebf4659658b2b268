"""bench.py itself: the parts that run without a GPU here, and the whole script on the GPU at a small
configuration.  The driver runs `python bench.py` once at the end of a build, so a slip in a leg that
the kernel tests never touch (the CPU baseline, the JSON line) must show up in the test suite first."""

from __future__ import annotations

import json
import os
import subprocess
import sys
import warnings
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


def test_bench_source_compiles_without_warnings():
    source = (ROOT / "bench.py").read_text()
    with warnings.catch_warnings():
        warnings.simplefilter("error")  # e.g. the SyntaxWarning of two adjacent expressions missing an operator
        compile(source, "bench.py", "exec")


def test_bench_refuses_more_than_one_gpu():
    done = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                          cwd=ROOT)
    assert done.returncode == 2
    assert "one GPU" in done.stderr and done.stdout == ""


@pytest.mark.parametrize("name,tokens", [("C1", 64), ("C2", 32), ("C1", None)])
def test_cpu_baseline_record(name, tokens, monkeypatch):
    sys.path.insert(0, str(ROOT))
    import bench

    record = bench.cpu_baseline(name, tokens)
    assert record["unit"] == "tokens/s" and record["kind"] == "port"
    assert record["value"] > 0 and record["cores"] >= 1
    assert ("all" if tokens is None else f"first {tokens}") in record["sample"]
    assert "timed call" in record["sample"]
    json.dumps(record)


@pytest.mark.gpu
@pytest.mark.parametrize("config", ["C5", "C1"])
def test_bench_line_on_the_gpu(config):
    """The whole script, every leg, at a configuration that takes seconds: one JSON line with the
    fields the benchmark contract names."""
    env = dict(os.environ)
    done = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--config", config, "--steps", "5", "--warmup", "2",
                           "--cpu-sample-tokens", "64"], capture_output=True, text=True, cwd=ROOT, env=env,
                          timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [line for line in done.stdout.splitlines() if line.strip()]
    assert len(lines) == 1
    line = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 5 and line["value"] > 0
    assert set(("bound", "achieved", "peak", "unit", "frac", "traffic")) <= set(line["roofline"])
    assert set(("value", "unit", "cores", "kind", "sample")) <= set(line["cpu_baseline"])
    assert "workload" in line["config"]
