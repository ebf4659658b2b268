"""Benchmark of the MoE expert-layer forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C3] [--no-cpu-baseline]

A step is one whole-layer forward (router -> dispatch -> grouped SwiGLU ->
shared experts -> combine) over one batch of synthetic, seeded input that is
already resident in HBM.  The timed region is exactly K calls of the C entry
point jtmoe_moe_forward bracketed by torch.cuda.synchronize().  After it, K more
steps are run through jtmoe_moe_forward_timed, which records a hipEvent on the
launch stream after every stage; the per-stage averages give the roofline
figures.  Prints ONE JSON line.
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
MFMA_F32_PEAK_TFLOPS = 157.3


def algorithmic_work(cfg: dict) -> dict:
    """Algorithmic flops / bytes per launch of each stage (one unit = one layer call)."""
    T = cfg["batch"] * cfg["seq"]
    H, E, K, I, Ns = cfg["H"], cfg["E"], cfg["K"], cfg["I"], cfg["Ns"]
    b = 2 if cfg["dtype"] == "bf16" else 4
    A = T * K
    Is = I * Ns
    return dict(
        router_bytes=T * H * b + H * E * b + E * 4 + A * 4 + A * b + T * E * 4,
        dispatch_bytes=A * 4 + 2 * E * 4 + 2 * A * 4 + T * H * b + A * H * b,
        dispatch_rows_bytes=A * 4 + T * H * b + A * H * b,
        combine_bytes=A * H * b + A * b + A * 4 + T * H * b + (T * H * b if Ns else 0),
        gate_up_flops=4 * A * H * I,
        down_flops=2 * A * I * H,
        shared_gate_up_flops=4 * T * H * Is,
        shared_down_flops=2 * T * Is * H,
        router_flops=2 * T * H * E,
    )


def measured_traffic(config: str, kernel: str):
    """HBM bytes per launch of `kernel` from the committed rocprofv3 --pmc summary (None if absent), and
    where that figure comes from.

    bench.py cannot read hardware counters itself; profiles/hbm_traffic.json holds the scaled
    FETCH_SIZE + WRITE_SIZE figures of the same command, names the command that produced them and the
    source revision of the kernels they were taken on (a schedule change makes them stale)."""
    path = ROOT / "profiles" / "hbm_traffic.json"
    try:
        table = json.loads(path.read_text())
        value = table[config][kernel]["hbm_bytes_per_launch"]
    except (OSError, KeyError, ValueError):
        return None, None
    return value, {"file": "profiles/hbm_traffic.json", "kernels_at": table.get("_kernels_at"),
                   "measured_on": table.get("_measured_on")}


def cpu_baseline(name: str, sample_tokens: int | None) -> dict:
    """The oracle (a NumPy port of the reference layer) timed on the host cores,
    on the first `sample_tokens` tokens of the same seeded workload (None: all of them)."""
    import numpy as np

    from oracle import moe_oracle as O

    inp = O.make_inputs(name, seed=0, tokens=sample_tokens)
    cfg = inp["cfg"]
    whole = sample_tokens is None
    if whole:
        sample_tokens = cfg["batch"] * cfg["seq"]
    kwargs = dict(top_k=cfg["K"], route_scale=1.0, dtype=cfg["dtype"], shared=inp["shared"])
    args = (inp["x"], inp["w_router"], inp["expert_bias"], inp["gate"], inp["up"], inp["down"])
    small = inp["x"][:, : min(64, sample_tokens)]
    O.moe_forward(small, *args[1:], **kwargs)  # first call excluded
    # whole calls until at least two seconds of host work have been timed, and never fewer than two calls
    # (at the large shapes a call takes several seconds: two of them, the mean reported)
    calls, t0 = 0, time.perf_counter()
    while True:
        out = O.moe_forward(*args, **kwargs)
        calls += 1
        total = time.perf_counter() - t0
        if (total >= 2.0 and calls >= 2) or calls >= 200:
            break
    dt = total / calls
    assert np.isfinite(out.y).all()
    cores = len(os.sched_getaffinity(0))
    try:
        from threadpoolctl import threadpool_info

        blas = [p.get("num_threads") for p in threadpool_info() if p.get("user_api") == "blas"]
        if blas:
            cores = int(max(blas))
    except Exception:
        pass
    return dict(
        value=sample_tokens / dt,
        unit="tokens/s",
        cores=cores,
        kind="port",
        sample=(f"all {sample_tokens} tokens of {name}" if whole else f"first {sample_tokens} tokens of {name}")
               + f" (seed-0 weights), NumPy oracle, {'emulated bf16' if cfg['dtype'] == 'bf16' else 'fp32'}, "
               + (f"{calls} timed calls of {dt:.3f} s each" if calls > 1 else f"one timed call of {dt:.2f} s")
               + " after a 64-token warm-up call",
    )


def graph_timing(x, w_r, bias, gate, upw, down, shared, cfg, steps, warmup=3) -> dict:
    """Small batches are bound by launching the layer's kernels from Python, not by the kernels: the same
    calls captured once into a HIP graph and replayed."""
    import torch

    from research_amd.graph import GraphedLayer

    layer = GraphedLayer(x, w_r, bias, gate, upw, down, cfg["K"], 1.0, shared=shared)
    for _ in range(max(warmup, 3)):
        layer.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        layer.replay()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    return {"ms_per_step": ms, "tokens_per_s": x.shape[0] / (ms * 1e-3), "steps": steps}


def block_timing(x, w_r, bias, gate, upw, down, shared, cfg, steps, layer_ms, warmup=3) -> dict:
    """x + post_norm(moe(pre_norm(x))): the layer with the decoder block's two RMSNorms and the residual
    add around it (the post-norm and the add run inside the combine kernel)."""
    import torch

    from research_amd import ops

    dev = x.device
    pre = torch.ones((cfg["H"],), dtype=torch.float32, device=dev)
    post = torch.full((cfg["H"],), 0.5, dtype=torch.float32, device=dev)

    def block():
        return ops.ffn_block_forward(x, pre, post, 1e-6, w_r, bias, gate, upw, down, cfg["K"], 1.0, shared=shared)

    def layer():
        return ops.moe_forward(x, w_r, bias, gate, upw, down, cfg["K"], 1.0, shared=shared)

    def timed(step):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    # The bare layer is timed again here, between two timings of the block, in the state of the chip that
    # the block is timed in: the headline figure was taken several legs earlier, and the clocks it ran at
    # are not the clocks of this moment.
    for _ in range(max(warmup, 3)):
        block()
    first = timed(block)
    bare = timed(layer)
    second = timed(block)
    ms = 0.5 * (first + second)
    return {"ms_per_step": ms, "tokens_per_s": x.shape[0] / (ms * 1e-3), "layer_ms_beside_it": bare,
            "over_layer_ms": ms - bare, "over_headline_ms": ms - layer_ms}


def train_timing(x, w_r, bias, gate, upw, down, shared, cfg, steps, work) -> dict:
    """Forward that keeps residuals + backward (all gradients): medians of event timings over `steps` pairs.

    Not the headline metric (that is the forward layer); reported beside it.  The backward does
    twice the matrix-product work of the forward: one data-gradient and one weight-gradient
    product for each forward product.
    """
    import torch

    from research_amd import grad

    dev = x.device
    dy = torch.randn(x.shape, device=dev).to(x.dtype)
    d_scores = torch.randn((x.shape[0], cfg["E"]), device=dev) * 0.01

    def fwd():
        return grad.moe_forward_train(x, w_r, bias, gate, upw, down, cfg["K"], 1.0, shared=shared)

    def bwd(result, residuals):
        return grad.moe_backward(x, dy, d_scores, w_r, gate, upw, down, shared, result, residuals, 1.0)

    for _ in range(3):  # lets torch's caching allocator settle on the buffers it will reuse
        result, residuals = fwd()
        bwd(result, residuals)
    torch.cuda.synchronize()
    # events are recorded for every step and read after one final synchronisation, so that the host
    # runs ahead of the GPU as it does in a training loop (no idle gaps from launch latency)
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    for e in ev:
        e[0].record()
        result, residuals = fwd()
        e[1].record()
        bwd(result, residuals)
        e[2].record()
    torch.cuda.synchronize()
    fwd_ms = statistics.median(e[0].elapsed_time(e[1]) for e in ev)
    bwd_ms = statistics.median(e[1].elapsed_time(e[2]) for e in ev)
    gemm_flops = 2.0 * (work["gate_up_flops"] + work["down_flops"] + work["shared_gate_up_flops"]
                        + work["shared_down_flops"])
    return {
        "forward_with_residuals_ms": fwd_ms,
        "backward_ms": bwd_ms,
        "tokens_per_s_forward_backward": x.shape[0] / ((fwd_ms + bwd_ms) * 1e-3),
        "backward_gemm_flops": gemm_flops,
        "backward_tflops": gemm_flops / (bwd_ms * 1e-3) / 1e12 if bwd_ms > 0 else 0.0,
        "gradients": "x, router, gate, up, down" + (", shared gate/up/down" if shared is not None else ""),
    }


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    # defaults: 50 timed steps after 20 untimed ones at the large configurations (C3: 54 + 135 ms of load);
    # the small ones get as many as keep the chip under load for about as long before and while timing
    # (its clocks need some tens of milliseconds to settle): C2 150 + 400, C5 300 + 800, C1 300 + 800
    parser.add_argument("--steps", type=int, default=None)
    parser.add_argument("--warmup", type=int, default=None)
    parser.add_argument("--config", default="C3", choices=["C1", "C2", "C3", "C4", "C5"])
    parser.add_argument("--cpu-sample-tokens", type=int, default=16384,
                        help="tokens of the workload the CPU baseline runs (the whole of C3 takes about 9 s of host work)")
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-train", action="store_true", help="skip the forward+backward timing")
    parser.add_argument("--no-block", action="store_true", help="skip the decoder-block and graph-replay timings")
    args = parser.parse_args()
    default_warmup, default_steps = {"C2": (150, 400), "C5": (300, 800), "C1": (300, 800)}.get(args.config, (20, 50))
    if args.steps is None:
        args.steps = default_steps
    if args.warmup is None:
        args.warmup = default_warmup
    if args.gpus != 1:
        print(f"bench.py measures one GPU: the layer runs with every expert local and no collective; "
              f"--gpus {args.gpus} is not supported in this build", file=sys.stderr)
        return 2

    import torch

    from research_amd import _ffi, ops
    from research_amd.synthetic import DESCRIPTIONS, make_inputs

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU path)", file=sys.stderr)
        return 2
    _ffi.load_library()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    inp = make_inputs(args.config, seed=0)
    cfg = inp["cfg"]
    tdtype = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float32
    T = cfg["batch"] * cfg["seq"]

    def up(a):
        return torch.from_numpy(a).to(dev).to(tdtype).contiguous()

    x = up(inp["x"].reshape(T, cfg["H"]))
    w_r, gate, upw, down = up(inp["w_router"]), up(inp["gate"]), up(inp["up"]), up(inp["down"])
    bias = torch.from_numpy(inp["expert_bias"]).to(dev)
    shared = None if inp["shared"] is None else tuple(up(m) for m in inp["shared"])
    del inp
    torch.cuda.synchronize()

    def step(stage_ms=None):
        return ops.moe_forward(x, w_r, bias, gate, upw, down, cfg["K"], 1.0, shared=shared, stage_ms=stage_ms)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps

    # per-call latencies (the reference's protocol: perf_counter around a blocking call)
    lat = []
    for _ in range(max(args.steps, 10)):
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        step()
        torch.cuda.synchronize()
        lat.append((time.perf_counter() - t1) * 1e3)
    lat.sort()

    # per-stage durations from hipEvents on the launch stream
    per_stage = [[] for _ in range(_ffi.NUM_STAGES)]
    for _ in range(args.steps):
        ms: list = []
        result = step(ms)
        for i, v in enumerate(ms):
            per_stage[i].append(v)
    stage_ms = {name: (sum(v) / len(v) if v else 0.0) for name, v in zip(_ffi.STAGE_NAMES, per_stage)}
    group_sizes = result.group_sizes.cpu().tolist()

    # The fused layer applies the permutation inside the GEMM's tile loads, so its dispatch stage
    # moves no rows.  The stand-alone dispatch entry point (histogram + scan + rank + row scatter
    # into packed_x) is what a caller of the stage API runs: time it on the same routing.
    def time_call(fn, iters):
        for _ in range(3):
            fn()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            fn()
        end.record()
        end.synchronize()
        return start.elapsed_time(end) / iters

    lib = _ffi.load_library()
    A_rows = T * cfg["K"]
    ids_fixed = result.expert_ids.clone()
    d_sizes = torch.empty((cfg["E"],), dtype=torch.int32, device=dev)
    d_offs = torch.empty_like(d_sizes)
    d_order = torch.empty((A_rows,), dtype=torch.int32, device=dev)
    d_inv = torch.empty_like(d_order)
    d_packed = torch.empty((A_rows, cfg["H"]), dtype=tdtype, device=dev)
    d_ws = torch.empty((lib.jtmoe_dispatch_workspace_bytes(A_rows, cfg["E"]),), dtype=torch.uint8, device=dev)
    code = _ffi.JTMOE_BF16 if cfg["dtype"] == "bf16" else _ffi.JTMOE_F32
    stream = torch.cuda.current_stream(dev).cuda_stream

    def dispatch_call(with_rows):
        rc = lib.jtmoe_dispatch(ids_fixed.data_ptr(), x.data_ptr() if with_rows else None, T, cfg["H"], cfg["E"],
                                cfg["K"], code, d_sizes.data_ptr(), d_offs.data_ptr(), d_order.data_ptr(),
                                d_inv.data_ptr(), d_packed.data_ptr(), d_ws.data_ptr(), d_ws.numel(), stream)
        assert rc == 0, _ffi.last_error(lib)

    dispatch_ms = time_call(lambda: dispatch_call(True), args.steps)
    dispatch_meta_ms = time_call(lambda: dispatch_call(False), args.steps)
    del d_packed

    work = algorithmic_work(cfg)
    peak = MFMA_BF16_PEAK_TFLOPS if cfg["dtype"] == "bf16" else MFMA_F32_PEAK_TFLOPS

    def tflops(flops, ms):
        return flops / (ms * 1e-3) / 1e12 if ms > 0 else 0.0

    def gbs(nbytes, ms):
        return nbytes / (ms * 1e-3) / 1e9 if ms > 0 else 0.0

    traffic, traffic_source = measured_traffic(args.config, "gate_up")
    gate_up_tf = tflops(work["gate_up_flops"], stage_ms["gate_up"])
    active = sum(1 for g in group_sizes if g > 0)
    elem = 2 if cfg["dtype"] == "bf16" else 4
    # bytes the gate/up launch must move: the gate and up matrices of every expert that received
    # a row, each token row once, the activation rows written
    gate_up_bytes = (2 * active * cfg["H"] * cfg["I"] + T * cfg["H"] + A_rows * cfg["I"]) * elem
    if args.config == "C5":
        # a few rows per expert: the launch streams the expert matrices once and is bound by HBM
        gate_up_gbs = gbs(gate_up_bytes, stage_ms["gate_up"])
        roofline = dict(
            kernel="grouped gate/up GEMM + SwiGLU (routed experts, weight streaming)",
            bound="hbm",
            achieved=gate_up_gbs,
            peak=HBM_PEAK_GBS,
            unit="GB/s",
            frac=gate_up_gbs / HBM_PEAK_GBS,
            traffic=traffic,
            traffic_source=traffic_source,
            avg_launch_ms=stage_ms["gate_up"],
            bytes_per_launch=gate_up_bytes,
        )
    else:
        roofline = dict(
            kernel="grouped gate/up GEMM + SwiGLU (routed experts)",
            bound="mfma",
            achieved=gate_up_tf,
            peak=peak,
            unit="TFLOP/s",
            frac=gate_up_tf / peak,
            traffic=traffic,
            traffic_source=traffic_source,
            avg_launch_ms=stage_ms["gate_up"],
            flops_per_launch=work["gate_up_flops"],
        )
    stages = dict(
        ms=stage_ms,
        standalone_dispatch_ms=dispatch_ms,
        standalone_dispatch_meta_ms=dispatch_meta_ms,
        grouped_gemm_mfma_util=tflops(work["gate_up_flops"] + work["down_flops"], stage_ms["gate_up"] + stage_ms["down"]) / peak,
        down_tflops=tflops(work["down_flops"], stage_ms["down"]),
        shared_tflops=tflops(work["shared_gate_up_flops"] + work["shared_down_flops"],
                             stage_ms["shared_gate_up"] + stage_ms["shared_down"]),
        router_gbs=gbs(work["router_bytes"], stage_ms["router"]),
        dispatch_gbs=gbs(work["dispatch_bytes"], dispatch_ms),
        dispatch_rows_gbs=gbs(work["dispatch_rows_bytes"], max(dispatch_ms - dispatch_meta_ms, 1e-6)),
        combine_gbs=gbs(work["combine_bytes"], stage_ms["combine"]),
        hbm_peak_gbs=HBM_PEAK_GBS,
    )
    # the HBM-bound stages as fractions of the 8 TB/s peak (algorithmic bytes / stage time / peak)
    stages["frac_of_hbm_peak"] = {
        "router": stages["router_gbs"] / HBM_PEAK_GBS,
        "dispatch": stages["dispatch_gbs"] / HBM_PEAK_GBS,
        "dispatch_rows": stages["dispatch_rows_gbs"] / HBM_PEAK_GBS,
        "combine": stages["combine_gbs"] / HBM_PEAK_GBS,
    }
    stages["frac_of_mfma_peak"] = {
        "gate_up": gate_up_tf / peak,
        "down": stages["down_tflops"] / peak,
        "shared": stages["shared_tflops"] / peak,
    }

    line = {
        "metric": "MoE layer tokens/s (64E top-8, d2048); grouped-GEMM MFMA util %",
        "value": T / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": cfg["dtype"],
        "data": "synthetic",
        "config": {
            "workload": f"{args.config}: {DESCRIPTIONS[args.config]}; x~N(0,1), weights~N(0,0.02), seed 0, "
                        "sigmoid top-k router (the reference's), inputs resident in HBM",
            "tokens": T, "d_model": cfg["H"], "experts": cfg["E"], "top_k": cfg["K"], "d_ff": cfg["I"],
            "shared_experts": cfg["Ns"],
            "group_rows_min_max": [min(group_sizes), max(group_sizes)],
        },
        "latency_ms": {
            "median": statistics.median(lat), "p10": lat[int(0.1 * (len(lat) - 1))],
            "p90": lat[int(0.9 * (len(lat) - 1))], "min": lat[0], "max": lat[-1],
        },
        "roofline": roofline,
        "stages": stages,
    }
    if lib.jtmoe_moe_forward_takes_decode_path(T, cfg["H"], cfg["E"], cfg["K"], cfg["I"], code):
        line["stages"]["note"] = ("decode path: the gate/up stage is one launch that runs every token through every "
                                  "expert and holds the router and the dispatch plan in a few of its workgroups")
    if not args.no_block:
        if T <= 2048:
            line["graph_replay"] = graph_timing(x, w_r, bias, gate, upw, down, shared, cfg, max(args.steps, 50), args.warmup)
        line["block"] = block_timing(x, w_r, bias, gate, upw, down, shared, cfg, args.steps, ms_per_step, args.warmup)
    if not args.no_train:
        line["train"] = train_timing(x, w_r, bias, gate, upw, down, shared, cfg, args.steps, work)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(args.config, None if args.cpu_sample_tokens >= T else args.cpu_sample_tokens)
        # the configuration BASELINE.json names for the CPU (C1: fp32, 2048 tokens, 8 experts), in full
        line["cpu_baseline_c1"] = cpu_baseline("C1", None)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
