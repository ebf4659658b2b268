"""The fused layer call and the stand-alone router + dispatch entry points give the same bits.

Inside jtmoe_moe_forward the router leaves work to the dispatch behind it: at large batches the
per-expert statistics (expert_counts / importance of _router_stats, moe.py:802-805) are summed by the
dispatch's histogram pass instead of by the router's atomics, and at small batches the router's
finishing workgroup writes the dispatch plan itself.  Whatever route a shape takes, every routing
output of the layer must equal, bit for bit, what jtmoe_router followed by jtmoe_dispatch return on
the same inputs (those two are tied to the oracle by test_gpu_parity.py); the statistics are sums in
32.32 fixed point, so the order of summation cannot show.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from research_amd import _ffi, ops
from test_gpu_parity import dev, host

pytestmark = pytest.mark.gpu

# (tokens, hidden, experts, top_k, d_ff, dtype): the routes are chosen by tokens, tokens * top_k,
# the dtype and whether hidden / experts suit the matrix-core router
CASES = [
    (0, 128, 16, 2, 64, "bf16"),      # empty batch: zeros everywhere
    (5, 128, 16, 2, 64, "bf16"),      # finishing workgroup writes the plan
    (64, 2048, 64, 8, 128, "bf16"),   # the decode shape of the benchmark
    (200, 256, 256, 16, 64, "bf16"),  # 256 experts: the 64-token finishing workgroup is out, tokens > 64
    (50, 256, 256, 16, 64, "bf16"),   # 256 experts: 64-token finishing workgroup with the plan
    (256, 128, 32, 8, 64, "bf16"),    # the largest batch of the small-batch router
    (257, 128, 32, 8, 64, "bf16"),    # 64-token workgroups, one-workgroup dispatch with the statistics
    (1024, 128, 128, 8, 64, "bf16"),  # 8192 assignments: the largest one-workgroup dispatch
    (1025, 128, 128, 8, 64, "bf16"),  # 8200 assignments: histogram and rank passes with the statistics
    (5000, 192, 64, 6, 64, "bf16"),   # several chunks, ragged last chunk: histogram + rank passes
    (33000, 128, 48, 8, 64, "bf16"),  # 258 chunks: histogram, scan and rank passes
    (300, 100, 24, 3, 40, "bf16"),    # hidden and experts the matrix-core router does not take
    (7, 48, 5, 2, 24, "f32"),
    (2100, 64, 8, 4, 32, "f32"),      # fp32: generic router, 8400 assignments
    (0, 64, 8, 4, 32, "f32"),
]


@pytest.mark.parametrize("tokens,hidden,experts,top_k,d_ff,dtype", CASES)
def test_layer_routing_outputs_equal_the_stand_alone_entry_points(gpu, tokens, hidden, experts, top_k, d_ff, dtype):
    rng = np.random.default_rng(tokens * 31 + experts)
    x = dev(rng.standard_normal((tokens, hidden)).astype(np.float32), gpu, dtype)
    w_router = dev((rng.standard_normal((hidden, experts)) * 0.1).astype(np.float32), gpu, dtype)
    bias = dev((rng.standard_normal(experts) * 0.01).astype(np.float32), gpu)
    gate = dev((rng.standard_normal((experts, hidden, d_ff)) * 0.05).astype(np.float32), gpu, dtype)
    up = dev((rng.standard_normal((experts, hidden, d_ff)) * 0.05).astype(np.float32), gpu, dtype)
    down = dev((rng.standard_normal((experts, d_ff, hidden)) * 0.05).astype(np.float32), gpu, dtype)

    layer = ops.moe_forward(x, w_router, bias, gate, up, down, top_k, 1.5)
    route = ops.router(x, w_router, bias, top_k, 1.5)
    plan = ops.dispatch(route.expert_ids, experts)

    for name in ("expert_ids", "weights", "scores", "expert_counts", "importance"):
        assert torch.equal(getattr(layer, name), getattr(route, name)), name
    for name in ("group_sizes", "offsets", "source_order", "inverse"):
        assert torch.equal(getattr(layer, name), getattr(plan, name)), name
    # and the statistics are what the ids and weights say
    stats = O.router_stats(host(route.expert_ids), host(route.weights), experts)
    assert np.array_equal(host(layer.expert_counts), stats.expert_counts)
    np.testing.assert_allclose(host(layer.importance), stats.importance, rtol=1e-5, atol=1e-5)
    assert int(layer.group_sizes.sum()) == tokens * top_k


def test_layer_statistics_do_not_depend_on_what_the_buffers_held(gpu):
    """The layer's scratch is never cleared between calls: a second call on other inputs through the same
    workspace and output buffers must not see the first one's sums."""
    rng = np.random.default_rng(9)
    H, E, K, I = 128, 32, 4, 64
    w_router = dev((rng.standard_normal((H, E)) * 0.1).astype(np.float32), gpu, "bf16")
    gate = dev((rng.standard_normal((E, H, I)) * 0.05).astype(np.float32), gpu, "bf16")
    up = dev((rng.standard_normal((E, H, I)) * 0.05).astype(np.float32), gpu, "bf16")
    down = dev((rng.standard_normal((E, I, H)) * 0.05).astype(np.float32), gpu, "bf16")
    for tokens in (4096, 3000, 40, 4096):
        x = dev(rng.standard_normal((tokens, H)).astype(np.float32), gpu, "bf16")
        layer = ops.moe_forward(x, w_router, None, gate, up, down, K, 1.0)
        route = ops.router(x, w_router, None, K, 1.0)
        assert torch.equal(layer.expert_counts, route.expert_counts), tokens
        assert torch.equal(layer.importance, route.importance), tokens
        assert float(layer.expert_counts.sum()) == tokens * K


def test_layer_routing_outputs_on_seeded_random_shapes(gpu):
    """Forty shapes drawn from a fixed seed (expert counts 1 ... 256 including odd ones, top-k up to 16,
    batches from one token to a few thousand, hidden sizes the matrix-core router takes and others):
    the layer call against the stand-alone entry points, bit for bit, for both score functions."""
    check_random_layer_shapes(gpu, seed=2024, cases=40)


def check_random_layer_shapes(gpu, seed: int, cases: int) -> None:
    rng = np.random.default_rng(seed)
    for case in range(cases):
        experts = int(rng.choice([1, 2, 3, 5, 8, 16, 24, 32, 63, 64, 100, 128, 255, 256]))
        top_k = int(rng.integers(1, min(experts, 16) + 1))
        tokens = int(rng.choice([1, 2, 15, 16, 17, 63, 64, 65, 200, 256, 257, 600, 1030, 2500]))
        hidden = int(rng.choice([8, 40, 64, 128, 192, 256]))
        d_ff = int(rng.choice([8, 24, 64]))
        dtype = "bf16" if rng.random() < 0.75 else "f32"
        score_func = "softmax" if rng.random() < 0.3 else "sigmoid"
        x = dev(rng.standard_normal((tokens, hidden)).astype(np.float32), gpu, dtype)
        w_router = dev((rng.standard_normal((hidden, experts)) * 0.2).astype(np.float32), gpu, dtype)
        bias = dev((rng.standard_normal(experts) * 0.01).astype(np.float32), gpu) if rng.random() < 0.5 else None
        gate = dev((rng.standard_normal((experts, hidden, d_ff)) * 0.05).astype(np.float32), gpu, dtype)
        up = dev((rng.standard_normal((experts, hidden, d_ff)) * 0.05).astype(np.float32), gpu, dtype)
        down = dev((rng.standard_normal((experts, d_ff, hidden)) * 0.05).astype(np.float32), gpu, dtype)
        tag = f"case {case}: T={tokens} H={hidden} E={experts} K={top_k} I={d_ff} {dtype} {score_func}"
        print("[layer paths]", tag, flush=True)
        layer = ops.moe_forward(x, w_router, bias, gate, up, down, top_k, 1.0, score_func=score_func)
        route = ops.router(x, w_router, bias, top_k, 1.0, score_func=score_func)
        plan = ops.dispatch(route.expert_ids, experts)
        for name in ("expert_ids", "weights", "scores", "expert_counts", "importance"):
            assert torch.equal(getattr(layer, name), getattr(route, name)), f"{tag}: {name}"
        for name in ("group_sizes", "offsets", "source_order", "inverse"):
            assert torch.equal(getattr(layer, name), getattr(plan, name)), f"{tag}: {name}"
        d = O.dispatch(host(route.expert_ids), experts)
        assert np.array_equal(host(plan.source_order), d.source_order), tag
        assert np.array_equal(host(plan.group_sizes), d.group_sizes), tag
        assert bool(torch.isfinite(layer.y.float()).all()), tag


# (tokens, hidden, experts, top_k, d_ff, shared width): at most 64 tokens, tokens * top_k >= 2 * experts,
# 16 / 32 / 64 experts, hidden a multiple of 128
DECODE_CASES = [
    (64, 2048, 64, 8, 1408, 0),   # the decode shape of the benchmark
    (64, 2048, 64, 8, 128, 256),  # with shared experts
    (16, 256, 64, 8, 64, 0),      # tokens * top_k = 2 * experts: the smallest batch that takes the path
    (40, 128, 16, 2, 192, 0),     # one slice of the hidden dimension, three token blocks (the last ragged)
    (64, 256, 32, 4, 128, 0),
    (48, 384, 16, 2, 64, 64),     # three slices
    (1, 1920, 16, 16, 64, 0),     # one token that picks every expert; 15 chunks: slices of two, the last of one
    (33, 192, 8, 8, 64, 64),      # 8 experts, hidden not a multiple of 128: the ordinary path
    (15, 256, 64, 8, 64, 0),      # one token short: the ordinary path (the comparison must hold either way)
]


@pytest.mark.parametrize("tokens,hidden,experts,top_k,d_ff,shared_width", DECODE_CASES)
def test_decode_path_equals_the_stand_alone_operators(gpu, tokens, hidden, experts, top_k, d_ff, shared_width):
    """At decode-sized batches one launch runs every token through every expert while a few of its
    workgroups are the router and write the dispatch plan, and the down projection picks the routed rows.
    Every output must equal, bit for bit, router -> dispatch -> gathering grouped SwiGLU -> combine called
    one by one, twice in a row, and through a workspace that a larger call has used in between."""
    rng = np.random.default_rng(tokens * 131 + experts)
    x = dev(rng.standard_normal((tokens, hidden)).astype(np.float32), gpu, "bf16")
    w_router = dev((rng.standard_normal((hidden, experts)) * 0.1).astype(np.float32), gpu, "bf16")
    gate = dev((rng.standard_normal((experts, hidden, d_ff)) * 0.05).astype(np.float32), gpu, "bf16")
    up = dev((rng.standard_normal((experts, hidden, d_ff)) * 0.05).astype(np.float32), gpu, "bf16")
    down = dev((rng.standard_normal((experts, d_ff, hidden)) * 0.05).astype(np.float32), gpu, "bf16")
    shared = None
    if shared_width:
        shared = tuple(dev((rng.standard_normal(s) * 0.05).astype(np.float32), gpu, "bf16")
                       for s in ((hidden, shared_width), (hidden, shared_width), (shared_width, hidden)))

    route = ops.router(x, w_router, None, top_k, 1.0)
    plan = ops.dispatch(route.expert_ids, experts)
    packed_y = ops.grouped_swiglu_gather(x, plan.source_order, top_k, gate, up, down, plan.group_sizes, plan.offsets)
    want = ops.combine(packed_y, plan.inverse, route.weights, None if shared is None else ops.shared_swiglu(x, *shared))

    first = ops.moe_forward(x, w_router, None, gate, up, down, top_k, 1.0, shared=shared)
    assert torch.equal(first.y, want)
    for name in ("expert_ids", "weights", "scores", "expert_counts", "importance"):
        assert torch.equal(getattr(first, name), getattr(route, name)), name
    for name in ("group_sizes", "offsets", "source_order", "inverse"):
        assert torch.equal(getattr(first, name), getattr(plan, name)), name
    big = dev(rng.standard_normal((300, hidden)).astype(np.float32), gpu, "bf16")
    ops.moe_forward(big, w_router, None, gate, up, down, top_k, 1.0, shared=shared)  # other rows through the same workspace
    again = ops.moe_forward(x, w_router, None, gate, up, down, top_k, 1.0, shared=shared)
    assert torch.equal(again.y, want)
    torch.cuda.synchronize()


def test_decode_path_on_seeded_random_shapes(gpu):
    """The same comparison on 48 shapes drawn around the path's conditions (token counts either side of 64
    and of top_k * tokens = 2 * experts, 8 ... 64 experts, hidden sizes with one, several and ragged
    slices, with and without shared experts): whichever path a shape takes, the layer equals its operators
    called one by one."""
    rng = np.random.default_rng(20251)
    taken = 0
    for _ in range(48):
        experts = int(rng.choice([8, 16, 32, 64]))
        top_k = int(rng.integers(1, min(experts, 16) + 1))
        tokens = int(rng.integers(1, 70))
        hidden = int(rng.choice([128, 192, 256, 384, 512, 640, 1024, 1152, 2048, 2176]))
        d_ff = int(rng.choice([64, 128, 192, 320, 704]))
        shared_width = int(rng.choice([0, 0, 64, 128]))
        decode = bool(_ffi.load_library().jtmoe_moe_forward_takes_decode_path(tokens, hidden, experts, top_k, d_ff,
                                                                             _ffi.JTMOE_BF16))
        taken += decode
        print(f"[layer paths] decode sweep: T={tokens} H={hidden} E={experts} K={top_k} I={d_ff} shared={shared_width} "
              f"decode path={decode}", flush=True)
        test_decode_path_equals_the_stand_alone_operators(gpu, tokens, hidden, experts, top_k, d_ff, shared_width)
    assert 8 <= taken <= 40  # the draw covers both sides


def test_decode_path_follows_work_on_the_callers_stream(gpu):
    """The call is ordered on the caller's stream like any other: its input may still be being written
    there when the call is enqueued, and its output is read there right after."""
    rng = np.random.default_rng(77)
    T, H, E, K, I = 64, 512, 64, 8, 128
    w_router = dev((rng.standard_normal((H, E)) * 0.1).astype(np.float32), gpu, "bf16")
    gate = dev((rng.standard_normal((E, H, I)) * 0.05).astype(np.float32), gpu, "bf16")
    up = dev((rng.standard_normal((E, H, I)) * 0.05).astype(np.float32), gpu, "bf16")
    down = dev((rng.standard_normal((E, I, H)) * 0.05).astype(np.float32), gpu, "bf16")
    base = dev(rng.standard_normal((T, H)).astype(np.float32), gpu, "bf16")
    want = ops.moe_forward((base.float() * 2).to(torch.bfloat16), w_router, None, gate, up, down, K, 1.0).y.clone()
    torch.cuda.synchronize()
    stream = torch.cuda.Stream(device=gpu)
    stream.wait_stream(torch.cuda.current_stream(gpu))
    with torch.cuda.stream(stream):
        for _ in range(5):
            filler = torch.randn((4096, 4096), device=gpu) @ torch.randn((4096, 4096), device=gpu)  # keeps the stream busy
            x = (base.float() * 2).to(torch.bfloat16)  # written on this stream right before the call
            y = ops.moe_forward(x, w_router, None, gate, up, down, K, 1.0).y
            doubled = y.float() * 2  # read on this stream right after the call
            assert torch.equal(doubled, want.float() * 2)
            del filler
    torch.cuda.current_stream(gpu).wait_stream(stream)
    torch.cuda.synchronize()


def test_decode_path_on_two_streams_at_once(gpu):
    """Calls share no state but their arguments: decode calls enqueued on two streams, each with its own
    workspace and outputs, may run at the same time and give the results of calls made one after the other
    (the arrival word of the decode launch lives in the workspace; also after a workspace was filled with
    ones, i.e. starts from a word that is neither zero nor a tag)."""
    rng = np.random.default_rng(5)
    T, H, E, K, I = 64, 1024, 64, 8, 256
    w_router = dev((rng.standard_normal((H, E)) * 0.1).astype(np.float32), gpu, "bf16")
    gate = dev((rng.standard_normal((E, H, I)) * 0.05).astype(np.float32), gpu, "bf16")
    up = dev((rng.standard_normal((E, H, I)) * 0.05).astype(np.float32), gpu, "bf16")
    down = dev((rng.standard_normal((E, I, H)) * 0.05).astype(np.float32), gpu, "bf16")
    xs = [dev(rng.standard_normal((T, H)).astype(np.float32), gpu, "bf16") for _ in range(2)]
    want = [ops.moe_forward(x, w_router, None, gate, up, down, K, 1.0) for x in xs]
    torch.cuda.synchronize()
    nbytes = ops._lib().jtmoe_workspace_bytes(T, H, E, K, I, 0, ops._code(torch.bfloat16))
    spaces = [torch.full((nbytes,), 0xff, dtype=torch.uint8, device=gpu) for _ in range(2)]
    streams = [torch.cuda.Stream(device=gpu) for _ in range(2)]
    torch.cuda.synchronize()  # the fills above ran on the default stream
    got = [[], []]
    for _ in range(20):
        for i in range(2):
            with torch.cuda.stream(streams[i]):
                got[i].append(ops.moe_forward(xs[i], w_router, None, gate, up, down, K, 1.0, workspace=spaces[i]))
    torch.cuda.synchronize()
    for i in range(2):
        for r in got[i]:
            assert torch.equal(r.y, want[i].y) and torch.equal(r.source_order, want[i].source_order)
            assert torch.equal(r.expert_counts, want[i].expert_counts)


def test_calls_from_four_host_threads_at_once(gpu):
    """The entry points are called from whatever thread the host's executor uses
    (src/jaxtitan/kernels/cuda/rmsnorm/rmsnorm_ffi.cu:59-68: re-entrant, work only on the stream handed in):
    four threads, each with its own stream, workspace and shape -- a decode call, a small batch, one that
    takes the large-batch kernels, one in fp32 -- call the layer 25 times each at the same time (ctypes
    releases the interpreter lock for the duration of a call) and get what a single thread got."""
    import threading

    rng = np.random.default_rng(9)
    cases = []
    for tokens, hidden, experts, top_k, d_ff, dtype in [(64, 512, 64, 8, 128, "bf16"), (200, 256, 16, 2, 192, "bf16"),
                                                        (1500, 512, 32, 4, 128, "bf16"), (90, 64, 8, 2, 40, "f32")]:
        a = [dev(rng.standard_normal((tokens, hidden)).astype(np.float32), gpu, dtype),
             dev((rng.standard_normal((hidden, experts)) * 0.1).astype(np.float32), gpu, dtype), None,
             dev((rng.standard_normal((experts, hidden, d_ff)) * 0.05).astype(np.float32), gpu, dtype),
             dev((rng.standard_normal((experts, hidden, d_ff)) * 0.05).astype(np.float32), gpu, dtype),
             dev((rng.standard_normal((experts, d_ff, hidden)) * 0.05).astype(np.float32), gpu, dtype), top_k, 1.0]
        cases.append((a, ops.moe_forward(*a)))
    torch.cuda.synchronize()
    errors: list[str] = []
    start = threading.Barrier(len(cases))

    def worker(i):
        args, want = cases[i]
        try:
            stream = torch.cuda.Stream(device=gpu)
            start.wait()
            with torch.cuda.stream(stream):
                for n in range(25):
                    got = ops.moe_forward(*args)
                    stream.synchronize()
                    for name in ("y", "expert_ids", "weights", "scores", "expert_counts", "importance", "source_order"):
                        if not torch.equal(getattr(got, name), getattr(want, name)):
                            errors.append(f"thread {i} call {n}: {name} differs")
                            return
        except Exception as exc:  # noqa: BLE001 -- reported by the assertion below
            errors.append(f"thread {i}: {type(exc).__name__}: {exc}")

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(cases))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    torch.cuda.synchronize()
    assert not any(t.is_alive() for t in threads), "a thread did not finish"
    assert not errors, errors[:4]


@pytest.mark.parametrize("tokens", [40, 64, 300, 3000])
def test_layer_statistics_with_a_non_finite_token(gpu, tokens):
    """A token whose input is NaN has NaN logits, scores and route weights.  Its ids stay inside [0, E)
    (NaN scores are chosen last, lower index first: experts 0 .. K-1), it is counted like any other token,
    and its NaN weights add nothing to the importance sums (a 32.32 fixed-point sum has no NaN) -- on every
    route the statistics take: the router's finishing workgroup, the decode launch, the one-workgroup
    dispatch and the histogram pass."""
    rng = np.random.default_rng(tokens)
    H, E, K, I = 256, 64, 8, 64
    x = rng.standard_normal((tokens, H)).astype(np.float32)
    x[3, :] = np.nan
    w_router = dev((rng.standard_normal((H, E)) * 0.1).astype(np.float32), gpu, "bf16")
    gate = dev((rng.standard_normal((E, H, I)) * 0.05).astype(np.float32), gpu, "bf16")
    up = dev((rng.standard_normal((E, H, I)) * 0.05).astype(np.float32), gpu, "bf16")
    down = dev((rng.standard_normal((E, I, H)) * 0.05).astype(np.float32), gpu, "bf16")
    layer = ops.moe_forward(dev(x, gpu, "bf16"), w_router, None, gate, up, down, K, 1.0)
    ids, weights = host(layer.expert_ids), host(layer.weights)
    assert ids.min() >= 0 and ids.max() < E
    assert ids[3].tolist() == list(range(K)) and np.all(np.isnan(weights[3]))
    assert np.array_equal(host(layer.expert_counts), np.bincount(ids.reshape(-1), minlength=E).astype(np.float32))
    importance = host(layer.importance)
    assert np.all(np.isfinite(importance))
    clean = np.where(np.isnan(weights), 0.0, weights).astype(np.float64)
    want = np.zeros(E)
    np.add.at(want, ids.reshape(-1), clean.reshape(-1))
    np.testing.assert_allclose(importance, want, rtol=1e-5, atol=1e-5)
    # every other token is untouched by its neighbour
    others = np.delete(np.arange(tokens), 3)
    assert np.all(np.isfinite(host(layer.y)[others]))
