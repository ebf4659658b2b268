"""The bf16 configurations at their full sizes -- C2 (8192 tokens, d_model 1024, 16 experts, top-2,
d_ff 2816), C3 (the headline: 16384 tokens, d_model 2048, 64 experts, top-8, d_ff 1408, two shared
experts) and C4 (16384 tokens, 128 experts, top-8, d_ff 768, routing skewed by a Zipf expert bias:
groups of 0 ... ~9950 rows, several experts empty) -- checked through properties that do not need a
CPU run of the whole layer: permutation and histogram invariants, per-token independence against a
sub-batch, additivity of the shared experts, the oracle on a sample of tokens, and for the backward
pass exact homogeneity in the cotangent and additivity of the weight gradients over a split of the
batch.  The edge patterns of the reference's dispatcher tests (an empty expert, total skew;
tests/jaxtitan/test_model.py:580-587) appear here at scale in C4."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from research_amd import grad, ops
from test_gpu_parity import BF16_MAX_REL, dev, host, rel_err, report

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", params=["C2", "C3", "C4"])
def c3(request, gpu):
    """One configuration at full size on the GPU (the fixture keeps the headline's name)."""
    inp = O.make_inputs(request.param, seed=0)
    cfg = inp["cfg"]
    T = cfg["batch"] * cfg["seq"]
    d = dict(name=request.param, cfg=cfg, T=T, inp=inp)
    d["x"] = dev(inp["x"].reshape(T, cfg["H"]), gpu, "bf16")
    for k in ("w_router", "gate", "up", "down"):
        d[k] = dev(inp[k], gpu, "bf16")
    d["bias"] = dev(inp["expert_bias"], gpu)
    d["shared"] = tuple(dev(m, gpu, "bf16") for m in inp["shared"]) if inp["shared"] is not None else None
    yield d
    d.clear()
    torch.cuda.empty_cache()


def run(c3, x=None, shared=True):
    return ops.moe_forward(c3["x"] if x is None else x, c3["w_router"], c3["bias"], c3["gate"], c3["up"], c3["down"],
                           c3["cfg"]["K"], 1.0, shared=c3["shared"] if shared else None)


def test_full_size_plan_invariants(c3):
    cfg, T = c3["cfg"], c3["T"]
    A = T * cfg["K"]
    r = run(c3)
    ids = host(r.expert_ids).reshape(-1)
    order, inverse = host(r.source_order), host(r.inverse)
    sizes, offsets = host(r.group_sizes), host(r.offsets)
    assert sizes.sum() == A and np.array_equal(offsets, np.cumsum(sizes) - sizes)
    assert np.array_equal(sizes, np.bincount(ids, minlength=cfg["E"]))
    assert np.array_equal(np.sort(order), np.arange(A)) and np.array_equal(inverse[order], np.arange(A))
    packed_experts = ids[order]
    assert np.all(np.diff(packed_experts) >= 0)  # expert-major
    same = np.diff(packed_experts) == 0
    assert np.all(np.diff(order)[same] > 0)  # stable: ascending assignment index inside an expert
    assert np.array_equal(order, np.argsort(ids, kind="stable"))
    w = host(r.weights)
    np.testing.assert_allclose(w.sum(-1), 1.0, atol=2e-2)  # normalised route weights (bf16)
    assert np.array_equal(host(r.expert_counts), sizes.astype(np.float32))
    np.testing.assert_allclose(host(r.importance).sum(), w.astype(np.float64).sum(), rtol=1e-5)
    # no token picks an expert twice
    assert np.all(np.diff(np.sort(host(r.expert_ids), axis=1), axis=1) > 0)
    if c3["name"] == "C4":
        # the skewed stress case: the six disabled experts (and possibly more) get nothing, a fifth of the
        # experts take most of the assignments, and the largest group is many tiles tall
        print(f"[parity] C4 groups: empty={int((sizes == 0).sum())} min_nonempty={int(sizes[sizes > 0].min())} "
              f"max={int(sizes.max())} top20%_share={np.sort(sizes)[-cfg['E'] // 5:].sum() / A:.3f}", flush=True)
        assert (sizes == 0).sum() >= 6 and sizes.max() >= 8 * (A // cfg["E"])
        assert np.sort(sizes)[-cfg["E"] // 5:].sum() >= 0.6 * A


def test_full_size_rows_match_sub_batch_and_oracle_sample(c3, gpu):
    cfg, T = c3["cfg"], c3["T"]
    full = run(c3)
    rng = np.random.default_rng(0)
    pick = np.sort(rng.choice(T, size=96, replace=False))
    sub = run(c3, x=c3["x"][torch.from_numpy(pick).to(gpu)].contiguous())
    # A batch this small takes other router kernels (the k range shared out over workgroups) than the full
    # batch; all of them add a logit up in one order, so a token routes the same whatever shares its call
    # (the reference's invariant prefill + decode == full forward, tests/jaxtitan/test_infer.py:270-301).
    for name in ("expert_ids", "weights", "scores"):
        a, b = host(getattr(sub, name)), host(getattr(full, name))[pick]
        assert np.array_equal(a, b), f"{name}: {int((a != b).any(axis=1).sum())} of {len(pick)} rows differ from the full batch"
    err = rel_err(host(sub.y), host(full.y)[pick])
    print(f"[parity] {c3['name']} 96-token sub-batch against the same rows of the full batch: routing identical, "
          f"y max_rel={err:.3e}", flush=True)
    assert err <= 1e-2
    # the oracle on the same tokens, with the kernel's routing
    inp = c3["inp"]
    x2 = inp["x"].reshape(T, cfg["H"])[pick]
    ids = host(full.expert_ids)[pick]
    d = O.dispatch(ids, cfg["E"], O.cast_compute(x2, "bf16"))
    packed_y = O.grouped_swiglu(d.packed_x, inp["gate"], inp["up"], inp["down"], d.group_sizes, "bf16")
    shared_y = O.shared_swiglu(x2, *inp["shared"], "bf16") if inp["shared"] is not None else None
    want = O.combine(packed_y, d.inverse, host(full.weights)[pick], "bf16", shared_y)
    assert report(f"{c3['name']} full size, 96 sampled tokens", host(full.y)[pick], want) <= BF16_MAX_REL


def test_full_size_shared_experts_are_additive(c3):
    if c3["shared"] is None:
        pytest.skip("configuration without shared experts")
    with_shared, without = run(c3), run(c3, shared=False)
    assert torch.equal(with_shared.expert_ids, without.expert_ids)
    shared_y = ops.shared_swiglu(c3["x"], *c3["shared"])
    want = (without.y.float() + shared_y.float()).to(torch.bfloat16)
    assert torch.equal(with_shared.y, want)  # combine adds the shared output in the compute dtype, rounding once


def test_full_size_backward_is_homogeneous_and_additive(c3, gpu):
    cfg, T = c3["cfg"], c3["T"]
    result, residuals = grad.moe_forward_train(c3["x"], c3["w_router"], c3["bias"], c3["gate"], c3["up"], c3["down"],
                                               cfg["K"], 1.0, shared=c3["shared"])
    gen = torch.Generator(device=gpu).manual_seed(3)
    dy = torch.randn(c3["x"].shape, device=gpu, generator=gen).to(torch.bfloat16)
    args = (c3["w_router"], c3["gate"], c3["up"], c3["down"], c3["shared"], result, residuals, 1.0)
    g1 = grad.moe_backward(c3["x"], dy, None, *args)
    # homogeneity: a cotangent scaled by a power of two scales every gradient by the same factor, exactly
    g4 = grad.moe_backward(c3["x"], (dy.float() * 4).to(torch.bfloat16), None, *args)
    for name in ("dx", "d_w_router", "d_gate", "d_up", "d_down"):
        a, b = getattr(g1, name), getattr(g4, name)
        assert bool(torch.isfinite(a.float()).all())
        assert torch.equal((a.float() * 4).to(torch.bfloat16), b), name
    # additivity: cotangents that are zero outside one half of the tokens give gradients that add up
    lo, hi = dy.clone(), dy.clone()
    lo[T // 2:] = 0
    hi[: T // 2] = 0
    ga, gb = grad.moe_backward(c3["x"], lo, None, *args), grad.moe_backward(c3["x"], hi, None, *args)
    assert torch.equal(ga.dx[: T // 2], g1.dx[: T // 2]) and torch.equal(gb.dx[T // 2:], g1.dx[T // 2:])
    assert not ga.dx[T // 2:].any() and not gb.dx[: T // 2].any()
    for name in ("d_gate", "d_down", "d_w_router"):
        total = getattr(ga, name).float() + getattr(gb, name).float()
        ref = getattr(g1, name).float()
        err = float((total - ref).abs().max() / ref.abs().max())
        print(f"[parity] {c3['name']} full size additivity of {name}: max_rel={err:.3e}", flush=True)
        assert err <= BF16_MAX_REL
