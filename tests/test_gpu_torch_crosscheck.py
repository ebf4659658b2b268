"""Forward and backward of the whole layer at sizes the NumPy oracle is too slow for, cross-checked
against a composition of torch routines on the same GPU (autograd for the gradients).

This is not the parity oracle (tests/test_gpu_parity.py, tests/test_gpu_grad.py hold the kernels to
it at smaller sizes): it is a second opinion at shapes with more output tiles than CUs, where the
persistent schedules of the grouped GEMMs (several tiles per workgroup; weight-gradient pairs cut
by work and dealt longest group first) decide which workgroup computes what.  The torch side is
given the library's expert ids, so a near-tie in the router cannot make the two sides route
differently; everything else (scores, weights, experts, combine, shared experts, every gradient)
is its own.  bf16, max|a - b| / max|b| <= 2e-2 per tensor.
"""

from __future__ import annotations

import pytest
import torch

from research_amd import autograd as A

pytestmark = pytest.mark.gpu


def torch_layer_with_ids(x, w_router, gate, up, down, top_k, shared, ids):
    tokens, hidden = x.shape
    experts = w_router.shape[1]
    scores = torch.sigmoid((x @ w_router).float())
    top = torch.gather(scores, 1, ids)
    weights = (top / (top.sum(-1, keepdim=True) + 1e-20)).to(x.dtype)
    flat = ids.reshape(-1)
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=experts).tolist()
    packed = x[order // top_k]
    outs, start = [], 0
    for e, n in enumerate(counts):
        if n:
            rows = packed[start:start + n]
            outs.append((torch.nn.functional.silu(rows @ gate[e]) * (rows @ up[e])) @ down[e])
        start += n
    out = torch.cat(outs)
    inverse = torch.empty_like(order)
    inverse[order] = torch.arange(order.numel(), device=order.device)
    y = (out[inverse].reshape(tokens, top_k, hidden) * weights[..., None]).float().sum(1).to(x.dtype)
    if shared is not None:
        y = y + (torch.nn.functional.silu(x @ shared[0]) * (x @ shared[1])) @ shared[2]
    return y


@pytest.mark.parametrize(
    "tokens,hidden,experts,top_k,inter,shared_experts,skew",
    [(4096, 2048, 64, 8, 1408, 2, 0.0),    # the headline shape at a quarter of its tokens
     (6000, 1024, 128, 8, 768, 0, 2.0),    # many groups of very unequal sizes, some empty
     (5811, 512, 128, 2, 384, 1, 2.0),
     (3000, 2048, 16, 2, 704, 0, 0.5),
     (6933, 256, 16, 8, 768, 1, 0.5),      # an expert that every token selects
     (2500, 1024, 40, 4, 192, 0, 2.0),
     (7000, 512, 96, 6, 1408, 0, 0.0)],
)
def test_layer_and_gradients_agree_with_torch(gpu, tokens, hidden, experts, top_k, inter, shared_experts, skew):
    gen = torch.Generator(device=gpu)
    gen.manual_seed(tokens + experts)

    def draw(*shape, std=1.0):
        return (torch.randn(*shape, device=gpu, generator=gen) * std).to(torch.bfloat16)

    x, w_router = draw(tokens, hidden), draw(hidden, experts, std=0.05)
    gate, up = draw(experts, hidden, inter, std=0.03), draw(experts, hidden, inter, std=0.03)
    down = draw(experts, inter, hidden, std=0.03)
    bias = (-skew * torch.log(torch.arange(1, experts + 1, device=gpu).float())).contiguous()
    if experts > top_k + 3:
        bias[experts - 3:] = -50.0  # never selected: empty groups
    shared = None
    if shared_experts:
        width = inter * shared_experts
        shared = (draw(hidden, width, std=0.03), draw(hidden, width, std=0.03), draw(width, hidden, std=0.03))
    leaves = [x, w_router, gate, up, down] + (list(shared) if shared else [])
    for leaf in leaves:
        leaf.requires_grad_(True)
    dy = draw(tokens, hidden)

    y, _, ids = A.moe_layer(x, w_router, bias, gate, up, down, top_k, 1.0, shared=shared)
    y.backward(dy)
    got = [leaf.grad.clone() for leaf in leaves]
    for leaf in leaves:
        leaf.grad = None
    want_y = torch_layer_with_ids(x, w_router, gate, up, down, top_k, shared, ids.long())
    want_y.backward(dy)
    want = [leaf.grad for leaf in leaves]

    def rel(a, b):
        a, b = a.detach().float(), b.detach().float()
        scale = float(b.abs().max())
        return float((a - b).abs().max()) / (scale if scale > 0 else 1.0)

    names = ["x", "w_router", "gate", "up", "down", "shared_gate", "shared_up", "shared_down"]
    assert rel(y, want_y) <= 2e-2, f"y: {rel(y, want_y):.3e}"
    for name, a, b in zip(names, got, want):
        assert bool(torch.isfinite(a.float()).all()), name
        assert rel(a, b) <= 2e-2, f"d {name}: {rel(a, b):.3e}"
    sizes = torch.bincount(ids.reshape(-1).long(), minlength=experts)
    if skew >= 2.0:
        # the groups really are unequal, and some are empty
        assert int(sizes.max()) > 4 * int(sizes[sizes > 0].min()) and int((sizes == 0).sum()) >= 3
