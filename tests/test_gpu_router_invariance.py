"""A token's routing does not depend on the batch it is routed in.

The reference's invariant is prefill + decode == full forward (tests/jaxtitan/test_infer.py:270-301):
the layer is a per-token function, so the rows of a 64-token decode call must come out as they do
inside a prefill of thousands.  The router has several projection kernels (one workgroup walking the
whole hidden dimension for large batches; the hidden dimension shared out over workgroups, with and
without a finishing workgroup, for small ones); all of them add a logit up in one order, so logits,
scores, ids and weights of a row are equal bit for bit whatever the size of the call.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

from research_amd import ops
from test_gpu_parity import dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize(
    "hidden,experts,top_k",
    [(2048, 64, 8), (2048, 128, 8), (1024, 16, 2), (512, 256, 4), (128, 32, 2), (2176, 32, 2),
     (1920, 64, 6),  # 15 chunks of 128 rows: slices of two chunks, the last of one
     (192, 64, 4),   # not a multiple of 128: one kernel (and one slice) for every batch size
     (72, 24, 3)],   # no matrix-core path at all
)
@pytest.mark.parametrize("score_func", ["sigmoid", "softmax"])
def test_router_rows_do_not_depend_on_the_batch(gpu, hidden, experts, top_k, score_func):
    rng = np.random.default_rng(hidden * 7 + experts)
    tokens = 1500
    x = dev(rng.standard_normal((tokens, hidden)).astype(np.float32), gpu, "bf16")
    w = dev((rng.standard_normal((hidden, experts)) * 0.02).astype(np.float32), gpu, "bf16")
    bias = dev((rng.standard_normal(experts) * 0.05).astype(np.float32), gpu)
    full = ops.router(x, w, bias, top_k, 1.0, return_logits=True, score_func=score_func)
    for start, count in ((0, 1), (3, 16), (100, 17), (7, 64), (500, 200), (1000, 256), (900, 257), (64, 1000)):
        part = ops.router(x[start:start + count].contiguous(), w, bias, top_k, 1.0, return_logits=True,
                          score_func=score_func)
        for name in ("logits", "scores", "expert_ids", "weights"):
            a, b = getattr(part, name), getattr(full, name)[start:start + count]
            assert torch.equal(a, b), (f"H={hidden} E={experts} {score_func}: {name} of rows {start}..{start + count - 1} "
                                       f"differ from the {tokens}-token call in {int((a != b).any(dim=1).sum())} rows")


def test_decode_batch_routes_like_the_same_rows_of_a_prefill(gpu):
    """The layer call at the decode shape (64 tokens: router partial sums + finishing workgroup that also
    plans the dispatch) against the same rows inside a 4096-token call (64-token workgroups)."""
    rng = np.random.default_rng(5)
    T, H, E, K, I = 4096, 2048, 64, 8, 128
    x = dev(rng.standard_normal((T, H)).astype(np.float32), gpu, "bf16")
    w = dev((rng.standard_normal((H, E)) * 0.02).astype(np.float32), gpu, "bf16")
    gate, up = (dev((rng.standard_normal((E, H, I)) * 0.02).astype(np.float32), gpu, "bf16") for _ in range(2))
    down = dev((rng.standard_normal((E, I, H)) * 0.02).astype(np.float32), gpu, "bf16")
    full = ops.moe_forward(x, w, None, gate, up, down, K, 1.0)
    for start in (0, 1000, 4032):
        part = ops.moe_forward(x[start:start + 64].contiguous(), w, None, gate, up, down, K, 1.0)
        for name in ("scores", "expert_ids", "weights"):
            assert torch.equal(getattr(part, name), getattr(full, name)[start:start + 64]), name
