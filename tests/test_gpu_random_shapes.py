"""Randomised shapes for the four forward operators, against the same oracle checks as test_gpu_parity.

The parametrised cases there pick the shapes the configurations use and the edges of each code path;
this file draws odd ones (expert counts that are not powers of two, rows that are not multiples of
the vector width, single tokens, top_k = num_experts, skewed routings) from a fixed seed.
"""

from __future__ import annotations

import numpy as np
import pytest

import test_gpu_parity as P  # the tests directory is on sys.path under pytest (no package)

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_router_shapes(gpu, seed):
    rng = np.random.default_rng(seed)
    for _ in range(24):
        tokens = int(rng.choice([1, 2, 15, 16, 17, 63, 64, 65, 100, 255, 256, 257, 300, 700]))
        experts = int(rng.choice([1, 3, 8, 16, 24, 32, 64, 100, 128, 256]))
        top_k = int(rng.integers(1, min(experts, 8) + 1))
        dtype = "bf16" if rng.random() < 0.75 else "f32"
        # fp32 sums of thousands of terms differ from NumPy's by more than the 1-ulp bar of the check
        hidden = int(rng.choice([8, 72, 128, 256, 384, 512] if dtype == "f32" else [8, 72, 128, 256, 512, 1024, 2048, 2176]))
        x = rng.standard_normal((tokens, hidden)).astype(np.float32)
        w = (rng.standard_normal((hidden, experts)) * 0.02).astype(np.float32)
        bias = (rng.standard_normal(experts) * 0.05).astype(np.float32) if rng.random() < 0.5 else None
        print(f"router {dtype} T={tokens} H={hidden} E={experts} K={top_k}", flush=True)
        P.check_router_end_to_end(gpu, x, w, bias, top_k, float(rng.choice([1.0, 2.5])), dtype)


@pytest.mark.parametrize("seed", [21, 22, 23, 24])
def test_random_dispatch_shapes(gpu, seed):
    rng = np.random.default_rng(seed)
    for _ in range(24):
        tokens = int(rng.choice([1, 3, 64, 127, 128, 129, 500, 1023, 1024, 1025, 2047, 4096, 9000]))
        top_k = int(rng.choice([1, 2, 3, 8]))
        experts = int(rng.choice([1, 2, 5, 8, 16, 63, 64, 128, 255, 256]))
        hidden = int(rng.choice([1, 7, 8, 40, 256]))
        dtype = "bf16" if rng.random() < 0.6 else "f32"
        skew = rng.random() < 0.4
        ids = (np.minimum(rng.zipf(1.3, size=(tokens, top_k)) - 1, experts - 1) if skew
               else rng.integers(0, experts, size=(tokens, top_k))).astype(np.int32)
        x = rng.standard_normal((tokens, hidden)).astype(np.float32)
        print(f"dispatch T={tokens} K={top_k} E={experts} H={hidden} {dtype} skew={skew}", flush=True)
        P.check_dispatch(gpu, ids, experts, x, dtype)


@pytest.mark.parametrize("seed", [31, 32, 33, 34])
def test_random_expert_and_combine_shapes(gpu, seed):
    rng = np.random.default_rng(seed)
    for _ in range(16):
        dtype = "bf16" if rng.random() < 0.8 else "f32"
        tokens = int(rng.choice([1, 5, 40, 64, 130, 300, 600]))
        hidden = int(rng.choice([8, 24, 64, 128, 200, 512, 1024]))
        experts = int(rng.choice([1, 2, 5, 8, 16, 64]))
        top_k = int(rng.integers(1, min(experts, 4) + 1))
        inter = int(rng.choice([8, 40, 64, 136, 256, 704]))
        print(f"grouped_swiglu {dtype} T={tokens} H={hidden} E={experts} K={top_k} I={inter}", flush=True)
        P.test_grouped_swiglu_matches_oracle(gpu, tokens, hidden, experts, top_k, inter, dtype)
    for _ in range(16):
        dtype = "bf16" if rng.random() < 0.7 else "f32"
        tokens = int(rng.choice([1, 4, 5, 63, 130, 1000]))
        hidden = int(rng.choice([3, 8, 64, 72, 512, 2048, 4096, 4104]))
        top_k = int(rng.choice([1, 2, 3, 8]))
        print(f"combine {dtype} T={tokens} H={hidden} K={top_k}", flush=True)
        P.test_combine_is_bit_exact(gpu, tokens, hidden, top_k, dtype, bool(rng.random() < 0.5))


@pytest.mark.parametrize("seed", [41, 42, 43, 44, 1001, 1007, 1012, 1014])
def test_random_gradient_shapes(gpu, seed):
    """The backward operators on odd shapes: rows that leave the fast GEMM paths, single tokens,
    one expert, top_k = num_experts."""
    import test_gpu_grad as G

    rng = np.random.default_rng(seed)
    for _ in range(10):
        tokens = int(rng.choice([1, 5, 40, 130, 300]))
        hidden = int(rng.choice([8, 24, 64, 200, 512]))
        experts = int(rng.choice([1, 2, 5, 8, 16]))
        top_k = int(rng.integers(1, min(experts, 4) + 1))
        inter = int(rng.choice([8, 40, 64, 136, 256]))
        dtype = "f32" if hidden <= 64 and inter <= 64 and rng.random() < 0.5 else "bf16"
        print(f"expert gradients {dtype} T={tokens} H={hidden} E={experts} K={top_k} I={inter}", flush=True)
        G.test_expert_gradients_match_oracle(gpu, tokens, hidden, experts, top_k, inter, dtype)
    for _ in range(6):
        tokens, hidden, inter = int(rng.choice([1, 7, 64, 300])), int(rng.choice([8, 72, 256, 1024])), int(rng.choice([8, 40, 704]))
        # fp32 only where the sums are short: the element-wise fp32 bar of that check is tighter than the
        # difference between two summation orders over hundreds of terms
        dtype = "f32" if hidden <= 72 and inter <= 40 and rng.random() < 0.5 else "bf16"
        print(f"shared gradients {dtype} T={tokens} H={hidden} I={inter}", flush=True)
        G.test_shared_gradients_match_oracle(gpu, tokens, hidden, inter, dtype)
    for _ in range(8):
        dtype = "bf16" if rng.random() < 0.7 else "f32"
        tokens, hidden = int(rng.choice([1, 9, 64, 257, 600])), int(rng.choice([8, 72, 256, 1024]))
        experts = int(rng.choice([1, 3, 8, 24, 64, 256]))
        top_k = int(rng.integers(1, min(experts, 8) + 1))
        print(f"router gradients {dtype} T={tokens} H={hidden} E={experts} K={top_k}", flush=True)
        G.test_router_gradients_match_oracle(gpu, tokens, hidden, experts, top_k, dtype, bool(rng.random() < 0.5))
