"""jtmoe_dispatch_static, the entry point that allocates nothing (its scratch is a buffer inside
the library's device image), against jtmoe_dispatch with a caller's workspace: identical plans and
packed rows, bit for bit, on two calls in a row that share the buffer, the second one smaller."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from research_amd import _ffi

STATIC_MAX_BYTES = 1 << 20  # JTMOE_DISPATCH_STATIC_MAX_BYTES


def _buffers(tokens, top_k, experts, hidden, dev):
    n = tokens * top_k
    return dict(
        group_sizes=torch.full((experts,), -7, dtype=torch.int32, device=dev),
        offsets=torch.full((experts,), -7, dtype=torch.int32, device=dev),
        source_order=torch.full((n,), -7, dtype=torch.int32, device=dev),
        inverse=torch.full((n,), -7, dtype=torch.int32, device=dev),
        packed_x=torch.zeros((n, hidden), dtype=torch.bfloat16, device=dev),
    )


def _run_pair(lib, seed, tokens, top_k, experts, hidden, dev):
    rng = np.random.default_rng(seed)
    ids_np = rng.integers(0, experts, size=(tokens, top_k), dtype=np.int32)
    ids_np[rng.random((tokens, top_k)) < 0.3] = experts // 2  # one crowded expert, others uneven
    ids = torch.from_numpy(ids_np).to(dev)
    x = torch.from_numpy(rng.standard_normal((tokens, hidden)).astype(np.float32)).to(dev).to(torch.bfloat16)
    stream = torch.cuda.current_stream(dev).cuda_stream
    ws_bytes = lib.jtmoe_dispatch_workspace_bytes(tokens * top_k, experts)
    assert 0 < ws_bytes <= STATIC_MAX_BYTES
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
    want = _buffers(tokens, top_k, experts, hidden, dev)
    got = _buffers(tokens, top_k, experts, hidden, dev)
    rc = lib.jtmoe_dispatch(ids.data_ptr(), x.data_ptr(), tokens, hidden, experts, top_k, _ffi.JTMOE_BF16,
                            want["group_sizes"].data_ptr(), want["offsets"].data_ptr(),
                            want["source_order"].data_ptr(), want["inverse"].data_ptr(),
                            want["packed_x"].data_ptr(), ws.data_ptr(), ws.numel(), stream)
    assert rc == 0, _ffi.last_error(lib)
    rc = lib.jtmoe_dispatch_static(ids.data_ptr(), x.data_ptr(), tokens, hidden, experts, top_k, _ffi.JTMOE_BF16,
                                   got["group_sizes"].data_ptr(), got["offsets"].data_ptr(),
                                   got["source_order"].data_ptr(), got["inverse"].data_ptr(),
                                   got["packed_x"].data_ptr(), stream)
    assert rc == 0, _ffi.last_error(lib)
    torch.cuda.synchronize(dev)
    for name in want:
        assert torch.equal(got[name], want[name]), f"{name} differs (tokens={tokens} experts={experts})"
    sizes = want["group_sizes"].cpu().numpy()
    assert np.array_equal(sizes, np.bincount(ids_np.reshape(-1), minlength=experts))


@pytest.mark.gpu
def test_dispatch_static_matches_dispatch_on_two_calls_the_second_smaller(gpu):
    lib = _ffi.load_library()
    # both sizes are above the single-workgroup path (8192 assignments), so both use the scratch
    _run_pair(lib, 0, tokens=32768, top_k=8, experts=64, hidden=256, dev=gpu)
    _run_pair(lib, 1, tokens=5000, top_k=4, experts=17, hidden=128, dev=gpu)


@pytest.mark.gpu
def test_dispatch_static_small_batches_and_empty_input(gpu):
    lib = _ffi.load_library()
    _run_pair(lib, 2, tokens=64, top_k=8, experts=64, hidden=128, dev=gpu)  # single-workgroup path
    experts = 8
    sizes = torch.full((experts,), -1, dtype=torch.int32, device=gpu)
    offsets = torch.full((experts,), -1, dtype=torch.int32, device=gpu)
    rc = lib.jtmoe_dispatch_static(None, None, 0, 0, experts, 2, _ffi.JTMOE_BF16, sizes.data_ptr(),
                                   offsets.data_ptr(), None, None, None,
                                   torch.cuda.current_stream(gpu).cuda_stream)
    assert rc == 0, _ffi.last_error(lib)
    torch.cuda.synchronize(gpu)
    assert sizes.eq(0).all() and offsets.eq(0).all()


def test_dispatch_static_rejects_sizes_beyond_its_buffer():
    lib = _ffi.load_library()
    # validation precedes every HIP call: 2^21 assignments over 256 experts need 2 MiB of histograms
    rc = lib.jtmoe_dispatch_static(1, None, 1 << 18, 0, 256, 8, _ffi.JTMOE_BF16, 1, 1, 1, 1, None, None)
    assert rc == -2 and "built-in" in _ffi.last_error(lib)
    rc = lib.jtmoe_dispatch_static(1, None, 16, 0, 300, 8, _ffi.JTMOE_BF16, 1, 1, 1, 1, None, None)
    assert rc == -2 and "exceeds" in _ffi.last_error(lib)
    rc = lib.jtmoe_dispatch_static(None, None, 16, 0, 8, 2, _ffi.JTMOE_BF16, 1, 1, 1, 1, None, None)
    assert rc == -1 and "null" in _ffi.last_error(lib)
