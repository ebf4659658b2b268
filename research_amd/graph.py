"""Replay of the layer from a captured HIP graph, for callers whose per-call host cost matters.

At 64 tokens the kernels of one layer call take about 0.19 ms.  The library's own host side adds
about 0.05 ms per call, hidden behind the GPU when calls are issued back to back; a caller with a
heavier host side (more Python between calls, a blocking wait after each) can capture the call
once and replay the same kernels with a single launch.  The reference gets the equivalent from
``jax.jit`` (its decode step, blocks.py:262-290, runs inside one compiled program).

The library's forward path only enqueues kernels (no allocation, no memset, no synchronisation),
so it can be captured as it is.  Shapes are fixed at capture; the caller copies new inputs into
``x`` (and may update the parameters in place) and calls ``replay()``.
"""

from __future__ import annotations

import torch

from research_amd import ops
from research_amd.errors import ContractError


class GraphedLayer:
    """ops.moe_forward captured for one input shape.  Outputs are overwritten by every replay."""

    def __init__(self, x, w_router, expert_bias, gate, up, down, top_k, route_scale=1.0, shared=None):
        if not x.is_cuda:
            raise ContractError("x must live on the GPU; there is no CPU path")
        self.x = x.clone()
        self._args = (w_router, expert_bias, gate, up, down, top_k, route_scale)
        self._shared = shared
        dev = x.device
        lib_bytes = ops._lib().jtmoe_workspace_bytes(
            x.shape[0], x.shape[1], w_router.shape[1], top_k, gate.shape[2], 0 if shared is None else shared[0].shape[1],
            ops._code(x.dtype))
        # a workspace of its own: the one ops caches per stream may be replaced while the graph lives
        self._workspace = torch.empty((max(int(lib_bytes), 256),), dtype=torch.uint8, device=dev)
        stream = torch.cuda.Stream(device=dev)
        stream.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(stream):
            for _ in range(2):  # first calls set kernel attributes and warm the allocator
                self._call()
        torch.cuda.current_stream(dev).wait_stream(stream)
        torch.cuda.synchronize(dev)
        self._graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self._graph):
            self.result = self._call()

    def _call(self) -> ops.LayerResult:
        w_router, expert_bias, gate, up, down, top_k, route_scale = self._args
        return ops.moe_forward(self.x, w_router, expert_bias, gate, up, down, top_k, route_scale,
                               shared=self._shared, workspace=self._workspace)

    def replay(self, x: torch.Tensor | None = None) -> ops.LayerResult:
        """Copy ``x`` (same shape and dtype as at capture) into the graph's input and run it."""
        if x is not None:
            if x.shape != self.x.shape or x.dtype != self.x.dtype:
                raise ContractError(f"input must have shape {list(self.x.shape)} and dtype {self.x.dtype}")
            self.x.copy_(x)
        self._graph.replay()
        return self.result
