"""The layer as a differentiable torch operation: forward through jtmoe_moe_forward_train, backward
through jtmoe_moe_backward.

This is the torch-side analogue of the custom VJP the reference asks of a forward-only kernel before
it may replace a training component (docs/kernel_backend_design.md:120-128): the forward keeps the
residuals, the backward consumes the cotangents of the two differentiable outputs (the layer output
and the router scores, which the sequence-balance loss reads, moe.py:828-840).  The expert bias
only enters the selection and receives no gradient (moe.py:139-140).
"""

from __future__ import annotations

import torch

from research_amd import grad, ops


class MoeLayerFunction(torch.autograd.Function):
    """(x, w_router, gate, up, down, shared_gate, shared_up, shared_down) -> (y, scores, expert_ids)."""

    @staticmethod
    def forward(ctx, x, w_router, gate, up, down, shared_gate, shared_up, shared_down, expert_bias, top_k,
                route_scale, score_func="sigmoid"):
        shared = None if shared_gate is None else (shared_gate, shared_up, shared_down)
        result, residuals = grad.moe_forward_train(x, w_router, expert_bias, gate, up, down, top_k, route_scale,
                                                   shared=shared, score_func=score_func)
        ctx.route_scale = route_scale
        ctx.score_func = score_func
        ctx.has_shared = shared is not None
        # Everything the backward pass reads goes through save_for_backward (which knows how to hold an
        # output such as the scores without a reference cycle); y itself is not needed again.
        shared_res = residuals.shared
        ctx.save_for_backward(x, w_router, gate, up, down, *(shared or ()),
                              result.expert_ids, result.weights, result.scores, result.group_sizes, result.offsets,
                              result.source_order, result.inverse, residuals.routed.gate_pre, residuals.routed.up_pre,
                              *((shared_res.gate_pre, shared_res.up_pre) if shared_res is not None else ()))
        ctx.mark_non_differentiable(result.expert_ids)
        return result.y, result.scores, result.expert_ids

    @staticmethod
    def backward(ctx, dy, d_scores, _d_ids):
        saved = list(ctx.saved_tensors)
        x, w_router, gate, up, down = saved[:5]
        rest = saved[5:]
        shared = None
        if ctx.has_shared:
            shared, rest = tuple(rest[:3]), rest[3:]
        ids, weights, scores, group_sizes, offsets, source_order, inverse, gate_pre, up_pre = rest[:9]
        shared_res = grad.ExpertResiduals(rest[9], rest[10]) if ctx.has_shared else None
        result = ops.LayerResult(None, ids, weights, scores, None, None, group_sizes, offsets, source_order, inverse)
        residuals = grad.LayerResiduals(grad.ExpertResiduals(gate_pre, up_pre), shared_res)
        if dy is None:
            dy = torch.zeros_like(x)
        g = grad.moe_backward(x, dy.contiguous(), None if d_scores is None else d_scores.contiguous(), w_router, gate,
                              up, down, shared, result, residuals, ctx.route_scale, score_func=ctx.score_func)
        ds = g.d_shared if g.d_shared is not None else (None, None, None)
        return g.dx, g.d_w_router, g.d_gate, g.d_up, g.d_down, ds[0], ds[1], ds[2], None, None, None, None


def moe_layer(x, w_router, expert_bias, gate, up, down, top_k, route_scale=1.0, shared=None, score_func="sigmoid"):
    """Differentiable layer on x [T,H]: returns (y [T,H], scores [T,E] float32, expert_ids [T,K] int32)."""
    sg, su, sd = shared if shared is not None else (None, None, None)
    return MoeLayerFunction.apply(x, w_router, gate, up, down, sg, su, sd, expert_bias, top_k, float(route_scale),
                                  score_func)


class SequenceBalanceLossFunction(torch.autograd.Function):
    """scores [B,S,E] (with expert_ids [B,S,K]) -> the sequence balance loss (moe.py:828-840), differentiable
    in the scores; the counts derived from the ids are constants."""

    @staticmethod
    def forward(ctx, scores, expert_ids, top_k):
        ctx.top_k = top_k
        ctx.save_for_backward(scores, expert_ids)
        return ops.sequence_balance_loss(expert_ids, scores, top_k=top_k)

    @staticmethod
    def backward(ctx, d_loss):
        scores, expert_ids = ctx.saved_tensors
        d_scores = ops.sequence_balance_loss_backward(expert_ids, scores, top_k=ctx.top_k,
                                                      d_loss=d_loss.to(torch.float32).reshape(1).contiguous())
        return d_scores, None, None


def sequence_balance_loss(expert_ids, scores, top_k):
    """The auxiliary loss as a differentiable function of the router scores [B,S,E]."""
    return SequenceBalanceLossFunction.apply(scores.contiguous(), expert_ids.contiguous(), int(top_k))
