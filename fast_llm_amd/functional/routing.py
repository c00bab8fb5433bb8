"""
Top-k routing on the HIP kernel path: the k largest router logits of every token, their experts, and the fp32
softmax over just those logits; differentiable with respect to the logits.

Reference: `MixtureOfExpertMLP._topk_routing` (fast_llm/layers/decoder/mlp/mixture_of_experts.py:243-244), which
does this with `torch.topk` and `torch.softmax(dtype=torch.float32)` and lets autograd derive the backward.
"""

import torch

from fast_llm_amd import _lib


def topk_routing_forward(logits: torch.Tensor, experts_per_token: int) -> tuple[torch.Tensor, torch.Tensor]:
    """(scores [tokens, k] fp32, top_experts [tokens, k] int64), experts in descending order of their logits."""
    assert logits.dim() == 2 and logits.is_contiguous()
    device = _lib.require_device(logits)
    tokens, experts = logits.shape
    if not 0 < experts_per_token <= experts:
        raise ValueError(f"experts_per_token={experts_per_token} with {experts} experts")
    scores = torch.empty((tokens, experts_per_token), dtype=torch.float32, device=logits.device)
    top_experts = torch.empty((tokens, experts_per_token), dtype=torch.int64, device=logits.device)
    _lib.call(
        "fm_topk_routing",
        device,
        _lib.ptr(logits.detach()),
        _lib.ptr(top_experts),
        _lib.ptr(scores),
        tokens,
        experts,
        experts_per_token,
        _lib.dtype_tag(logits.dtype),
    )
    return scores, top_experts


def topk_routing_backward(
    grad_scores: torch.Tensor, scores: torch.Tensor, top_experts: torch.Tensor, num_experts: int, dtype: torch.dtype
) -> torch.Tensor:
    """Gradient of the logits (`dtype`, [tokens, num_experts]) given the gradient of the scores."""
    device = _lib.require_device(scores)
    tokens, experts_per_token = scores.shape
    grad_logits = torch.empty((tokens, num_experts), dtype=dtype, device=scores.device)
    _lib.call(
        "fm_topk_routing_backward",
        device,
        _lib.ptr(grad_scores.to(torch.float32).contiguous()),
        _lib.ptr(scores),
        _lib.ptr(top_experts),
        _lib.ptr(grad_logits),
        tokens,
        num_experts,
        experts_per_token,
        _lib.dtype_tag(dtype),
    )
    return grad_logits


class _TopKRouting(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits: torch.Tensor, experts_per_token: int):
        scores, top_experts = topk_routing_forward(logits.contiguous(), experts_per_token)
        ctx.save_for_backward(scores, top_experts)
        ctx.num_experts, ctx.dtype = logits.size(-1), logits.dtype
        ctx.mark_non_differentiable(top_experts)
        return scores, top_experts

    @staticmethod
    def backward(ctx, grad_scores: torch.Tensor, _):
        scores, top_experts = ctx.saved_tensors
        return topk_routing_backward(grad_scores, scores, top_experts, ctx.num_experts, ctx.dtype), None


def topk_routing(logits: torch.Tensor, experts_per_token: int) -> tuple[torch.Tensor, torch.Tensor]:
    """`logits` [..., experts] -> (scores [..., k] fp32, top_experts [..., k] int64)."""
    flat = logits.flatten(0, -2)
    scores, top_experts = _TopKRouting.apply(flat, experts_per_token)
    shape = logits.shape[:-1] + (experts_per_token,)
    return scores.view(shape), top_experts.view(shape)
