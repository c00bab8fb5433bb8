"""
Top-k routing on the HIP kernel path: the k largest router logits of every token, their experts, and the fp32
softmax over just those logits; differentiable with respect to the logits.

Reference: `MixtureOfExpertMLP._topk_routing` (fast_llm/layers/decoder/mlp/mixture_of_experts.py:243-244), which
does this with `torch.topk` and `torch.softmax(dtype=torch.float32)` and lets autograd derive the backward.
"""

import dataclasses

import torch

from fast_llm_amd import _lib


@dataclasses.dataclass
class RouterCounts:
    """What the router's forward kernel counted on its way (per workgroup and routed expert, the tokens that selected
    the expert), kept so that `get_sparse_map(..., router_counts=...)` need not count `top_experts` again."""

    workspace: torch.Tensor  # as filled by fm_router_forward; opaque
    tokens: int
    routed_experts: int
    experts_per_token: int
    shared_experts: int
    # Identity of the `top_experts` tensor the counts belong to (its storage address and in-place version counter):
    # counts of other, or since edited, selections would give overlapping expert ranges.
    top_experts_address: int = 0
    top_experts_version: int = -1

    def describes(self, top_experts: torch.Tensor) -> bool:
        """Whether `top_experts` is the very tensor these counts were taken from, unmodified since."""
        return top_experts.data_ptr() == self.top_experts_address and top_experts._version == self.top_experts_version


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


def router_forward(
    logits: torch.Tensor, noise: torch.Tensor | None, experts_per_token: int, shared_experts: int
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, RouterCounts]:
    """One pass over `logits` [tokens, routed experts]: (scores fp32, top_experts int64, both
    [tokens, shared_experts + k]; losses [2] fp32 = load-balancing loss, z-loss; lse [tokens, 2] and statistics
    [2 * experts + 1], both kept for the backward; and the per-workgroup counts for the sparse map)."""
    assert logits.dim() == 2 and logits.is_contiguous()
    assert noise is None or (noise.shape == logits.shape and noise.dtype == logits.dtype and noise.is_contiguous())
    device = _lib.require_device(logits, noise)
    tokens, experts = logits.shape
    if not 0 < experts_per_token <= experts:
        raise ValueError(f"experts_per_token={experts_per_token} with {experts} experts")
    if tokens == 0:
        raise ValueError("no tokens to route")
    slots = shared_experts + experts_per_token
    new = lambda shape, dtype: torch.empty(shape, dtype=dtype, device=logits.device)  # noqa: E731
    scores, top_experts = new((tokens, slots), torch.float32), new((tokens, slots), torch.int64)
    lse, statistics, losses = new((tokens, 2), torch.float32), new(2 * experts + 1, torch.float32), new(2, torch.float32)
    workspace_size = _lib.lib().fm_router_workspace_size(tokens, experts)
    workspace = new(workspace_size, torch.uint8)
    _lib.call(
        "fm_router_forward",
        device,
        _lib.ptr(logits),
        _lib.ptr(noise),
        _lib.ptr(top_experts),
        _lib.ptr(scores),
        _lib.ptr(lse),
        _lib.ptr(statistics),
        _lib.ptr(losses),
        _lib.ptr(workspace),
        workspace_size,
        tokens,
        experts,
        experts_per_token,
        shared_experts,
        _lib.dtype_tag(logits.dtype),
    )
    counts = RouterCounts(
        workspace, tokens, experts, experts_per_token, shared_experts, top_experts.data_ptr(), top_experts._version
    )
    return scores, top_experts, losses, lse, statistics, counts


class _Router(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, noise, experts_per_token, shared_experts, auxiliary_loss_grad, z_loss_grad):
        logits = logits.detach().contiguous()
        noise = None if noise is None else noise.detach().contiguous()
        scores, top_experts, losses, lse, statistics, counts = router_forward(
            logits, noise, experts_per_token, shared_experts
        )
        ctx.save_for_backward(logits, noise, scores, top_experts, lse, statistics)
        ctx.shape = (experts_per_token, shared_experts)
        ctx.loss_grads = (auxiliary_loss_grad or 0.0, z_loss_grad or 0.0)
        ctx.mark_non_differentiable(top_experts, losses, counts.workspace)
        return scores, top_experts, losses, counts.workspace

    @staticmethod
    def backward(ctx, grad_scores, _, __, ___):
        logits, noise, scores, top_experts, lse, statistics = ctx.saved_tensors
        experts_per_token, shared_experts = ctx.shape
        device = _lib.require_device(logits)
        grad_logits = torch.empty_like(logits)
        _lib.call(
            "fm_router_backward",
            device,
            _lib.ptr(grad_scores.to(torch.float32).contiguous()),
            _lib.ptr(scores),
            _lib.ptr(top_experts),
            _lib.ptr(logits),
            _lib.ptr(noise),
            _lib.ptr(lse),
            _lib.ptr(statistics),
            _lib.ptr(grad_logits),
            float(ctx.loss_grads[0]),
            float(ctx.loss_grads[1]),
            logits.size(0),
            logits.size(1),
            experts_per_token,
            shared_experts,
            _lib.dtype_tag(logits.dtype),
        )
        return grad_logits, None, None, None, None, None


def router(
    logits: torch.Tensor,
    experts_per_token: int,
    *,
    shared_experts: int = 0,
    noise: torch.Tensor | None = None,
    auxiliary_loss_grad: float | None = None,
    z_loss_grad: float | None = None,
    return_counts: bool = False,
) -> tuple[torch.Tensor, ...]:
    """
    The router front end of `MixtureOfExpertMLP._forward` for top-k routing (reference:
    fast_llm/layers/decoder/mlp/mixture_of_experts.py:146-171, 237-278) in one pass over `logits` [..., routed experts]:
    z-loss, jitter (`noise`, the multiplier the caller drew), top-k + fp32 softmax, load-balancing loss, shared experts.
    Returns (scores [..., shared + k] fp32, top_experts int64, load_balancing_loss, z_loss); the two losses are
    detached scalars. `auxiliary_loss_grad` / `z_loss_grad` are the constant gradients the reference's `AuxiliaryLoss`
    (functional/utils.py:63-71) gives the losses when the scores are back-propagated:
    `unshared_experts * auxiliary_loss_coefficient * grad_scale` and `z_loss_coefficient * grad_scale`; None or 0:
    that loss contributes no gradient. With `return_counts` a fifth value follows: the `RouterCounts` to hand to
    `get_sparse_map` together with these `top_experts`.
    """
    flat = logits.flatten(0, -2)
    flat_noise = None if noise is None else noise.flatten(0, -2)
    scores, top_experts, losses, workspace = _Router.apply(
        flat, flat_noise, experts_per_token, shared_experts, auxiliary_loss_grad, z_loss_grad
    )
    shape = logits.shape[:-1] + (shared_experts + experts_per_token,)
    result = (scores.view(shape), top_experts.view(shape), losses[0], losses[1])
    if return_counts:
        result += (
            RouterCounts(
                workspace, flat.size(0), flat.size(1), experts_per_token, shared_experts,
                top_experts.data_ptr(), top_experts._version,
            ),
        )  # fmt: skip
    return result


def sinkhorn(cost: torch.Tensor, tolerance: float = 1e-5, eps: float = 1e-9) -> torch.Tensor:
    """Sinkhorn normalisation of exp(cost): alternately rescales rows and columns until the column scales move by less
    than `tolerance` on average; rows of the result sum to 1 / tokens, columns to about 1 / experts. No gradient.
    Reference: fast_llm/layers/decoder/mlp/mixture_of_experts.py:389-403 (a data-dependent number of small torch
    reductions over [tokens, experts]; it is upstream of the dropless path and stays in torch)."""
    with torch.no_grad():
        cost = torch.exp(cost.to(torch.float32))
        d0 = torch.ones(cost.shape[:-1], device=cost.device, dtype=cost.dtype)
        d1 = torch.ones(cost.shape[-1:], device=cost.device, dtype=cost.dtype)
        error = eps**-1
        d1_old = d1
        while error > tolerance:
            d0 = d0.numel() ** -1 / (torch.sum(d1 * cost, -1) + eps)
            d1 = d1.numel() ** -1 / (torch.sum((d0.unsqueeze(-1) * cost).flatten(0, -2), 0) + eps)
            error = torch.mean(torch.abs(d1_old - d1))
            d1_old = d1
        return d1 * cost * d0.unsqueeze(-1)


def sinkhorn_routing(logits: torch.Tensor, experts_per_token: int, training: bool) -> tuple[torch.Tensor, torch.Tensor]:
    """(scores, top_experts) of the reference's sinkhorn routing (mixture_of_experts.py:280-296): when training, the
    experts are the top-k of the sinkhorn-balanced logits and the scores are the activated logits gathered there;
    otherwise top-k of the activated logits. The activation is a sigmoid for one expert per token, else an fp32
    softmax cast back to the logits' dtype."""

    def activation(x: torch.Tensor) -> torch.Tensor:
        if experts_per_token == 1:
            return torch.sigmoid(x)
        return torch.softmax(x, dim=-1, dtype=torch.float32).type_as(x)

    if training:
        _, top_experts = torch.topk(sinkhorn(logits), k=experts_per_token, dim=-1)
        scores = torch.gather(activation(logits), -1, top_experts)
    else:
        scores, top_experts = torch.topk(activation(logits), k=experts_per_token, dim=-1)
    return scores, top_experts
