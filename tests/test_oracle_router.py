"""Pins the oracle's restatement of the router front end (oracle.moe_oracle.router) with formulations that do not
share its code: closed forms, a pure-Python double loop, and finite differences of the trained objective."""

import math

import pytest
import torch

from oracle import moe_oracle


def test_uniform_router_reaches_the_optimum_of_the_load_balancing_loss():
    """All logits equal: probabilities 1 / E, so the loss is k / E whatever is selected (the reference's comment at
    fast_llm/layers/decoder/mlp/mixture_of_experts.py:247-248), and logsumexp = c + log(E)."""
    tokens, experts, k, constant = 64, 8, 2, 0.75
    result = moe_oracle.router(torch.full((tokens, experts), constant), k)
    assert result.load_balancing_loss.item() == pytest.approx(k / experts, rel=1e-6)
    assert result.z_loss.item() == pytest.approx((constant + math.log(experts)) ** 2, rel=1e-6)
    assert torch.allclose(result.scores, torch.full((tokens, k), 1 / k))


def test_collapsed_router_reaches_the_worst_case():
    """Every token puts all its probability on the same k experts: the loss is 1 (same comment, :249)."""
    tokens, experts, k = 32, 8, 2
    logits = torch.zeros(tokens, experts)
    logits[:, [3, 5]] = 60.0
    result = moe_oracle.router(logits, k)
    assert result.load_balancing_loss.item() == pytest.approx(1.0, rel=1e-6)
    assert sorted(result.top_experts[0].tolist()) == [3, 5]


def _loop_router(logits, noise, k, shared):
    """Textbook definitions, token by token, in Python floats."""
    tokens, experts = len(logits), len(logits[0])
    probability_mean, selected_mean, z = [0.0] * experts, [0.0] * experts, 0.0
    all_scores, all_experts = [], []
    for t in range(tokens):
        row = logits[t]
        z += math.log(sum(math.exp(v) for v in row)) ** 2 / tokens
        routed = [v * n for v, n in zip(row, noise[t])] if noise is not None else row
        total = sum(math.exp(v) for v in routed)
        order = sorted(range(experts), key=lambda e: -routed[e])[:k]
        top_total = sum(math.exp(routed[e]) for e in order)
        for e in range(experts):
            probability_mean[e] += math.exp(routed[e]) / total / tokens
        for e in order:
            selected_mean[e] += 1 / tokens
        all_scores.append([1.0] * shared + [math.exp(routed[e]) / top_total for e in order])
        all_experts.append(list(range(experts, experts + shared)) + order)
    return all_scores, all_experts, sum(p * s for p, s in zip(probability_mean, selected_mean)), z


@pytest.mark.parametrize("with_noise", [False, True])
@pytest.mark.parametrize(("tokens", "experts", "k", "shared"), [(9, 5, 2, 0), (17, 8, 3, 2), (4, 3, 3, 1)])
def test_router_against_a_per_token_loop(tokens, experts, k, shared, with_noise):
    generator = torch.Generator().manual_seed(tokens)
    logits = torch.randn(tokens, experts, generator=generator, dtype=torch.float64)
    noise = torch.empty_like(logits).uniform_(0.9, 1.1, generator=generator) if with_noise else None
    result = moe_oracle.router(logits, k, shared, noise, compute_dtype=torch.float64)
    scores, top_experts, load_balancing_loss, z_loss = _loop_router(
        logits.tolist(), None if noise is None else noise.tolist(), k, shared
    )
    assert result.top_experts.tolist() == top_experts
    assert torch.allclose(result.scores, torch.tensor(scores, dtype=torch.float64), rtol=1e-12)
    assert result.load_balancing_loss.item() == pytest.approx(load_balancing_loss, rel=1e-12)
    assert result.z_loss.item() == pytest.approx(z_loss, rel=1e-12)


def test_router_backward_is_the_derivative_of_the_trained_objective():
    """`AuxiliaryLoss` makes the backward of the scores also carry auxiliary_loss_grad * d(loss)/d(logits): central
    differences of <scores, g> + a * load_balancing_loss + z * z_loss computed by the loop above."""
    tokens, experts, k, shared = 6, 5, 2, 1
    generator = torch.Generator().manual_seed(1)
    logits = torch.randn(tokens, experts, generator=generator, dtype=torch.float64)
    noise = torch.empty_like(logits).uniform_(0.9, 1.1, generator=generator)
    grad_scores = torch.randn(tokens, shared + k, generator=generator, dtype=torch.float64)
    auxiliary_loss_grad, z_loss_grad = 0.7, 0.3

    leaf = logits.clone().requires_grad_()
    result = moe_oracle.router(leaf, k, shared, noise, compute_dtype=torch.float64)
    grad = moe_oracle.router_backward(result, leaf, grad_scores, auxiliary_loss_grad, z_loss_grad)

    def objective(values):
        scores, _, load_balancing_loss, z_loss = _loop_router(values, noise.tolist(), k, shared)
        weighted = sum(s * g for row, grads in zip(scores, grad_scores.tolist()) for s, g in zip(row, grads))
        return weighted + auxiliary_loss_grad * load_balancing_loss + z_loss_grad * z_loss

    step = 1e-6
    for t in range(tokens):
        for e in range(experts):
            up, down = logits.tolist(), logits.tolist()
            up[t][e] += step
            down[t][e] -= step
            numeric = (objective(up) - objective(down)) / (2 * step)
            assert grad[t, e].item() == pytest.approx(numeric, rel=1e-5, abs=1e-8)
