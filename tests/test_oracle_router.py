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


def test_sinkhorn_balances_rows_and_columns():
    """What the iteration converges to is fixed by the mathematics: a rescaling d0[t] exp(cost[t, e]) d1[e] whose rows
    sum to 1 / T exactly after the last row step... and whose columns sum to 1 / E (the last step rescales columns),
    rows then within the tolerance. The ordering inside a row is changed only through the column scales."""
    generator = torch.Generator().manual_seed(0)
    tokens, experts = 96, 8
    cost = torch.randn(tokens, experts, generator=generator)
    cost[:, 0] += 2.0  # an expert everybody prefers
    balanced = moe_oracle.sinkhorn(cost, tolerance=1e-7)
    assert torch.allclose(balanced.sum(0), torch.full((experts,), 1 / experts), rtol=1e-4)
    assert torch.allclose(balanced.sum(1), torch.full((tokens,), 1 / tokens), rtol=2e-3)
    # It is a diagonal rescaling of exp(cost): the ratio to exp(cost) has rank one.
    ratio = balanced / torch.exp(cost)
    assert torch.allclose(ratio, ratio[:, :1] * ratio[:1, :] / ratio[0, 0], rtol=1e-4)
    # Balancing spreads the load: the plain top-1 sends most tokens to expert 0, the balanced one does not.
    plain = torch.bincount(cost.argmax(-1), minlength=experts)
    spread = torch.bincount(balanced.argmax(-1), minlength=experts)
    assert plain[0] > tokens // 2 and spread.max() <= 2 * tokens // experts


def test_sinkhorn_against_a_python_loop():
    generator = torch.Generator().manual_seed(1)
    tokens, experts, tolerance, eps = 5, 3, 1e-5, 1e-9
    cost = torch.randn(tokens, experts, generator=generator)
    c = [[math.exp(v) for v in row] for row in cost.tolist()]
    d0, d1 = [1.0] * tokens, [1.0] * experts
    while True:
        d0 = [(1 / tokens) / (sum(d1[e] * c[t][e] for e in range(experts)) + eps) for t in range(tokens)]
        new = [(1 / experts) / (sum(d0[t] * c[t][e] for t in range(tokens)) + eps) for e in range(experts)]
        error = sum(abs(a - b) for a, b in zip(new, d1)) / experts
        d1 = new
        if not error > tolerance:
            break
    expected = torch.tensor([[d0[t] * c[t][e] * d1[e] for e in range(experts)] for t in range(tokens)])
    assert torch.allclose(moe_oracle.sinkhorn(cost, tolerance, eps), expected, rtol=1e-5)


@pytest.mark.parametrize("k", [1, 2])
def test_sinkhorn_routing_scores_are_the_activated_logits(k):
    generator = torch.Generator().manual_seed(2)
    logits = torch.randn(40, 6, generator=generator)
    for training in (True, False):
        scores, top_experts = moe_oracle.sinkhorn_routing(logits, k, training)
        for t in range(logits.size(0)):
            row = logits[t].tolist()
            if k == 1:
                activated = [1 / (1 + math.exp(-v)) for v in row]
            else:
                total = sum(math.exp(v) for v in row)
                activated = [math.exp(v) / total for v in row]
            for j in range(k):
                assert scores[t, j].item() == pytest.approx(activated[top_experts[t, j]], rel=1e-5)
            if not training:  # plain top-k of the activated logits, in descending order
                order = sorted(range(len(row)), key=lambda e: -row[e])[:k]
                assert top_experts[t].tolist() == order
        assert len({tuple(sorted(r)) for r in top_experts.tolist()}) > 1


def test_router_input_and_per_expert_scale():
    generator = torch.Generator().manual_seed(3)
    x = torch.randn(7, 5, generator=generator)
    scale = torch.rand(5, generator=generator) + 0.5

    def rms(t):
        return t / torch.sqrt((t * t).mean(-1, keepdim=True) + 1e-5)

    out = moe_oracle.router_input(x, rms, scale, 5**-0.5)
    for t in range(7):
        row = x[t].tolist()
        norm = math.sqrt(sum(v * v for v in row) / 5 + 1e-5)
        for h in range(5):
            assert out[t, h].item() == pytest.approx(row[h] / norm * scale[h].item() * 5**-0.5, rel=1e-5)
    assert moe_oracle.router_input(x) is x
    scores, top = torch.rand(7, 2, generator=generator), torch.randint(0, 4, (7, 2), generator=generator)
    per_expert = torch.tensor([1.0, 2.0, 0.5, 3.0])
    scaled = moe_oracle.per_expert_scale(scores, top, per_expert)
    for t in range(7):
        for j in range(2):
            assert scaled[t, j].item() == pytest.approx(scores[t, j].item() * per_expert[top[t, j]].item())
    assert moe_oracle.per_expert_scale(scores, top, None) is scores


def test_nan_logits_rank_highest_like_torch_topk():
    """The contract for a NaN router logit is torch.topk's (the reference routes with it): NaN ranks above every
    number, the token selects that expert, and its scores are NaN."""
    logits = torch.tensor([[0.5, float("nan"), 2.0, 1.0], [3.0, 1.0, 2.0, 0.0]])
    scores, top_experts = moe_oracle.topk_routing(logits, 2)
    assert top_experts[0].tolist() == [1, 2] and top_experts[1].tolist() == [0, 2]
    assert torch.isnan(scores[0]).all() and torch.isfinite(scores[1]).all()
