"""Top-k routing on the GPU against torch.topk + fp32 softmax (what the reference's `_topk_routing` does,
fast_llm/layers/decoder/mlp/mixture_of_experts.py:243-244) and against autograd for the backward."""

import pytest
import torch

from fast_llm_amd import _lib
from fast_llm_amd.functional.routing import router, topk_routing
from oracle import moe_oracle

pytestmark = pytest.mark.gpu


# (tokens, experts, k): the reference's sparse-map test shapes plus the benchmark configurations' routers.
_SHAPES = [(2048, 8, 2), (2048, 6, 2), (2048, 8, 8), (256, 8, 2), (5627, 8, 2), (2048, 64, 2), (512, 64, 6), (300, 128, 8), (7, 1000, 64), (1, 1, 1)]


def _distinct_logits(tokens, experts, dtype, generator):
    """Router logits without ties within a row, so that the order of the selected experts does not depend on a
    tie-breaking rule (torch.topk leaves it open): random normals in fp32; in half precision, where random values
    collide, a random permutation of `experts` consecutive representable numbers starting at 1."""
    if dtype == torch.float32:
        return torch.randn(tokens, experts, generator=generator)
    one = torch.ones((), dtype=dtype).view(torch.int16).item()
    values = (torch.arange(experts, dtype=torch.int16) + one).view(dtype)
    order = torch.rand(tokens, experts, generator=generator).argsort(dim=-1)
    return values[order]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize(("tokens", "experts", "k"), _SHAPES)
def test_topk_routing_forward(tokens, experts, k, dtype, device):
    generator = torch.Generator().manual_seed(tokens + experts)
    logits = _distinct_logits(tokens, experts, dtype, generator)
    expected_scores, expected_experts = moe_oracle.topk_routing(logits.float(), k)
    scores, top_experts = topk_routing(logits.to(device), k)
    assert scores.dtype == torch.float32 and top_experts.dtype == torch.int64
    assert torch.equal(top_experts.cpu(), expected_experts)
    assert torch.allclose(scores.cpu(), expected_scores, rtol=2e-6, atol=1e-7)
    assert torch.allclose(scores.sum(-1).cpu(), torch.ones(tokens), atol=1e-5)


def test_topk_routing_ties_go_to_the_lower_expert(device):
    logits = torch.tensor([[1.0, 3.0, 3.0, 2.0, 3.0], [0.0, 0.0, 0.0, 0.0, 0.0]], device=device)
    scores, top_experts = topk_routing(logits, 3)
    assert top_experts.tolist() == [[1, 2, 4], [0, 1, 2]]
    assert torch.allclose(scores.cpu(), torch.full((2, 3), 1 / 3))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize(("tokens", "experts", "k"), [(1000, 8, 2), (333, 64, 6), (100, 130, 8), (5, 1000, 64)])
def test_topk_routing_backward(tokens, experts, k, dtype, device):
    generator = torch.Generator().manual_seed(3)
    logits = _distinct_logits(tokens, experts, dtype, generator)
    grad_scores = torch.randn(tokens, k, generator=generator)

    reference_logits = logits.float().clone().requires_grad_()
    reference_scores, _ = moe_oracle.topk_routing(reference_logits, k)
    reference_scores.backward(grad_scores)

    gpu_logits = logits.detach().to(device).requires_grad_()
    scores, top_experts = topk_routing(gpu_logits, k)
    assert not top_experts.requires_grad
    scores.backward(grad_scores.to(device))
    assert gpu_logits.grad.dtype == dtype
    tolerance = 1e-6 if dtype == torch.float32 else 1e-2
    error = (gpu_logits.grad.float().cpu() - reference_logits.grad).abs().max()
    assert error <= tolerance * max(reference_logits.grad.abs().max().item(), 1e-6)
    # exactly zero where no expert was selected
    selected = torch.zeros(tokens, experts, dtype=torch.bool).scatter_(1, top_experts.cpu(), True)
    assert (gpu_logits.grad.cpu()[~selected] == 0).all()


def _spaced_logits(tokens, experts, dtype, generator):
    """Rows that stay free of ties after a jitter of a few percent, also in half precision: a random permutation of
    1, 1.25, 1.5, ... (exact in bf16 up to 64 experts), plus a small perturbation in fp32."""
    values = 1 + 0.25 * torch.arange(experts, dtype=torch.float32)
    order = torch.rand(tokens, experts, generator=generator).argsort(dim=-1)
    logits = values[order]
    if dtype == torch.float32:
        logits = logits + 0.05 * torch.randn(tokens, experts, generator=generator)
    return logits.to(dtype)


# (tokens, experts, k, shared experts, jitter): the benchmark's routers, a token count that leaves workgroups of the
# forward kernel with unequal or no share, more experts than a wavefront has lanes.
_ROUTER_CASES = [
    (8192, 8, 2, 0, False),
    (2048, 8, 2, 1, True),
    (1000, 64, 6, 2, False),
    (16411, 8, 2, 0, True),
    (37, 8, 3, 0, False),
    (300, 130, 8, 3, False),
    (5, 1000, 60, 4, False),
    (1, 2, 1, 0, True),
    (16384, 128, 8, 0, False),  # the routers of the wide and fine-grained configurations at full size
    (16384, 64, 6, 2, False),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize(("tokens", "experts", "k", "shared", "jitter"), _ROUTER_CASES)
def test_router_forward_and_backward(tokens, experts, k, shared, jitter, dtype, device):
    generator = torch.Generator().manual_seed(tokens + experts)
    if jitter:
        logits = _spaced_logits(tokens, experts, dtype, generator)
        noise = torch.empty(tokens, experts).uniform_(0.99, 1.01, generator=generator).to(dtype)
    else:
        logits, noise = _distinct_logits(tokens, experts, dtype, generator), None
    grad_scores = torch.randn(tokens, shared + k, generator=generator)
    auxiliary_loss_grad, z_loss_grad = 0.01 * experts * tokens, 0.001 * tokens

    # The oracle in the reference's arithmetic: the jitter product in `dtype`, softmaxes in fp32.
    leaf = logits.clone().requires_grad_()
    expected = moe_oracle.router(leaf, k, shared, noise)
    expected_grad = moe_oracle.router_backward(expected, leaf, grad_scores, auxiliary_loss_grad, z_loss_grad)

    gpu_logits = logits.to(device).requires_grad_()
    scores, top_experts, load_balancing_loss, z_loss = router(
        gpu_logits,
        k,
        shared_experts=shared,
        noise=None if noise is None else noise.to(device),
        auxiliary_loss_grad=auxiliary_loss_grad,
        z_loss_grad=z_loss_grad,
    )
    assert scores.dtype == torch.float32 and top_experts.dtype == torch.int64
    assert not load_balancing_loss.requires_grad and not z_loss.requires_grad
    assert torch.equal(top_experts.cpu(), expected.top_experts)
    assert torch.allclose(scores.cpu(), expected.scores.detach(), rtol=2e-6, atol=1e-7)
    assert load_balancing_loss.item() == pytest.approx(expected.load_balancing_loss.item(), rel=1e-5)
    assert z_loss.item() == pytest.approx(expected.z_loss.item(), rel=1e-5)

    scores.backward(grad_scores.to(device))
    assert gpu_logits.grad.dtype == dtype
    tolerance = 1e-5 if dtype == torch.float32 else 1e-2
    error = (gpu_logits.grad.float().cpu() - expected_grad.float()).abs().max().item()
    assert error <= tolerance * expected_grad.float().abs().max().item()


def test_router_without_trained_losses_matches_plain_topk_routing(device):
    generator = torch.Generator().manual_seed(2)
    logits = torch.randn(777, 16, generator=generator).to(device)
    grad_scores = torch.randn(777, 4, generator=generator).to(device)
    plain_logits, fused_logits = logits.clone().requires_grad_(), logits.clone().requires_grad_()
    plain_scores, plain_experts = topk_routing(plain_logits, 4)
    fused_scores, fused_experts, _, _ = router(fused_logits, 4)
    assert torch.equal(plain_experts, fused_experts) and torch.equal(plain_scores, fused_scores)
    plain_scores.backward(grad_scores)
    fused_scores.backward(grad_scores)
    assert torch.equal(plain_logits.grad, fused_logits.grad)


def test_router_statistics_do_not_depend_on_scheduling(device):
    logits = torch.randn(30000, 64, generator=torch.Generator().manual_seed(4)).to(device)
    first = router(logits, 6)
    for _ in range(3):
        again = router(logits, 6)
        assert all(torch.equal(a, b) for a, b in zip(first, again))


def test_routing_feeds_the_layer(device):
    """The layer's router path uses the kernel and stays differentiable down to the router weights."""
    from fast_llm_amd.layers.moe import DroplessMoEMLP

    torch.manual_seed(0)
    layer = DroplessMoEMLP(256, 256, 8, 2, dtype=torch.bfloat16, device=device)
    x = torch.randn(512, 256, dtype=torch.bfloat16, device=device, requires_grad=True)
    out = layer(x)
    out.float().square().mean().backward()
    assert torch.isfinite(out).all() and x.grad is not None and layer.router.grad is not None
    assert layer.router.grad.abs().sum() > 0


def test_layer_with_shared_experts_and_trained_router_losses(device):
    """The whole block, router included, against the oracle's router followed by its per-expert loop, with torch
    autograd of both for the gradients down to the router weights."""
    from fast_llm_amd.layers.moe import LOAD_BALANCING_LOSS, ROUTER_Z_LOSS, DroplessMoEMLP

    torch.manual_seed(1)
    tokens, hidden, ffn, experts, k, shared = 384, 128, 128, 6, 2, 1
    coefficient, z_coefficient, grad_scale = 0.05, 0.002, 3.0
    layer = DroplessMoEMLP(
        hidden, ffn, experts, k, shared_experts=shared, auxiliary_loss_coefficient=coefficient,
        z_loss_coefficient=z_coefficient, init_std=0.1, dtype=torch.float32, device=device,
    )  # fmt: skip
    x = torch.randn(tokens, hidden, device=device, requires_grad=True)
    grad_output = torch.randn(tokens, hidden, device=device)
    losses = {}
    out = layer(x, grad_scale=grad_scale, losses=losses)
    out.backward(grad_output)

    leaves = [t.detach().cpu().clone().requires_grad_() for t in (x, layer.router, layer.layer_1, layer.layer_2)]
    x_cpu, router_weight, weight_1, weight_2 = leaves
    routed = moe_oracle.router(torch.nn.functional.linear(x_cpu, router_weight), k, shared)
    expected = moe_oracle.looped_moe(x_cpu, routed.scores, routed.top_experts, weight_1, weight_2, experts)
    objective = (
        (expected * grad_output.cpu()).sum()
        + (experts - shared) * coefficient * grad_scale * routed.load_balancing_loss
        + z_coefficient * grad_scale * routed.z_loss
    )
    objective.backward()

    def close(actual, reference, tolerance=1e-4):
        return (actual.cpu() - reference).abs().max() <= tolerance * reference.abs().max()

    assert close(out.detach(), expected.detach())
    assert losses[LOAD_BALANCING_LOSS][0].item() == pytest.approx(routed.load_balancing_loss.item(), rel=1e-5)
    assert losses[ROUTER_Z_LOSS][0].item() == pytest.approx(routed.z_loss.item(), rel=1e-5)
    assert close(x.grad, x_cpu.grad)
    assert close(layer.router.grad, router_weight.grad)
    assert close(layer.layer_1.grad_buffer, weight_1.grad) and close(layer.layer_2.grad_buffer, weight_2.grad)


def test_router_with_masked_experts_and_full_selection(device):
    """Experts masked out with -inf logits (how the forced-empty benchmark case is built) are never selected, get
    probability 0 and a zero gradient; with k equal to the number of experts every expert is selected and the scores
    are the full softmax."""
    generator = torch.Generator().manual_seed(8)
    logits = torch.randn(300, 8, generator=generator)
    logits[:, 5] = float("-inf")
    leaf = logits.clone().requires_grad_()
    expected = moe_oracle.router(leaf, 2)
    grad_scores = torch.randn(300, 2, generator=generator)
    expected_grad = moe_oracle.router_backward(expected, leaf, grad_scores, 0.3, 0.1)
    gpu_logits = logits.to(device).requires_grad_()
    scores, top_experts, load_balancing_loss, z_loss = router(gpu_logits, 2, auxiliary_loss_grad=0.3, z_loss_grad=0.1)
    assert torch.equal(top_experts.cpu(), expected.top_experts) and not (top_experts == 5).any()
    assert load_balancing_loss.item() == pytest.approx(expected.load_balancing_loss.item(), rel=1e-5)
    assert z_loss.item() == pytest.approx(expected.z_loss.item(), rel=1e-5)
    scores.backward(grad_scores.to(device))
    assert torch.isfinite(gpu_logits.grad).all() and (gpu_logits.grad[:, 5] == 0).all()
    assert torch.allclose(gpu_logits.grad.cpu(), expected_grad, rtol=1e-4, atol=1e-7)

    logits = torch.randn(64, 6, generator=generator)
    scores, top_experts, _, _ = router(logits.to(device), 6)
    assert torch.equal(top_experts.cpu().sort(dim=-1).values, torch.arange(6).expand(64, 6))
    full = torch.softmax(logits, dim=-1)
    assert torch.allclose(scores.cpu(), full.gather(1, top_experts.cpu()), rtol=2e-6, atol=1e-7)


# (tokens, routed experts, k, shared): the five benchmark configurations' routers, shared experts, token counts that
# leave the router's last workgroups short or empty, more than 1024 x 16 tokens (several map chunks per workgroup),
# and slot counts that do not divide the map kernel's chunk of 1024 entries.
_HANDOFF_CASES = [
    (512, 8, 2, 0), (8192, 8, 2, 0), (16384, 64, 6, 0), (16384, 128, 8, 0), (8192, 8, 2, 2), (100, 6, 3, 1),
    (1, 4, 2, 0), (17, 5, 5, 3), (40000, 16, 7, 1), (70001, 1000, 3, 0), (5627, 60, 56, 8),
]  # fmt: skip


@pytest.mark.parametrize(("tokens", "experts", "k", "shared"), _HANDOFF_CASES)
@pytest.mark.parametrize("zipf", [False, True])
def test_sparse_map_from_the_routers_counts(tokens, experts, k, shared, zipf, device):
    """The router already counts the tokens of every expert; the map built from those counts (no counting pass over
    `top_experts`) equals the map built from `top_experts` alone and the oracle's map, bit for bit."""
    from fast_llm_amd.functional.sparse_copy import get_sparse_map

    generator = torch.Generator().manual_seed(tokens + 31 * experts + shared)
    logits = torch.randn(tokens, experts, generator=generator)
    if zipf:  # load imbalance, near-empty experts
        logits += 3 * torch.log(torch.arange(1, experts + 1, dtype=torch.float32) ** -1.2)
    scores, top_experts, _, _, counts = router(logits.to(device), k, shared_experts=shared, return_counts=True)
    total = experts + shared
    with _lib.KernelTimer() as timer:
        handed = get_sparse_map(top_experts, total, router_counts=counts)
    assert set(timer.durations_ms()) == {"fm_sparse_map_from_router"}
    counted = get_sparse_map(top_experts, total)
    expected = moe_oracle.sparse_map(top_experts.cpu(), total)
    for name in ("sparse_rows", "expert_ends", "expert_pad_begins"):
        ours = getattr(handed, name)
        assert ours.dtype == getattr(counted, name).dtype
        assert torch.equal(ours, getattr(counted, name)), name
        assert torch.equal(ours.cpu().long(), getattr(expected, name)), name
    assert handed.num_rows == counted.num_rows == expected.num_rows
    with pytest.raises(AssertionError):  # counts of another routing
        get_sparse_map(top_experts[: tokens // 2 + 1], total, router_counts=counts) if tokens > 1 else get_sparse_map(
            top_experts, total + 1, router_counts=counts
        )


def test_router_counts_of_edited_selections_are_not_used(device):
    """Counts belong to the `top_experts` tensor the router returned, as it was: a copy of it, or the tensor itself
    after an in-place edit (a masking or dropping hook), is counted afresh, and the map is the edited selection's."""
    from fast_llm_amd.functional.sparse_copy import get_sparse_map

    tokens, experts, k = 3000, 16, 4
    logits = torch.randn(tokens, experts, generator=torch.Generator().manual_seed(11))
    _, top_experts, _, _, counts = router(logits.to(device), k, return_counts=True)
    with _lib.KernelTimer() as timer:
        copied = get_sparse_map(top_experts.clone(), experts, router_counts=counts)
    assert set(timer.durations_ms()) == {"fm_sparse_map"}
    assert torch.equal(copied.sparse_rows, get_sparse_map(top_experts, experts).sparse_rows)
    top_experts[::3, 0] = (top_experts[::3, 0] + 5) % experts  # the counts no longer describe these selections
    with _lib.KernelTimer() as timer:
        edited = get_sparse_map(top_experts, experts, router_counts=counts)
    assert set(timer.durations_ms()) == {"fm_sparse_map"}
    expected = moe_oracle.sparse_map(top_experts.cpu(), experts)
    for name in ("sparse_rows", "expert_ends", "expert_pad_begins"):
        assert torch.equal(getattr(edited, name).cpu().long(), getattr(expected, name)), name


def _rms_norm(hidden: int, device) -> torch.nn.Module:
    class RMSNorm(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.rand(hidden, device=device) + 0.5)

        def forward(self, x):
            return x * torch.rsqrt((x.float() ** 2).mean(-1, keepdim=True) + 1e-5).to(x.dtype) * self.weight

    return RMSNorm()


@pytest.mark.parametrize("routing", ["aux_loss", "sinkhorn"])
@pytest.mark.parametrize("training", [True, False])
def test_layer_with_router_input_options(routing, training, device):
    """The router's own view of the input (normalisation layer, per-feature scale, constant), the per-expert scale on
    the scores and sinkhorn routing (fast_llm/layers/decoder/mlp/config.py:101-122, 147-151;
    mixture_of_experts.py:130-175, 280-296): the whole block against the oracle's restatement of those steps followed by
    its per-expert loop, gradients down to every router-side parameter by torch autograd of the restatement."""
    from fast_llm_amd.layers.moe import DroplessMoEMLP

    torch.manual_seed(7)
    tokens, hidden, ffn, experts, k = 320, 128, 128, 8, 2
    norm = _rms_norm(hidden, device)
    layer = DroplessMoEMLP(
        hidden, ffn, experts, k, routing=routing, router_normalization=norm, router_scale=True,
        router_input_scale=hidden**-0.5 * 8, router_per_expert_scale=True, auxiliary_loss_coefficient=0.0,
        init_std=0.1, dtype=torch.float32, device=device,
    )  # fmt: skip
    with torch.no_grad():
        layer.router_scale.uniform_(0.5, 1.5)
        layer.router_per_expert_scale.uniform_(0.5, 1.5)
    layer.train(training)
    x = torch.randn(tokens, hidden, device=device, requires_grad=True)
    grad_output = torch.randn(tokens, hidden, device=device)
    out = layer(x)
    if training:
        out.backward(grad_output)

    parameters = (x, layer.router, layer.layer_1, layer.layer_2, norm.weight, layer.router_scale, layer.router_per_expert_scale)
    leaves = [t.detach().cpu().clone().requires_grad_() for t in parameters]
    x_cpu, router_weight, weight_1, weight_2, norm_weight, scale, expert_scale = leaves

    def cpu_norm(t):
        return t * torch.rsqrt((t**2).mean(-1, keepdim=True) + 1e-5) * norm_weight

    router_in = moe_oracle.router_input(x_cpu, cpu_norm, scale, hidden**-0.5 * 8)
    logits = torch.nn.functional.linear(router_in, router_weight)
    if routing == "sinkhorn":
        scores, top_experts = moe_oracle.sinkhorn_routing(logits, k, training)
    else:
        routed = moe_oracle.router(logits, k)
        scores, top_experts = routed.scores, routed.top_experts
    scores = moe_oracle.per_expert_scale(scores, top_experts, expert_scale)
    expected = moe_oracle.looped_moe(x_cpu, scores, top_experts, weight_1, weight_2, experts)

    def close(actual, reference, tolerance=2e-4):
        return (actual.cpu() - reference).abs().max() <= tolerance * reference.abs().max()

    gpu_scores, gpu_experts = layer.route(x.detach())
    assert torch.equal(gpu_experts.cpu(), top_experts)
    assert close(gpu_scores.detach(), scores.detach(), 1e-5)
    assert close(out.detach(), expected.detach())
    if training:
        (expected * grad_output.cpu()).sum().backward()
        assert close(x.grad, x_cpu.grad)
        for ours, theirs in ((layer.router, router_weight), (norm.weight, norm_weight), (layer.router_scale, scale),
                             (layer.router_per_expert_scale, expert_scale)):  # fmt: skip
            assert close(ours.grad, theirs.grad), ours.shape
        assert close(layer.layer_1.grad_buffer, weight_1.grad) and close(layer.layer_2.grad_buffer, weight_2.grad)


def test_sinkhorn_on_the_gpu_matches_the_restatement(device):
    from fast_llm_amd.functional.routing import sinkhorn, sinkhorn_routing

    generator = torch.Generator().manual_seed(11)
    logits = torch.randn(500, 16, generator=generator)
    assert torch.allclose(sinkhorn(logits.to(device)).cpu(), moe_oracle.sinkhorn(logits), rtol=1e-4, atol=1e-9)
    for k in (1, 3):
        for training in (True, False):
            scores, top_experts = sinkhorn_routing(logits.to(device), k, training)
            expected_scores, expected_experts = moe_oracle.sinkhorn_routing(logits, k, training)
            assert torch.equal(top_experts.cpu(), expected_experts)
            assert torch.allclose(scores.cpu(), expected_scores, rtol=1e-5)
    with pytest.raises(ValueError):
        from fast_llm_amd.layers.moe import DroplessMoEMLP

        DroplessMoEMLP(64, 64, 4, 1, routing="sinkhorn", shared_experts=1, device=device)


def test_nan_logits_rank_highest_like_torch_topk(device):
    """A NaN logit is selected first (torch.topk's order, which the reference's routing inherits) and makes the
    token's scores NaN; every slot still names a valid expert, and other tokens are unaffected. Both routing kernels."""
    generator = torch.Generator().manual_seed(5)
    logits = torch.randn(64, 8, generator=generator)
    logits[3, 6] = float("nan")
    logits[10, 0] = logits[10, 7] = float("nan")  # two NaNs: the lower expert first
    expected_scores, expected_experts = moe_oracle.topk_routing(logits, 2)
    for function in (
        lambda: topk_routing(logits.to(device), 2),
        lambda: router(logits.to(device), 2)[:2],
    ):
        scores, top_experts = function()
        assert top_experts[3, 0].item() == 6 and top_experts[10].tolist() == [0, 7]
        assert ((top_experts >= 0) & (top_experts < 8)).all()
        clean = torch.ones(64, dtype=torch.bool)
        clean[[3, 10]] = False
        assert torch.equal(top_experts.cpu()[clean], expected_experts[clean])
        assert torch.allclose(scores.cpu()[clean], expected_scores[clean], rtol=2e-6, atol=1e-7)
        assert torch.isnan(scores[3]).all() and torch.isnan(scores[10]).all()
