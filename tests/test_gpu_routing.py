"""Top-k routing on the GPU against torch.topk + fp32 softmax (what the reference's `_topk_routing` does,
fast_llm/layers/decoder/mlp/mixture_of_experts.py:243-244) and against autograd for the backward."""

import pytest
import torch

from fast_llm_amd.functional.routing import topk_routing
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
