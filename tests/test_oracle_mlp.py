"""Pins the oracle's activation, the composed dropless MLP and the looped MoE."""

import pytest
import torch

from oracle import moe_oracle
from tests.helpers import REFERENCE_FIXTURES, rms_diff

_TORCH_ACTIVATIONS = {
    "gelu": lambda x: torch.nn.functional.gelu(x, approximate="tanh"),
    "silu": torch.nn.functional.silu,
    "relu": torch.nn.functional.relu,
    "squared_relu": lambda x: torch.pow(torch.nn.functional.relu(x), 2),
    "identity": lambda x: x,
}


@pytest.mark.parametrize("gated", [True, False])
@pytest.mark.parametrize("activation", REFERENCE_FIXTURES["activation"]["activations"])
def test_activation_matches_torch_autograd(gated, activation):
    """Same construction as the reference's test (tests/functional/test_triton_kernels.py:167-193), in float64."""
    fixture = REFERENCE_FIXTURES["activation"]
    torch.manual_seed(0)
    input_ = torch.randn(fixture["rows"], fixture["columns"] * (2 if gated else 1), dtype=torch.float64)
    input_.requires_grad_(True)
    grad_output = torch.randn(fixture["rows"], fixture["columns"], dtype=torch.float64)
    if gated:
        x1, x2 = input_.chunk(2, dim=-1)
        expected = _TORCH_ACTIVATIONS[activation](x1) * x2
    else:
        expected = _TORCH_ACTIVATIONS[activation](input_)
    expected.backward(grad_output)
    output = moe_oracle.mlp_activation_forward(input_.detach(), gated, activation, compute_dtype=torch.float64)
    grad_input, recomputed = moe_oracle.mlp_activation_backward(
        grad_output, input_.detach(), gated, activation, compute_dtype=torch.float64
    )
    # The tanh-gelu constants of the reference are rounded to 8 digits, hence 1e-7 for gelu.
    tolerance = 1e-7 if activation == "gelu" else 1e-13
    assert rms_diff(output, expected.detach()) < tolerance
    assert rms_diff(recomputed, expected.detach()) < tolerance
    assert rms_diff(grad_input, input_.grad) < tolerance


def test_silu_derivative_is_finite_at_the_extremes():
    x = torch.tensor([[-200.0, -88.0, -20.0, 0.0, 20.0, 88.0, 200.0]])
    grad, _ = moe_oracle.mlp_activation_backward(torch.ones_like(x), x, False, "silu")
    assert torch.isfinite(grad).all()
    torch.testing.assert_close(grad[0, [0, 3, 6]], torch.tensor([0.0, 0.5, 1.0]))


def _textbook_moe(x, scores, top_experts, weight_1, weight_2, experts):
    """Token-by-token mixture: y[t] = sum_j s[t, j] * W2_e^T (silu(Wg_e x) * (Wu_e x)), e = top_experts[t, j]."""
    ffn = weight_2.size(0) // experts
    out = torch.zeros_like(x)
    for t in range(x.size(0)):
        for j in range(top_experts.size(1)):
            e = int(top_experts[t, j])
            w1 = weight_1[e * 2 * ffn : (e + 1) * 2 * ffn]
            gate, up = w1[:ffn] @ x[t], w1[ffn:] @ x[t]
            hidden = torch.nn.functional.silu(gate) * up
            out[t] = out[t] + scores[t, j] * (hidden @ weight_2[e * ffn : (e + 1) * ffn])
    return out


def _make_problem(tokens, hidden, ffn, experts, top_k, seed, empty_expert=None):
    generator = torch.Generator().manual_seed(seed)
    normal = lambda *shape: torch.randn(*shape, dtype=torch.float64, generator=generator)  # noqa: E731
    x, grad = normal(tokens, hidden), normal(tokens, hidden)
    weight_1, weight_2 = normal(experts * 2 * ffn, hidden) / 8, normal(experts * ffn, hidden) / 8
    logits = normal(tokens, experts)
    if empty_expert is not None:
        logits[:, empty_expert] = float("-inf")
    scores, top_experts = moe_oracle.topk_routing(logits, top_k)
    return x, grad, weight_1, weight_2, scores.double(), top_experts


def test_looped_moe_matches_textbook_mixture():
    x, grad, weight_1, weight_2, scores, top_experts = _make_problem(19, 8, 6, 4, 2, seed=0)
    leaves = [t.clone().requires_grad_(True) for t in (x, scores, weight_1, weight_2)]
    expected = _textbook_moe(leaves[0], leaves[1], top_experts, leaves[2], leaves[3], 4)
    expected.backward(grad)
    result = moe_oracle.looped_moe_forward_backward(x, scores, top_experts, weight_1, weight_2, 4, grad)
    for ours, theirs in zip(
        (result.output, result.grad_input, result.grad_scores, result.grad_weight_1, result.grad_weight_2),
        (expected.detach(), *(leaf.grad for leaf in leaves)),
    ):
        torch.testing.assert_close(ours, theirs, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("empty_expert", [None, 2])
@pytest.mark.parametrize("pad", [8, 128])
def test_dropless_mlp_matches_looped_moe(empty_expert, pad):
    """The dropless algebra (NaN in every padding row) equals the per-expert loop: output, input gradient, score
    gradient and both weight gradients; no NaN reaches a result."""
    experts, top_k = 5, 2
    x, grad, weight_1, weight_2, scores, top_experts = _make_problem(41, 16, 12, experts, top_k, 1, empty_expert)
    sparse_map = moe_oracle.sparse_map(top_experts, experts, pad)
    dropless = moe_oracle.dropless_mlp_forward_backward(
        x, scores, weight_1, weight_2, sparse_map, grad, compute_dtype=torch.float64
    )
    looped = moe_oracle.looped_moe_forward_backward(x, scores, top_experts, weight_1, weight_2, experts, grad)
    for name in ("output", "grad_input", "grad_scores", "grad_weight_1", "grad_weight_2"):
        ours, theirs = getattr(dropless, name), getattr(looped, name)
        assert torch.isfinite(ours).all(), name
        torch.testing.assert_close(ours, theirs, rtol=1e-11, atol=1e-12, msg=name)
    if empty_expert is not None:
        ffn = weight_2.size(0) // experts
        assert (dropless.grad_weight_2[empty_expert * ffn : (empty_expert + 1) * ffn] == 0).all()
    # Padding rows of the intermediates do carry the poison: it is the consumers that must skip them.
    padding = ~sparse_map.real_row_mask()
    padding[int(sparse_map.expert_ends[-1]) :] = False
    assert padding.any() and dropless.intermediates["layer_1"][padding].isnan().all()


def test_dropless_mlp_reference_test_configuration_fp32():
    """The configuration of the reference's `test_dropless_mlp` (tests/functional/test_functional.py:89-183), scaled
    down in width, in fp32: dropless vs looped within that test's rms thresholds."""
    fixture = REFERENCE_FIXTURES["dropless_mlp"]
    experts, top_k, std = fixture["experts"], fixture["experts_per_token"], fixture["std"]
    tokens, hidden, ffn = fixture["tokens"], 128, 256
    torch.manual_seed(0)
    x = torch.randn(tokens, hidden)
    router = torch.normal(0, std, (experts, hidden))
    scores, top_experts = moe_oracle.topk_routing(x @ router.t(), top_k)
    grad = torch.randn(tokens, hidden)
    weight_1 = torch.normal(0, std, (ffn * 2 * experts, hidden))
    weight_2 = torch.normal(0, std, (ffn * experts, hidden))
    sparse_map = moe_oracle.sparse_map(top_experts, experts)
    dropless = moe_oracle.dropless_mlp_forward_backward(x, scores, weight_1, weight_2, sparse_map, grad)
    looped = moe_oracle.looped_moe_forward_backward(x, scores, top_experts, weight_1, weight_2, experts, grad)
    assert rms_diff(dropless.output, looped.output) < fixture["rms_output"]
    assert rms_diff(dropless.grad_input, looped.grad_input) < fixture["rms_input_grad"]
    assert rms_diff(dropless.grad_scores, looped.grad_scores) < fixture["rms_scores_grad"]
    assert rms_diff(dropless.grad_weight_1, looped.grad_weight_1) < fixture["rms_weight_grad"]
    assert rms_diff(dropless.grad_weight_2, looped.grad_weight_2) < fixture["rms_weight_grad"]
