"""Pins the oracle's copies and grouped matrix products with formulations that do not share code with it."""

import pytest
import torch

from oracle import moe_oracle
from tests.helpers import REFERENCE_FIXTURES, fixture_sparse_map, rms_diff


def _small_map(tokens=37, experts=5, top_k=3, pad=8, seed=0):
    generator = torch.Generator().manual_seed(seed)
    logits = torch.randn(tokens, experts, generator=generator)
    scores, top_experts = moe_oracle.topk_routing(logits, top_k)
    return moe_oracle.sparse_map(top_experts, experts, pad), scores.double(), generator


def test_dispatch_and_combine_match_explicit_loops():
    sparse_map, scores, generator = _small_map()
    x = torch.randn(sparse_map.num_rows_dense, 6, dtype=torch.float64, generator=generator)
    y = torch.randn(sparse_map.num_rows, 6, dtype=torch.float64, generator=generator)
    for use_scores in (False, True):
        s = scores if use_scores else None
        dispatched = moe_oracle.copy_dense_to_sparse(x, s, sparse_map, fill=-7.0, compute_dtype=torch.float64)
        combined = moe_oracle.copy_sparse_to_dense(y, s, sparse_map, compute_dtype=torch.float64)
        expected_dispatch = torch.full_like(dispatched, -7.0)
        expected_combine = torch.zeros_like(combined)
        for t in range(sparse_map.num_rows_dense):
            for j in range(sparse_map.num_experts_per_token):
                row = int(sparse_map.sparse_rows[t, j])
                weight = float(scores[t, j]) if use_scores else 1.0
                expected_dispatch[row] = x[t] * weight
                expected_combine[t] += y[row] * weight
        assert torch.equal(dispatched, expected_dispatch)
        torch.testing.assert_close(combined, expected_combine, rtol=1e-14, atol=1e-14)
        # Dispatch and combine are adjoint on the real rows: <dispatch(x), y> == <x, combine(y)>.
        mask = sparse_map.real_row_mask()
        lhs = (dispatched[mask] * y[mask]).sum()
        rhs = (x * combined).sum()
        torch.testing.assert_close(lhs, rhs, rtol=1e-12, atol=1e-12)


def test_unscored_dispatch_is_a_bit_copy_and_skips_padding():
    sparse_map, _, generator = _small_map(seed=3)
    x = torch.randn(sparse_map.num_rows_dense, 4, generator=generator).to(torch.bfloat16)
    out = moe_oracle.copy_dense_to_sparse(x, None, sparse_map, fill=float("nan"))
    mask = sparse_map.real_row_mask()
    assert out[~mask].isnan().all() and not out[mask].isnan().any()
    assert torch.equal(out[sparse_map.sparse_rows[:, 1]], x)


def test_grad_score_is_the_autograd_gradient_of_combine():
    sparse_map, scores, generator = _small_map(seed=5)
    y = torch.randn(sparse_map.num_rows, 6, dtype=torch.float64, generator=generator)
    grad_output = torch.randn(sparse_map.num_rows_dense, 6, dtype=torch.float64, generator=generator)
    scores = scores.clone().requires_grad_(True)
    y_leaf = y.clone().requires_grad_(True)
    rows = sparse_map.sparse_rows
    combined = (y_leaf[rows] * scores[:, :, None]).sum(1)
    combined.backward(grad_output)
    grad_scores = moe_oracle.copy_sparse_to_dense_grad_score(y, grad_output, sparse_map, compute_dtype=torch.float64)
    torch.testing.assert_close(grad_scores, scores.grad, rtol=1e-13, atol=1e-13)
    # and the input gradient of the combine is the scored dispatch of grad_output
    grad_input = moe_oracle.copy_dense_to_sparse(grad_output, scores.detach(), sparse_map, compute_dtype=torch.float64)
    torch.testing.assert_close(grad_input, y_leaf.grad, rtol=1e-13, atol=1e-13)


def _expert_of_rows(sparse_map) -> torch.Tensor:
    # The docstring formula of the reference: sparse_index[i] = sum(expert_ends <= i).
    rows = torch.arange(sparse_map.num_rows)
    return (sparse_map.expert_ends[None, :] <= rows[:, None]).sum(1)


@pytest.mark.parametrize("case", REFERENCE_FIXTURES["sparse_matmul"]["cases"])
def test_grouped_matmuls_on_reference_fixtures(case):
    """Formulas of fast_llm/functional/triton/sparse_linear.py:267-273, 394-400, 527-535 evaluated with one dense
    matmul over a block-embedded operand, on the reference's hand-written expert layouts."""
    torch.manual_seed(0)
    sparse_map = fixture_sparse_map(case)
    std = REFERENCE_FIXTURES["sparse_matmul"]["std"]
    dense_dim, sparse_dim, experts, tokens = case["dense_dim"], case["sparse_dim"], sparse_map.num_experts, sparse_map.num_rows
    expert = _expert_of_rows(sparse_map)
    one_hot = torch.nn.functional.one_hot(expert, experts).double()  # [rows, E]

    # output-sparse: out[i, js] = sum_k lhs[i, k] rhs[k, js + N_s * e(i)]
    lhs = torch.normal(0, std, (tokens, dense_dim), dtype=torch.float64)
    rhs = torch.normal(0, std, (dense_dim, sparse_dim * experts), dtype=torch.float64)
    full = (lhs @ rhs).view(tokens, experts, sparse_dim)
    expected = (full * one_hot[:, :, None]).sum(1)
    out = moe_oracle.output_sparse_matmul(lhs, rhs, sparse_map, compute_dtype=torch.float64)
    assert rms_diff(out, expected) < 1e-14

    # input-inner-sparse: out[i, j] = sum_ks lhs[i, ks] rhs[ks + K_s * e(i), j]
    lhs = torch.normal(0, std, (tokens, sparse_dim), dtype=torch.float64)
    rhs = torch.normal(0, std, (sparse_dim * experts, dense_dim), dtype=torch.float64)
    embedded = (one_hot[:, :, None] * lhs[:, None, :]).reshape(tokens, experts * sparse_dim)
    out = moe_oracle.input_inner_sparse_matmul(lhs, rhs, sparse_map, compute_dtype=torch.float64)
    assert rms_diff(out, embedded @ rhs) < 1e-14

    # input-row-sparse: out[is + M_s * e, j] = sum_{ks real row of e} lhs[is, ks] rhs[ks, j]
    lhs = torch.normal(0, std, (sparse_dim, tokens), dtype=torch.float64)
    rhs = torch.normal(0, std, (tokens, dense_dim), dtype=torch.float64)
    rows = torch.arange(tokens)
    begins = sparse_map.expert_begins
    real = (rows[None, :] >= begins[:, None]) & (rows[None, :] < sparse_map.expert_pad_begins[:, None])  # [E, rows]
    expected = torch.einsum("ik,ek,kj->eij", lhs, real.double(), rhs).reshape(experts * sparse_dim, dense_dim)
    out = moe_oracle.input_row_sparse_matmul(lhs, rhs, sparse_map, compute_dtype=torch.float64)
    assert rms_diff(out, expected) < 1e-14
    # Padding rows must not leak even when they hold NaN.
    poisoned = rhs.clone()
    poisoned[~real.any(0)] = float("nan")
    out = moe_oracle.input_row_sparse_matmul(lhs, poisoned, sparse_map, compute_dtype=torch.float64)
    assert rms_diff(out, expected) < 1e-14
    if 0 in case["tokens_per_expert"]:
        empty = case["tokens_per_expert"].index(0)
        assert (out[empty * sparse_dim : (empty + 1) * sparse_dim] == 0).all()


def test_grouped_matmul_accumulate_and_phantom_rows():
    case = REFERENCE_FIXTURES["sparse_matmul"]["cases"][0]
    sparse_map = fixture_sparse_map(case)
    sparse_map.num_rows += 128  # a phantom tail past the last expert
    torch.manual_seed(1)
    lhs = torch.randn(sparse_map.num_rows, 16, dtype=torch.float64)
    rhs = torch.randn(16, 8 * 3, dtype=torch.float64)
    previous = torch.randn(sparse_map.num_rows, 8, dtype=torch.float64)
    plain = moe_oracle.output_sparse_matmul(lhs, rhs, sparse_map, out=previous.clone(), compute_dtype=torch.float64)
    added = moe_oracle.output_sparse_matmul(
        lhs, rhs, sparse_map, out=previous.clone(), accumulate=True, compute_dtype=torch.float64
    )
    used = sparse_map.expert_ends[-1]
    assert torch.equal(plain[used:], previous[used:]) and torch.equal(added[used:], previous[used:])
    torch.testing.assert_close(added[:used], plain[:used] + previous[:used], rtol=1e-14, atol=1e-14)
