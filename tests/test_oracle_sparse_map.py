"""Pins `oracle.moe_oracle.sparse_map` without the reference: brute force on small inputs and structural invariants
on the shapes the reference's own test uses (tests/functional/test_triton_kernels.py:255-290)."""

import pytest
import torch

from oracle import moe_oracle
from tests.helpers import REFERENCE_FIXTURES, brute_force_sparse_map


@pytest.mark.parametrize(
    ("tokens", "experts", "top_k", "pad"),
    [(1, 1, 1, 128), (7, 3, 2, 4), (64, 8, 2, 8), (100, 6, 3, 16), (33, 5, 5, 128), (50, 16, 1, 1), (200, 4, 2, 128)],
)
def test_sparse_map_matches_brute_force(tokens, experts, top_k, pad):
    generator = torch.Generator().manual_seed(tokens * 1000 + experts)
    _, top_experts = torch.topk(torch.randn(tokens, experts, generator=generator), top_k, dim=-1)
    ends, pad_begins, rows = brute_force_sparse_map(top_experts.tolist(), experts, pad)
    result = moe_oracle.sparse_map(top_experts, experts, pad)
    assert result.expert_ends.tolist() == ends
    assert result.expert_pad_begins.tolist() == pad_begins
    assert result.sparse_rows.tolist() == rows


def test_sparse_map_repeated_expert_in_a_token_is_stable():
    # Not produced by top-k, but the flattened order must still break ties: slot order inside a token.
    top_experts = torch.tensor([[1, 1], [0, 1], [1, 0]])
    ends, pad_begins, rows = brute_force_sparse_map(top_experts.tolist(), 2, 4)
    result = moe_oracle.sparse_map(top_experts, 2, 4)
    assert result.sparse_rows.tolist() == rows == [[4, 5], [0, 6], [7, 1]]
    assert result.expert_ends.tolist() == ends == [4, 8]
    assert result.expert_pad_begins.tolist() == pad_begins == [2, 8]


@pytest.mark.parametrize(("tokens", "experts", "top_k"), REFERENCE_FIXTURES["sparse_map"]["cases"])
def test_sparse_map_invariants_on_reference_shapes(tokens, experts, top_k):
    torch.manual_seed(tokens + experts + top_k)
    _, top_experts = torch.topk(torch.randn(tokens, experts), top_k, dim=-1)
    result = moe_oracle.sparse_map(top_experts, experts)
    pad = moe_oracle.MAX_DROPLESS_BLOCK_SIZE_ROW
    # Shape rules asserted by the reference's test.
    assert result.num_rows_dense == tokens and result.num_rows_unpadded == tokens * top_k
    assert result.num_rows % pad == 0 and result.num_rows > result.num_rows_unpadded
    assert result.num_rows == (tokens * top_k + experts * pad) // pad * pad
    counts = torch.bincount(top_experts.flatten(), minlength=experts)
    begins = result.expert_begins
    assert (result.expert_ends % pad == 0).all()
    assert (result.expert_pad_begins - begins == counts).all()
    assert (result.expert_ends - result.expert_pad_begins < pad).all()
    assert (result.expert_ends - result.expert_pad_begins >= 0).all()
    assert result.expert_ends[-1] <= result.num_rows
    # sparse_rows is injective into the real rows of the right expert ...
    rows = result.sparse_rows.flatten()
    assert rows.unique().numel() == rows.numel()
    flat = top_experts.flatten()
    assert (rows >= begins[flat]).all() and (rows < result.expert_pad_begins[flat]).all()
    assert result.real_row_mask().sum() == rows.numel()
    # ... and inside an expert the rows ascend with the flattened (token, slot) index.
    for e in range(experts):
        expert_rows = rows[flat == e]
        assert (expert_rows == begins[e] + torch.arange(expert_rows.numel())).all()


def test_sparse_map_dynamic_shape_and_empty_expert():
    top_experts = torch.tensor([[0, 2], [2, 0], [0, 2]])
    result = moe_oracle.sparse_map(top_experts, 4, 128, dynamic_shape=True)
    assert result.expert_ends.tolist() == [128, 128, 256, 256]
    assert result.expert_pad_begins.tolist() == [3, 128, 131, 256]
    assert result.num_rows == 256
    assert moe_oracle.sparse_map(top_experts, 4, 128).num_rows == (6 + 4 * 128) // 128 * 128
