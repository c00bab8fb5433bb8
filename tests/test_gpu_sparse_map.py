"""Sparse map on the GPU, through the C ABI, bit-exact against the oracle."""

import pytest
import torch

from fast_llm_amd.functional.config import MAX_DROPLESS_BLOCK_SIZE_ROW
from fast_llm_amd.functional.sparse_copy import get_sparse_map
from fast_llm_amd.workloads import WORKLOADS, make_inputs
from oracle import moe_oracle
from tests.helpers import REFERENCE_FIXTURES, brute_force_sparse_map

pytestmark = pytest.mark.gpu


def _assert_same_map(actual, expected):
    for name in ("num_rows_dense", "num_rows", "num_rows_unpadded", "num_experts", "num_experts_per_token"):
        assert getattr(actual, name) == getattr(expected, name), name
    for name in ("expert_ends", "expert_pad_begins", "sparse_rows"):
        ours, theirs = getattr(actual, name).cpu().to(torch.int64), getattr(expected, name)
        assert ours.shape == theirs.shape, name
        assert torch.equal(ours, theirs), f"{name}: {(ours != theirs).sum().item()} mismatches"


@pytest.mark.parametrize(("tokens", "experts", "top_k"), REFERENCE_FIXTURES["sparse_map"]["cases"])
def test_reference_shapes(tokens, experts, top_k, device):
    """The cases of the reference's test (tests/functional/test_triton_kernels.py:255-290)."""
    torch.manual_seed(tokens * 7 + experts)
    _, top_experts = torch.topk(torch.randn(tokens, experts), top_k, dim=-1)
    actual = get_sparse_map(top_experts.to(device), experts)
    _assert_same_map(actual, moe_oracle.sparse_map(top_experts, experts))
    assert actual.num_rows % MAX_DROPLESS_BLOCK_SIZE_ROW == 0 and actual.num_rows > actual.num_rows_unpadded
    assert actual.sparse_rows.dtype == (torch.int16 if actual.num_rows < 32768 else torch.int32)
    assert actual.expert_ends.dtype == actual.expert_pad_begins.dtype == actual.sparse_rows.dtype


@pytest.mark.parametrize("name", list(WORKLOADS))
def test_benchmark_configurations(name, device):
    inputs = make_inputs(WORKLOADS[name], seed=1, weights=False)
    workload = WORKLOADS[name]
    actual = get_sparse_map(inputs.top_experts.to(device), workload.experts)
    _assert_same_map(actual, moe_oracle.sparse_map(inputs.top_experts, workload.experts))
    expected_dtype = torch.int16 if name in ("tiny", "mixtral", "imbalanced") else torch.int32
    assert actual.sparse_rows.dtype == expected_dtype


@pytest.mark.parametrize(
    ("tokens", "experts", "top_k", "pad"),
    [(1, 1, 1, 128), (1, 8, 8, 128), (3, 2, 1, 1), (1025, 3, 2, 64), (4096, 1, 1, 128), (777, 130, 5, 32),
     (300, 1024, 4, 8), (64, 1000, 64, 16), (100000, 7, 3, 128)],
)
def test_edge_shapes(tokens, experts, top_k, pad, device):
    torch.manual_seed(tokens + experts)
    _, top_experts = torch.topk(torch.randn(tokens, experts), top_k, dim=-1)
    actual = get_sparse_map(top_experts.to(device), experts, pad_to_multiple=pad)
    _assert_same_map(actual, moe_oracle.sparse_map(top_experts, experts, pad))


def test_empty_experts_skew_and_repeats(device):
    # All tokens on two experts of sixteen, the rest empty; an expert repeated inside a token; int32 input.
    top_experts = torch.tensor([[3, 3], [9, 3], [3, 9]] * 500)
    ends, pad_begins, rows = brute_force_sparse_map(top_experts.tolist(), 16, 128)
    actual = get_sparse_map(top_experts.to(device=device, dtype=torch.int32), 16)
    assert actual.expert_ends.tolist() == ends
    assert actual.expert_pad_begins.tolist() == pad_begins
    assert actual.sparse_rows.tolist() == rows


def test_dynamic_shape_and_determinism(device):
    inputs = make_inputs(WORKLOADS["wide"], seed=2, weights=False)
    top_experts = inputs.top_experts.to(device)
    first = get_sparse_map(top_experts, 128, dynamic_shape=True)
    expected = moe_oracle.sparse_map(inputs.top_experts, 128, dynamic_shape=True)
    assert first.num_rows == expected.num_rows == int(expected.expert_ends[-1])
    for _ in range(3):
        again = get_sparse_map(top_experts, 128, dynamic_shape=True)
        assert torch.equal(again.sparse_rows, first.sparse_rows)
        assert torch.equal(again.expert_ends, first.expert_ends)


def test_out_of_range_experts_are_dropped_not_written_out_of_bounds(device):
    top_experts = torch.tensor([[0, 5], [-1, 1], [1, 7], [2, 0]])
    actual = get_sparse_map(top_experts.to(device), 3, pad_to_multiple=4)
    assert actual.sparse_rows.tolist() == [[0, -1], [-1, 4], [5, -1], [8, 1]]
    assert actual.expert_ends.tolist() == [4, 8, 12]
    assert actual.expert_pad_begins.tolist() == [2, 6, 9]


def test_too_many_experts_is_an_error(device):
    with pytest.raises(ValueError, match="num_experts"):
        get_sparse_map(torch.zeros(4, 1, dtype=torch.int64, device=device), 4096)
