"""Shared helpers of the test-suite: fixtures the reference's tests hold, comparison metrics, brute-force checkers."""

import json
import pathlib

import torch

from oracle import moe_oracle

GOLDEN = pathlib.Path(__file__).resolve().parent / "golden"
REFERENCE_FIXTURES = json.loads((GOLDEN / "reference_fixtures.json").read_text())


def rms_diff(x: torch.Tensor, y: torch.Tensor) -> float:
    """The reference's comparison metric (fast_llm/utils.py:70-73)."""
    return (torch.norm(x.double() - y.double(), 2) / x.numel() ** 0.5).item()


def max_rel_err(x: torch.Tensor, y: torch.Tensor) -> float:
    """max|x - y| / max|y|: the parity metric of the benchmark configurations."""
    scale = y.double().abs().max().item()
    diff = (x.double() - y.double()).abs().max().item()
    return diff / scale if scale > 0 else diff


def rel_rms_err(x: torch.Tensor, y: torch.Tensor) -> float:
    """||x - y|| / ||y||: the relative RMS error of the reference's benchmark runner
    (tools/benchmark/triton_kernels/runner.py:305-312)."""
    scale = torch.norm(y.double(), 2).item()
    diff = torch.norm(x.double() - y.double(), 2).item()
    return diff / scale if scale > 0 else diff


def max_block_rel_err(x: torch.Tensor, y: torch.Tensor, block_rows: int = 256, block_columns: int = 256) -> float:
    """max over blocks (the size of a kernel tile) of max|x - y| in the block / max|y| in the block: a wrong tile of
    small values cannot hide behind a large value elsewhere in the tensor. A block where y is all zero counts its
    absolute error. Runs on the tensors' device."""
    assert x.shape == y.shape and x.dim() == 2
    rows, columns = x.shape
    padded_rows, padded_columns = -(-rows // block_rows) * block_rows, -(-columns // block_columns) * block_columns

    def block_max(t: torch.Tensor) -> torch.Tensor:
        padded = torch.zeros(padded_rows, padded_columns, dtype=torch.float32, device=t.device)
        padded[:rows, :columns] = t
        return padded.view(padded_rows // block_rows, block_rows, padded_columns // block_columns, block_columns).amax(dim=(1, 3))

    diff = block_max((x.float() - y.float()).abs())
    scale = block_max(y.float().abs())
    return torch.where(scale > 0, diff / scale.clamp_min(1e-30), diff).max().item()


def fixture_sparse_map(case: dict, dtype: torch.dtype = torch.int64) -> moe_oracle.OracleSparseMap:
    """The hand-built map of the reference's sparse-matmul tests (tests/functional/test_sparse_matmul.py:51-62):
    only expert_ends, expert_pad_begins, num_rows and num_experts are set."""
    ends = list(case["expert_ends"])
    begins = [0] + ends[:-1]
    pad_begins = [begin + tokens for begin, tokens in zip(begins, case["tokens_per_expert"])]
    return moe_oracle.OracleSparseMap(
        sparse_rows=None,
        expert_ends=torch.tensor(ends, dtype=dtype),
        expert_pad_begins=torch.tensor(pad_begins, dtype=dtype),
        num_rows_dense=None,
        num_rows=ends[-1],
        num_rows_unpadded=None,
        num_experts=len(ends),
        num_experts_per_token=None,
    )


def to_device_map(oracle_map, device, index_dtype: torch.dtype | None = None):
    """An oracle map as the product's `SparseMap` on `device`."""
    from fast_llm_amd.functional.sparse_copy import SparseMap

    def move(tensor):
        if tensor is None:
            return None
        return tensor.to(device=device, dtype=index_dtype or tensor.dtype)

    return SparseMap(
        sparse_rows=move(oracle_map.sparse_rows),
        expert_ends=move(oracle_map.expert_ends),
        expert_pad_begins=move(oracle_map.expert_pad_begins),
        num_rows_dense=oracle_map.num_rows_dense,
        num_rows=oracle_map.num_rows,
        num_rows_unpadded=oracle_map.num_rows_unpadded,
        num_experts=oracle_map.num_experts,
        num_experts_per_token=oracle_map.num_experts_per_token,
    )


def brute_force_sparse_map(top_experts: list[list[int]], num_experts: int, pad: int):
    """O(M * E) pure-python statement of the map: count, pad, prefix, then rank by scanning all earlier entries."""
    flat = [expert for row in top_experts for expert in row]
    counts = [sum(1 for expert in flat if expert == e) for e in range(num_experts)]
    padded = [-(-count // pad) * pad for count in counts]
    ends, total = [], 0
    for value in padded:
        total += value
        ends.append(total)
    begins = [end - value for end, value in zip(ends, padded)]
    pad_begins = [begin + count for begin, count in zip(begins, counts)]
    rows = []
    for i, expert in enumerate(flat):
        earlier = sum(1 for other in flat[:i] if other == expert)
        rows.append(begins[expert] + earlier)
    k = len(top_experts[0]) if top_experts else 0
    return ends, pad_begins, [rows[i * k : (i + 1) * k] for i in range(len(top_experts))]
