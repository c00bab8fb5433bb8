"""
Sparse map and the dense <-> sparse copies of the dropless MoE, on HIP kernels.

Same names, signatures and semantics as the reference module fast_llm/functional/triton/sparse_copy.py; each function
cites the reference lines it stands in for. Every function launches kernels of `libfastmoe_hip.so` on the current
stream of the tensors' device and allocates its outputs with torch.
"""

import dataclasses

import torch

from fast_llm_amd import _lib
from fast_llm_amd.functional.config import MAX_DROPLESS_BLOCK_SIZE_ROW, KernelConfig
from fast_llm_amd.functional.utils import Assert, wrap_forward_backward


@dataclasses.dataclass()
class SparseMap:
    """Reference: fast_llm/functional/triton/sparse_copy.py:10-24."""

    sparse_rows: torch.Tensor
    # The end row for each expert, including padding. `expert_ends[i] = expert_begins[i] + padded_tokens_per_expert[i]`
    expert_ends: torch.Tensor
    # The end row for each expert, excluding padding. `expert_pad_begins[i] = expert_begins[i] + tokens_per_expert[i]`
    expert_pad_begins: torch.Tensor
    # The number of rows in the dense tensor, i.e., the number of tokens.
    num_rows_dense: int
    # The number of sparse rows, including padding (a worst-case static bound unless `dynamic_shape`).
    num_rows: int
    # The number of sparse rows, excluding padding. `num_rows_unpadded = num_rows_dense * num_experts_per_token`
    num_rows_unpadded: int
    num_experts: int
    num_experts_per_token: int


def get_sparse_map(
    top_experts: torch.Tensor,
    num_experts: int,
    *,
    dynamic_shape: bool = False,
    pad_to_multiple: int = MAX_DROPLESS_BLOCK_SIZE_ROW,
    block_size=KernelConfig.POINTWISE_BLOCK_SIZE,
    use_triton: bool | None = None,
    router_counts=None,
) -> SparseMap:
    """
    Expert histogram, padded expert offsets and the stable sparse row of every (token, slot).
    Reference: fast_llm/functional/triton/sparse_copy.py:258-301 (`block_size` is a Triton launch parameter there and
    has no effect here; `use_triton=False` selects the reference's torch path, which this package does not have).
    `router_counts` (not in the reference's signature): the `RouterCounts` that `functional.routing.router` returned
    together with these very `top_experts`; the map is then built from the router's counts, without the pass that
    counts `top_experts`. Same result. Counts that belong to another tensor, or to one modified in place since the
    routing (masking, capacity or dropping hooks), are not used: the map then counts `top_experts` itself.
    """
    KernelConfig.enabled(top_experts.device, use_triton)
    Assert.eq(top_experts.dim(), 2)
    device = _lib.require_device(top_experts)
    num_rows_dense, num_experts_per_token = top_experts.shape
    num_rows_unpadded = num_rows_dense * num_experts_per_token
    max_rows = (num_rows_unpadded + num_experts * pad_to_multiple) // pad_to_multiple * pad_to_multiple
    dtype = torch.int16 if max_rows < 32768 else torch.int32

    if router_counts is not None and not router_counts.describes(top_experts):
        router_counts = None
    top_experts = top_experts.to(torch.int64).contiguous()
    sparse_rows = torch.empty((num_rows_dense, num_experts_per_token), dtype=dtype, device=device)
    expert_ends = torch.empty(num_experts, dtype=dtype, device=device)
    expert_pad_begins = torch.empty(num_experts, dtype=dtype, device=device)
    library = _lib.lib()
    if router_counts is not None:
        Assert.eq(router_counts.tokens, num_rows_dense)
        Assert.eq(router_counts.shared_experts + router_counts.experts_per_token, num_experts_per_token)
        Assert.eq(router_counts.shared_experts + router_counts.routed_experts, num_experts)
        _lib.require_device(top_experts, router_counts.workspace)
        workspace_size = library.fm_sparse_map_from_router_workspace_size(num_rows_dense, num_experts)
        workspace = torch.empty(workspace_size, dtype=torch.uint8, device=device)
        _lib.call(
            "fm_sparse_map_from_router",
            device,
            _lib.ptr(top_experts),
            _lib.ptr(router_counts.workspace),
            router_counts.workspace.numel() * router_counts.workspace.element_size(),
            num_rows_dense,
            num_experts,
            router_counts.experts_per_token,
            router_counts.shared_experts,
            pad_to_multiple,
            _lib.index_tag(dtype),
            _lib.ptr(sparse_rows),
            _lib.ptr(expert_ends),
            _lib.ptr(expert_pad_begins),
            _lib.ptr(workspace),
            workspace_size,
        )
        return _finish_sparse_map(
            sparse_rows, expert_ends, expert_pad_begins, num_experts, dynamic_shape, max_rows
        )
    workspace_size = library.fm_sparse_map_workspace_size(num_rows_dense, num_experts_per_token, num_experts)
    workspace = torch.empty(workspace_size, dtype=torch.uint8, device=device)
    _lib.call(
        "fm_sparse_map",
        device,
        _lib.ptr(top_experts),
        num_rows_dense,
        num_experts_per_token,
        num_experts,
        pad_to_multiple,
        _lib.index_tag(dtype),
        _lib.ptr(sparse_rows),
        _lib.ptr(expert_ends),
        _lib.ptr(expert_pad_begins),
        _lib.ptr(workspace),
        workspace_size,
    )
    return _finish_sparse_map(sparse_rows, expert_ends, expert_pad_begins, num_experts, dynamic_shape, max_rows)


def _finish_sparse_map(
    sparse_rows: torch.Tensor,
    expert_ends: torch.Tensor,
    expert_pad_begins: torch.Tensor,
    num_experts: int,
    dynamic_shape: bool,
    max_rows: int,
) -> SparseMap:
    num_rows_dense, num_experts_per_token = sparse_rows.shape
    return SparseMap(
        sparse_rows=sparse_rows,
        expert_ends=expert_ends,
        expert_pad_begins=expert_pad_begins,
        num_rows_dense=num_rows_dense,
        num_rows=expert_ends[-1].item() if dynamic_shape else max_rows,
        num_rows_unpadded=num_rows_dense * num_experts_per_token,
        num_experts=num_experts,
        num_experts_per_token=num_experts_per_token,
    )


def _copy_arguments(dense: torch.Tensor, sparse: torch.Tensor, scores: torch.Tensor | None, sparse_map: SparseMap):
    Assert.eq(dense.dim(), 2)
    Assert.eq(sparse.dim(), 2)
    Assert.eq(dense.size(0), sparse_map.num_rows_dense)
    Assert.eq(dense.size(1), sparse.size(1))
    Assert.eq(sparse.size(0), sparse_map.num_rows)
    Assert.eq(dense.dtype, sparse.dtype)
    Assert.eq(tuple(sparse_map.sparse_rows.shape), (sparse_map.num_rows_dense, sparse_map.num_experts_per_token))
    assert dense.is_contiguous() and sparse.is_contiguous() and sparse_map.sparse_rows.is_contiguous()
    if scores is not None:
        Assert.eq(tuple(scores.shape), tuple(sparse_map.sparse_rows.shape))
        assert scores.is_contiguous()
    return (
        sparse_map.num_rows_dense,
        dense.size(1),
        sparse_map.num_experts_per_token,
        sparse.size(0),
        _lib.dtype_tag(dense.dtype),
        _lib.dtype_tag(torch.float32 if scores is None else scores.dtype),
        _lib.index_tag(sparse_map.sparse_rows.dtype),
    )


def copy_dense_to_sparse(input_: torch.Tensor, scores: torch.Tensor | None, sparse_map: SparseMap) -> torch.Tensor:
    """
    output[sparse_row[dense_row, :]] = input_[dense_row, None] * (score[dense_row, :] or 1)
    Padding rows of the output stay uninitialised. Reference: sparse_copy.py:52-66.
    """
    device = _lib.require_device(input_, scores, sparse_map.sparse_rows)
    # A worst-case static shape.
    out = input_.new_empty((sparse_map.num_rows, input_.size(1)))
    shape = _copy_arguments(input_, out, scores, sparse_map)
    _lib.call(
        "fm_copy_dense_to_sparse",
        device,
        _lib.ptr(input_),
        _lib.ptr(scores),
        _lib.ptr(sparse_map.sparse_rows),
        _lib.ptr(out),
        *shape[:4],
        shape[4],
        shape[5],
        shape[6],
    )
    return out


def copy_sparse_to_dense(input_: torch.Tensor, scores: torch.Tensor | None, sparse_map: SparseMap) -> torch.Tensor:
    """
    output[dense_row] = (input_[sparse_row[dense_row, :]] * (score[dense_row, :] or 1)).sum(1)
    Reference: sparse_copy.py:93-108.
    """
    device = _lib.require_device(input_, scores, sparse_map.sparse_rows)
    out = input_.new_empty((sparse_map.num_rows_dense, input_.size(1)))
    shape = _copy_arguments(out, input_, scores, sparse_map)
    _lib.call(
        "fm_copy_sparse_to_dense",
        device,
        _lib.ptr(input_),
        _lib.ptr(scores),
        _lib.ptr(sparse_map.sparse_rows),
        _lib.ptr(out),
        *shape[:4],
        shape[4],
        shape[5],
        shape[6],
    )
    return out


def copy_sparse_to_dense_grad_score(
    input_: torch.Tensor, grad_output: torch.Tensor, sparse_map: SparseMap
) -> torch.Tensor:
    """
    grad_scores[dense_row, top_index] = (input_[sparse_row[dense_row, top_index]] * grad_output[dense_row]).sum()
    The result has the dtype of `input_`, as in the reference (sparse_copy.py:151-165).
    """
    device = _lib.require_device(input_, grad_output, sparse_map.sparse_rows)
    out = input_.new_empty(sparse_map.num_rows_dense, sparse_map.num_experts_per_token)
    shape = _copy_arguments(grad_output, input_, None, sparse_map)
    _lib.call(
        "fm_copy_sparse_to_dense_grad_score",
        device,
        _lib.ptr(input_),
        _lib.ptr(grad_output),
        _lib.ptr(sparse_map.sparse_rows),
        _lib.ptr(out),
        *shape[:4],
        shape[4],
        _lib.dtype_tag(out.dtype),
        shape[6],
    )
    return out


def copy_dense_to_sparse_forward(
    input_: torch.Tensor, sparse_map: SparseMap
) -> tuple[torch.Tensor, tuple[SparseMap, tuple[int, ...]]]:
    """Reference: sparse_copy.py:168-171."""
    return copy_dense_to_sparse(input_.flatten(0, -2), None, sparse_map), (sparse_map, input_.shape)


def copy_dense_to_sparse_backward(
    grad_output: torch.Tensor, context: tuple[SparseMap, tuple[int, ...]]
) -> torch.Tensor:
    """Reference: sparse_copy.py:174-178."""
    sparse_map, input_shape = context
    return copy_sparse_to_dense(grad_output.contiguous(), None, sparse_map).view(input_shape)


copy_dense_to_sparse_autograd = wrap_forward_backward(copy_dense_to_sparse_forward, copy_dense_to_sparse_backward)


def copy_sparse_to_dense_forward(
    input_: torch.Tensor, scores: torch.Tensor, sparse_map: SparseMap
) -> tuple[torch.Tensor, tuple[SparseMap, torch.Tensor, torch.Tensor]]:
    """Reference: sparse_copy.py:184-187."""
    return copy_sparse_to_dense(input_, scores, sparse_map), (sparse_map, input_, scores)


def copy_sparse_to_dense_backward(grad_output: torch.Tensor, context: tuple[SparseMap, torch.Tensor, torch.Tensor]):
    """
    grad_input = copy_dense_to_sparse(grad_output, scores), grad_scores = copy_sparse_to_dense_grad_score(input_,
    grad_output), computed by one kernel that reads `grad_output` once. Reference: sparse_copy.py:190-194.
    """
    sparse_map, input_, scores = context
    device = _lib.require_device(input_, grad_output, scores, sparse_map.sparse_rows)
    grad_output = grad_output.contiguous()
    grad_input = grad_output.new_empty((sparse_map.num_rows, grad_output.size(1)))
    grad_scores = input_.new_empty(sparse_map.num_rows_dense, sparse_map.num_experts_per_token)
    shape = _copy_arguments(grad_output, input_, scores, sparse_map)
    Assert.eq(input_.shape, grad_input.shape)
    _lib.call(
        "fm_copy_sparse_to_dense_backward",
        device,
        _lib.ptr(input_),
        _lib.ptr(grad_output),
        _lib.ptr(scores),
        _lib.ptr(sparse_map.sparse_rows),
        _lib.ptr(grad_input),
        _lib.ptr(grad_scores),
        *shape[:4],
        shape[4],
        shape[5],
        _lib.dtype_tag(grad_scores.dtype),
        shape[6],
    )
    return grad_input, grad_scores


copy_sparse_to_dense_autograd = wrap_forward_backward(copy_sparse_to_dense_forward, copy_sparse_to_dense_backward)
