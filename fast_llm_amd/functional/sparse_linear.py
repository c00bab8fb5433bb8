"""
The three grouped ("sparse") matrix products of the dropless MoE MLP, on gfx950 MFMA kernels.

Same names, signatures and semantics as fast_llm/functional/triton/sparse_linear.py. Operands are passed with their
strides, so transposed views (`weight.t()`, `activations.t()`) are consumed in place and never copied.
"""

import torch

from fast_llm_amd import _lib
from fast_llm_amd.functional.config import KernelConfig
from fast_llm_amd.functional.sparse_copy import SparseMap
from fast_llm_amd.functional.utils import Assert, div


def _launch(
    name: str,
    lhs: torch.Tensor,
    rhs: torch.Tensor,
    out: torch.Tensor,
    sparse_map: SparseMap | None,
    dims: tuple[int, int, int],
    accumulate: bool,
    with_pad_begins: bool = False,
) -> torch.Tensor:
    Assert.eq(lhs.dim(), 2)
    Assert.eq(rhs.dim(), 2)
    Assert.eq(out.dim(), 2)
    Assert.eq(lhs.dtype, rhs.dtype)
    if sparse_map is None:
        expert_ends = expert_pad_begins = None
        num_experts, index_dtype = 1, torch.int32
    else:
        expert_ends, expert_pad_begins = sparse_map.expert_ends, sparse_map.expert_pad_begins
        num_experts, index_dtype = sparse_map.num_experts, expert_ends.dtype
        Assert.eq(expert_ends.numel(), num_experts)
        assert expert_ends.is_contiguous()
        if with_pad_begins:
            Assert.eq(expert_pad_begins.numel(), num_experts)
            Assert.eq(expert_pad_begins.dtype, index_dtype)
            assert expert_pad_begins.is_contiguous()
    device = _lib.require_device(lhs, rhs, out, expert_ends, expert_pad_begins if with_pad_begins else None)
    pointers = [_lib.ptr(lhs.detach()), _lib.ptr(rhs.detach()), _lib.ptr(out), _lib.ptr(expert_ends)]
    if with_pad_begins:
        pointers.append(_lib.ptr(expert_pad_begins))
    # Scratch for the tile table and for splitting the last round of a launch with few, long tiles. A torch allocation
    # per call: the caching allocator hands the same block back to calls on one stream and keeps calls on different
    # streams apart, also under graph capture. Whether a product splits depends on its dimensions and this switch only.
    workspace, workspace_size = None, 0
    if KernelConfig.grouped_gemm_workspace:
        size_function = (
            _lib.lib().fm_input_row_sparse_matmul_workspace_size
            if with_pad_begins
            else _lib.lib().fm_grouped_gemm_workspace_size
        )
        workspace_size = size_function(*dims, num_experts, _lib.dtype_tag(lhs.dtype))
        if workspace_size:
            workspace = torch.empty(workspace_size, dtype=torch.uint8, device=device)
    _lib.call(
        name,
        device,
        *pointers,
        *dims,
        num_experts,
        lhs.stride(0),
        lhs.stride(1),
        rhs.stride(0),
        rhs.stride(1),
        out.stride(0),
        out.stride(1),
        int(accumulate),
        _lib.dtype_tag(lhs.dtype),
        _lib.dtype_tag(out.dtype),
        _lib.index_tag(index_dtype),
        _lib.ptr(workspace),
        workspace_size,
        label=f"{name}[{dims[0]}x{dims[1]}x{dims[2]}]",
    )
    return out


def dense_matmul(
    lhs: torch.Tensor, rhs: torch.Tensor, out: torch.Tensor | None = None, accumulate: bool = False
) -> torch.Tensor:
    """
    Standard matrix multiplication: the grouped kernel with a single group.
    Reference: fast_llm/functional/triton/sparse_linear.py:148-182.
    """
    row_dim, inner_dim = lhs.shape
    inner_dim_1, col_dim = rhs.shape
    Assert.eq(inner_dim, inner_dim_1)
    if out is None:
        assert not accumulate
        out = lhs.new_empty(row_dim, col_dim)
    return _launch("fm_output_sparse_matmul", lhs, rhs, out, None, (row_dim, col_dim, inner_dim), accumulate)


def output_sparse_matmul(
    lhs: torch.Tensor,
    rhs: torch.Tensor,
    sparse_map: SparseMap | None = None,
    out: torch.Tensor | None = None,
    accumulate: bool = False,
) -> torch.Tensor:
    """
    Output-sparse matrix multiplication with a sparse column dimension
    and a mapping row_index -> sparse_index (obtained from expert_ends).
    Ex.: MLP layer 1 forward (Y = X x W1^T), MLP layer 2 input grad (gY = gZ x W2).
    Formula: out[i, js] = sum_k(lhs[i, k] * rhs[k, jd]), where jd = js + col_sparse_dim * sparse_index[i]
      sparse_index[i] = sum(expert_ends <= i)
    Expert boundaries must be multiples of 128 rows. Rows past the last expert are not written.
    Reference: sparse_linear.py:261-307.
    """
    if sparse_map is None:
        return dense_matmul(lhs, rhs, out, accumulate)
    row_dim, inner_dim = lhs.shape
    inner_dim_1, col_dense_dim = rhs.shape
    Assert.eq(row_dim, sparse_map.num_rows)
    Assert.eq(inner_dim, inner_dim_1)
    col_sparse_dim = div(col_dense_dim, sparse_map.num_experts)
    if out is None:
        assert not accumulate
        out = lhs.new_empty(row_dim, col_sparse_dim)
    Assert.eq(tuple(out.shape), (row_dim, col_sparse_dim))
    return _launch(
        "fm_output_sparse_matmul", lhs, rhs, out, sparse_map, (row_dim, col_sparse_dim, inner_dim), accumulate
    )


def input_inner_sparse_matmul(
    lhs: torch.Tensor,
    rhs: torch.Tensor,
    sparse_map: SparseMap | None = None,
    out: torch.Tensor | None = None,
    accumulate: bool = False,
) -> torch.Tensor:
    """
    Left-input-sparse matrix multiplication with a sparse inner dimension
    and a mapping row_index -> sparse_index (obtained from expert_ends).
    Ex.: MLP layer 2 forward (Z = Y x W2^T), MLP layer 1 input grad (gX = gY x W1).
    Formula: out[i, j] = sum_ks(lhs[i, ks] * rhs[kd, j]), where kd = ks + inner_sparse_dim * sparse_index[i]
      sparse_index[i] = sum(expert_ends <= i)
    Reference: sparse_linear.py:388-434.
    """
    if sparse_map is None:
        return dense_matmul(lhs, rhs, out, accumulate)
    row_dim, inner_sparse_dim = lhs.shape
    inner_dense_dim, col_dim = rhs.shape
    Assert.eq(inner_sparse_dim, div(inner_dense_dim, sparse_map.num_experts))
    Assert.eq(row_dim, sparse_map.num_rows)
    if out is None:
        assert not accumulate
        out = lhs.new_empty(row_dim, col_dim)
    Assert.eq(tuple(out.shape), (row_dim, col_dim))
    return _launch(
        "fm_input_inner_sparse_matmul", lhs, rhs, out, sparse_map, (row_dim, col_dim, inner_sparse_dim), accumulate
    )


def input_row_sparse_matmul(
    lhs: torch.Tensor,
    rhs: torch.Tensor,
    sparse_map: SparseMap | None = None,
    out: torch.Tensor | None = None,
    accumulate: bool = False,
) -> torch.Tensor:
    """
    Left-input-sparse matrix multiplication with a sparse row dimension
    and a mapping inner_index -> sparse_index.
    Ex.: MLP layer 1 weight grad (gW1 = gY^T x X), MLP layer 2 weight grad (gW2^T = Y^T x gZ).
    Formula: out[id, j] = sum_ks(lhs[is, ks] * rhs[ks, j]), where
      sparse_begin[sparse_index[id]] <= ks < sparse_end[sparse_index[id]],
      id = is + row_sparse_dim * sparse_index[id],
      sparse_index[id] = id // row_sparse_dim
    Padding rows are replaced by zeros before the product, whatever they hold. `out` may have a wider dtype than the
    operands (fp32 gradient buffers). Reference: sparse_linear.py:520-570.
    """
    if sparse_map is None:
        return dense_matmul(lhs, rhs, out, accumulate)
    row_sparse_dim, inner_dim = lhs.shape
    inner_dim_1, col_dim = rhs.shape
    Assert.eq(inner_dim, inner_dim_1)
    Assert.eq(inner_dim, sparse_map.num_rows)
    row_dense_dim = row_sparse_dim * sparse_map.num_experts
    if out is None:
        assert not accumulate
        out = lhs.new_empty(row_dense_dim, col_dim)
    Assert.eq(tuple(out.shape), (row_dense_dim, col_dim))
    return _launch(
        "fm_input_row_sparse_matmul",
        lhs,
        rhs,
        out,
        sparse_map,
        (row_sparse_dim, col_dim, inner_dim),
        accumulate,
        with_pad_begins=True,
    )


class OutputSparseLinear(torch.autograd.Function):
    """Reference: sparse_linear.py:573-586."""

    @staticmethod
    def forward(ctx, lhs: torch.Tensor, rhs: torch.Tensor, sparse_map: SparseMap):  # noqa
        ctx.sparse_map = sparse_map
        ctx.save_for_backward(lhs, rhs)
        return output_sparse_matmul(lhs, rhs, sparse_map)

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, None]:  # noqa
        grad_out = grad_out.contiguous()
        lhs, rhs = ctx.saved_tensors
        grad_lhs = input_inner_sparse_matmul(grad_out, rhs.t(), ctx.sparse_map)
        grad_rhs = input_row_sparse_matmul(grad_out.t(), lhs, ctx.sparse_map).t()
        return grad_lhs, grad_rhs, None


output_sparse_linear_autograd = OutputSparseLinear.apply


class InputSparseLinear(torch.autograd.Function):
    """Reference: sparse_linear.py:592-605."""

    @staticmethod
    def forward(ctx, lhs: torch.Tensor, rhs: torch.Tensor, sparse_map: SparseMap):  # noqa
        ctx.sparse_map = sparse_map
        ctx.save_for_backward(lhs, rhs)
        return input_inner_sparse_matmul(lhs, rhs, sparse_map)

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, None]:  # noqa
        grad_out = grad_out.contiguous()
        lhs, rhs = ctx.saved_tensors
        grad_lhs = output_sparse_matmul(grad_out, rhs.t(), ctx.sparse_map)
        grad_rhs = input_row_sparse_matmul(lhs.t(), grad_out, ctx.sparse_map)
        return grad_lhs, grad_rhs, None


input_sparse_linear_autograd = InputSparseLinear.apply
