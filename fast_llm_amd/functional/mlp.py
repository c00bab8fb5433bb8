"""
The MoE MLP: gated activation kernels and the forward/backward orchestration with activation recomputation.

Same names, positional signatures and recompute semantics as fast_llm/functional/triton/mlp.py, single GPU
(`group` must be None, `sequence_parallel` False). Weight gradients are side effects into `weight.grad_buffer`.
"""

import typing

import torch

from fast_llm_amd import _lib
from fast_llm_amd.functional.config import ActivationType, KernelConfig, MLPRecomputeLevel
from fast_llm_amd.functional.linear import (
    input_parallel_linear_forward,
    maybe_transpose,
    output_parallel_linear_backward,
    output_parallel_linear_forward,
    update_linear_gradients,
)
from fast_llm_amd.functional.sparse_copy import (
    SparseMap,
    copy_dense_to_sparse_backward,
    copy_dense_to_sparse_forward,
    copy_sparse_to_dense_backward,
    copy_sparse_to_dense_forward,
)
from fast_llm_amd.functional.sparse_linear import output_sparse_matmul
from fast_llm_amd.functional.utils import wrap_forward_backward


def _activation_tag(activation_type: ActivationType | str) -> int:
    name = str(activation_type.value if isinstance(activation_type, ActivationType) else activation_type)
    if name not in _lib.ACTIVATIONS:
        # Same set as the reference's kernels (fast_llm/functional/triton/mlp.py:49-67 has no sigmoid either).
        raise NotImplementedError(f"activation `{name}` has no kernel")
    return _lib.ACTIVATIONS[name]


def _row_limit(sparse_map: SparseMap | None, tensor: torch.Tensor) -> tuple[int | None, int]:
    """(device address of the number of rows in use, its index tag) for a [num_rows, ...] buffer of `sparse_map`: the
    last entry of `expert_ends`. The rows after it belong to no expert and need not be streamed through."""
    if sparse_map is None or tensor.dim() != 2 or tensor.size(0) != sparse_map.num_rows:
        return None, 0
    ends = sparse_map.expert_ends
    return ends.data_ptr() + (ends.numel() - 1) * ends.element_size(), _lib.index_tag(ends.dtype)


def mlp_activation_forward(
    input_: torch.Tensor, gated: bool, activation_type: ActivationType, sparse_map: SparseMap | None = None
):
    """
    out = act(input_[..., :n]) * input_[..., n:] if gated else act(input_).
    Reference: `triton_mlp_activation_forward`, fast_llm/functional/triton/mlp.py:142-162. With `sparse_map` (not in
    the reference's signature) the rows past the last expert's end are skipped instead of computed from garbage.
    """
    assert input_.is_contiguous()
    device = _lib.require_device(input_)
    n_cols = input_.size(-1) // (2 if gated else 1)
    output = input_.new_empty(input_.shape[:-1] + (n_cols,))
    _lib.call(
        "fm_mlp_activation_forward",
        device,
        _lib.ptr(input_.detach()),
        _lib.ptr(output),
        output.numel() // n_cols if n_cols else 0,
        n_cols,
        int(gated),
        _activation_tag(activation_type),
        _lib.dtype_tag(input_.dtype),
        *_row_limit(sparse_map, input_),
    )
    return output, (input_, gated, activation_type, sparse_map)


def mlp_activation_backward(grad_output: torch.Tensor, context: tuple, recompute: bool = False):
    """
    Input gradient of the activation, optionally with the recomputed forward output.
    Reference: `triton_mlp_activation_backward`, fast_llm/functional/triton/mlp.py:165-190.
    """
    assert grad_output.is_contiguous()
    input_, gated, activation_type, *rest = context
    sparse_map = rest[0] if rest else None
    device = _lib.require_device(input_, grad_output)
    grad_input = torch.empty_like(input_)
    output = torch.empty_like(grad_output) if recompute else None
    n_cols = grad_output.size(-1)
    _lib.call(
        "fm_mlp_activation_backward",
        device,
        _lib.ptr(grad_output),
        _lib.ptr(grad_input),
        _lib.ptr(input_.detach()),
        _lib.ptr(output),
        grad_output.numel() // n_cols if n_cols else 0,
        n_cols,
        int(gated),
        _activation_tag(activation_type),
        _lib.dtype_tag(input_.dtype),
        *_row_limit(sparse_map, input_),
    )
    return grad_input, output


mlp_activation_autograd = wrap_forward_backward(mlp_activation_forward, mlp_activation_backward)

# The reference's names for the same three functions.
triton_mlp_activation_forward = mlp_activation_forward
triton_mlp_activation_backward = mlp_activation_backward
triton_mlp_activation_autograd = mlp_activation_autograd


def torch_mlp_activation(input_: torch.Tensor, gated: bool, activation_type: ActivationType) -> torch.Tensor:
    """Plain torch statement of the activation (reference: fast_llm/functional/triton/mlp.py:195-204)."""
    if gated:
        x1, x2 = input_.chunk(2, dim=-1)
        return activation_type.activation_fn(x1) * x2
    return activation_type.activation_fn(input_)


def _fusable(lhs: torch.Tensor, weight_t: torch.Tensor, gated: bool, sparse_map: SparseMap | None, *biases) -> bool:
    """Whether a layer-1 product / layer-2 input gradient may take the kernel with the gated activation in its
    epilogue; the library has the last word (`NotImplementedError`: shapes it cannot tile)."""
    return (
        gated
        and sparse_map is not None
        and all(bias is None for bias in biases)
        and lhs.dtype in (torch.bfloat16, torch.float16)
        and weight_t.dtype == lhs.dtype
        and lhs.dim() == 2
        and lhs.stride(1) == 1
        and weight_t.stride(0) == 1
    )


def _launch_fused(name: str, lhs: torch.Tensor, weight_t: torch.Tensor, tensors: tuple, sparse_map: SparseMap,
                  activation_dim: int, activation_type: ActivationType, label_columns: int) -> None:  # fmt: skip
    device = _lib.require_device(lhs, weight_t, *tensors)
    _lib.call(
        name,
        device,
        _lib.ptr(lhs.detach()),
        _lib.ptr(weight_t.detach()),
        *(_lib.ptr(tensor) for tensor in tensors),
        _lib.ptr(sparse_map.expert_ends),
        lhs.size(0),
        activation_dim,
        lhs.size(1),
        sparse_map.num_experts,
        lhs.stride(0),
        lhs.stride(1),
        weight_t.stride(0),
        weight_t.stride(1),
        _activation_tag(activation_type),
        _lib.dtype_tag(lhs.dtype),
        _lib.index_tag(sparse_map.expert_ends.dtype),
        label=f"{name}[{lhs.size(0)}x{label_columns}x{lhs.size(1)}]",
    )


def gated_layer_1_forward(
    input_: torch.Tensor, weight_1: torch.Tensor, sparse_map: SparseMap, activation_type: ActivationType, keep_layer_1: bool
) -> tuple[torch.Tensor | None, torch.Tensor]:
    """
    (layer-1 output or None, activation output) of a gated sparse MLP in one kernel: `output_sparse_matmul` with
    `triton_mlp_activation_forward` in its epilogue (reference: the two calls at fast_llm/functional/triton/mlp.py:246-258).
    Bit-identical to the two separate kernels. Raises NotImplementedError for shapes the fused kernel does not take.
    """
    activation_dim = weight_1.size(0) // sparse_map.num_experts // 2
    layer_1 = input_.new_empty(input_.size(0), 2 * activation_dim) if keep_layer_1 else None
    output = input_.new_empty(input_.size(0), activation_dim)
    _launch_fused(
        "fm_output_sparse_matmul_gated_activation", input_, weight_1.t(), (layer_1, output), sparse_map,
        activation_dim, activation_type, 2 * activation_dim,
    )  # fmt: skip
    return layer_1, output


def gated_layer_2_input_backward(
    grad_output: torch.Tensor, weight_2_t: torch.Tensor, sparse_map: SparseMap, layer_1: torch.Tensor,
    activation_type: ActivationType, recompute: bool,
) -> tuple[torch.Tensor, torch.Tensor | None]:  # fmt: skip
    """
    (gradient of the layer-1 output, recomputed activation output or None): the layer-2 input gradient
    `output_sparse_matmul(grad_output, weight_2_t)` handed tile by tile to `triton_mlp_activation_backward` instead
    of being stored (reference: fast_llm/functional/triton/mlp.py:352-359, 373-375). Bit-identical to the two kernels.
    """
    assert layer_1.is_contiguous()
    activation_dim = layer_1.size(1) // 2
    grad_layer_1 = torch.empty_like(layer_1)
    output = layer_1.new_empty(layer_1.size(0), activation_dim) if recompute else None
    _launch_fused(
        "fm_output_sparse_matmul_gated_activation_backward", grad_output, weight_2_t,
        (layer_1.detach(), grad_layer_1, output), sparse_map, activation_dim, activation_type, activation_dim,
    )  # fmt: skip
    return grad_layer_1, output


def mlp_forward(
    input_: torch.Tensor,
    scores: torch.Tensor | None,
    weight_1: torch.Tensor,
    bias_1: torch.Tensor | None,
    weight_2: torch.Tensor,
    bias_2: torch.Tensor | None,
    gated: bool,
    activation_type: ActivationType,
    group: typing.Any,
    sequence_parallel: bool,
    training: bool = True,
    recompute_level: MLPRecomputeLevel = MLPRecomputeLevel.none,
    transposed_layer_2_weight: bool = False,
    sparse_map: SparseMap | None = None,
    use_triton: bool | None = None,
) -> tuple[torch.Tensor, list[typing.Any] | None]:
    """
    dispatch -> layer 1 -> activation -> layer 2 -> combine. Returns the output and the context list for
    `mlp_backward`; `recompute_level` decides which intermediates the context keeps.
    Reference: fast_llm/functional/triton/mlp.py:207-311.
    """
    if group is not None or sequence_parallel:
        raise NotImplementedError("tensor/sequence parallelism is not part of this single-GPU path")
    KernelConfig.enabled(input_.device, use_triton)

    # Sparse copy
    input_shape = input_.shape
    intermediate_0 = input_ if sparse_map is None else copy_dense_to_sparse_forward(input_, sparse_map)[0]

    # Layer 1 and activation: one kernel where the library has one, else the reference's two steps.
    intermediate_2 = None
    if KernelConfig.fuse_activation and _fusable(intermediate_0, weight_1.t(), gated, sparse_map, bias_1):
        try:
            intermediate_1, intermediate_2 = gated_layer_1_forward(
                intermediate_0, weight_1, sparse_map, activation_type, training and not recompute_level.recompute_layer_1
            )
        except NotImplementedError:
            pass
    if intermediate_2 is None:
        intermediate_1, _ = output_parallel_linear_forward(
            intermediate_0, weight_1, bias_1, group, False, False, True, sparse_map
        )
        intermediate_2, _ = mlp_activation_forward(intermediate_1, gated, activation_type, sparse_map)

    if recompute_level.recompute_sparse_input:
        intermediate_0 = None
    else:
        input_ = None
    if recompute_level.recompute_layer_1:
        intermediate_1 = None

    # Layer 2
    intermediate_3, _ = input_parallel_linear_forward(
        intermediate_2, weight_2, bias_2, group, False, transposed_layer_2_weight, True, sparse_map
    )

    # Context
    if recompute_level.recompute_activation or not training:
        intermediate_2 = None

    # Sparse copy
    if sparse_map is None:
        output = intermediate_3
        intermediate_3 = None
    else:
        output, _ = copy_sparse_to_dense_forward(intermediate_3, scores, sparse_map)

    context = (
        [
            input_,
            scores,
            intermediate_0,
            intermediate_1,
            intermediate_2,
            intermediate_3,
            weight_1,
            bias_1,
            weight_2,
            bias_2,
            gated,
            activation_type,
            group,
            sequence_parallel,
            transposed_layer_2_weight,
            sparse_map,
            input_shape,
            use_triton,
        ]
        if training
        else None
    )
    return output, context


def mlp_backward(grad_output: torch.Tensor, context: list[typing.Any]) -> tuple[torch.Tensor, torch.Tensor]:
    """
    Backward of `mlp_forward`: returns (grad_input, grad_scores); weight gradients go to the grad buffers.
    Reference: fast_llm/functional/triton/mlp.py:314-415.
    """
    (
        input_,
        scores,
        intermediate_0,
        intermediate_1,
        intermediate_2,
        intermediate_3,
        weight_1,
        bias_1,
        weight_2,
        bias_2,
        gated,
        activation_type,
        group,
        sequence_parallel,
        transposed_layer_2_weight,
        sparse_map,
        input_shape,
        use_triton,
    ) = context
    context.clear()

    # Sparse copy
    if sparse_map is None:
        grad_scores = None
    else:
        grad_output, grad_scores = copy_sparse_to_dense_backward(grad_output, (sparse_map, intermediate_3, scores))

    # Sparse input recomputation
    if intermediate_0 is None:
        intermediate_0 = input_ if sparse_map is None else copy_dense_to_sparse_forward(input_, sparse_map)[0]

    # Layer 1 recomputation
    if intermediate_1 is None:
        intermediate_1 = output_parallel_linear_forward(
            intermediate_0, weight_1, bias_1, group, False, False, True, sparse_map
        )[0]

    # Layer 2 input grad, then activation recomputation and/or backward: in one kernel where the library has one
    # (the reference computes the layer 2 input grad before the two recomputations; they are independent).
    weight_2_t = maybe_transpose(weight_2, transposed_layer_2_weight)
    grad_intermediate_1 = None
    if KernelConfig.fuse_activation and _fusable(grad_output, weight_2_t, gated, sparse_map):
        try:
            grad_intermediate_1, intermediate_2_ = gated_layer_2_input_backward(
                grad_output, weight_2_t, sparse_map, intermediate_1, activation_type, intermediate_2 is None
            )
        except NotImplementedError:
            pass
    if grad_intermediate_1 is None:
        if sparse_map is None:
            grad_intermediate_2 = grad_output.matmul(weight_2_t)
        else:
            grad_intermediate_2 = output_sparse_matmul(grad_output, weight_2_t, sparse_map)
        grad_intermediate_1, intermediate_2_ = mlp_activation_backward(
            grad_intermediate_2.contiguous(), (intermediate_1, gated, activation_type, sparse_map), intermediate_2 is None
        )
        del grad_intermediate_2

    # Layer 2 parameter grad
    del intermediate_1
    update_linear_gradients(
        intermediate_2_ if intermediate_2 is None else intermediate_2,
        weight_2,
        bias_2,
        grad_output,
        transposed_layer_2_weight,
        sparse_map,
    )
    del grad_output, intermediate_2, intermediate_2_

    # Layer 1 backward
    grad_input = output_parallel_linear_backward(
        grad_intermediate_1,
        (intermediate_0, weight_1, bias_1, group, False, False, True, sparse_map),
    )

    # Sparse copy
    if sparse_map is not None:
        grad_input = copy_dense_to_sparse_backward(grad_input, (sparse_map, input_shape))

    return grad_input, grad_scores


mlp_autograd = wrap_forward_backward(mlp_forward, mlp_backward)


def mlp_autograd_looped(
    hidden_states: torch.Tensor,
    scores: torch.Tensor,
    top_experts: torch.Tensor,
    weight_1: torch.Tensor,
    weight_2: torch.Tensor,
    num_experts: int,
    gated: bool,
    activation_type: ActivationType,
    group: typing.Any,
    sequence_parallel: bool,
    training: bool = True,
    recompute_level: MLPRecomputeLevel = MLPRecomputeLevel.none,
) -> torch.Tensor:
    """
    The looped MoE: one dense MLP per expert over the tokens routed to it, output scaled by the score and added.
    Weight gradients land in the per-expert slices of the grad buffers. On the GPU this is the slow, simple
    alternative to the dropless path and is what the dropless path is compared with.
    Reference: fast_llm/functional/triton/mlp.py:421-527 (the chunk bookkeeping of `ChunkWeight`/`ChunkWeightPost` is
    done here by handing each expert a view of the weight with a view of the grad buffer).
    """
    from fast_llm_amd.tensor import param_get_and_unset_is_zero

    scores = scores.to(hidden_states.dtype)
    expert_mask = torch.nn.functional.one_hot(top_experts, num_classes=num_experts).permute(2, 1, 0)
    output = torch.zeros_like(hidden_states)

    is_zero = [weight.param_grad_is_zero for weight in (weight_1, weight_2)]
    chunks = []
    for weight, zero in zip((weight_1, weight_2), is_zero):
        weight_chunks = weight.detach().chunk(num_experts)
        for weight_chunk, grad_chunk in zip(weight_chunks, weight.grad_buffer.chunk(num_experts)):
            weight_chunk.requires_grad_(weight.requires_grad)
            weight_chunk.grad_buffer = grad_chunk
            weight_chunk.param_grad_is_zero = zero
        chunks.append(weight_chunks)

    class _Finish(torch.autograd.Function):
        # Runs first in backward: nothing to do. Exists so `_Start.backward` runs after every expert's backward.
        @staticmethod
        def forward(ctx, x):
            return x.view_as(x)

        @staticmethod
        def backward(ctx, grad):
            return grad

    class _Start(torch.autograd.Function):
        # Runs last in backward: experts without tokens still owe a zero gradient; consume the weight flags.
        @staticmethod
        def forward(ctx, x):
            return x.view_as(x)

        @staticmethod
        def backward(ctx, grad):
            for weight, weight_chunks in zip((weight_1, weight_2), chunks):
                if param_get_and_unset_is_zero(weight):
                    for weight_chunk in weight_chunks:
                        if weight_chunk.param_grad_is_zero:
                            weight_chunk.grad_buffer.zero_()
            return grad

    hidden_states = _Start.apply(hidden_states)
    for expert_idx, (weight_1_chunk, weight_2_chunk) in enumerate(zip(*chunks)):
        row, column = torch.where(expert_mask[expert_idx])
        if column.size(0) > 0:
            output[column] += (
                mlp_autograd(
                    hidden_states[column],
                    None,
                    weight_1_chunk,
                    None,
                    weight_2_chunk,
                    None,
                    gated,
                    activation_type,
                    group,
                    sequence_parallel,
                    training,
                    recompute_level,
                    True,
                )
                * scores[column, row, None]
            )
    return _Finish.apply(output)
