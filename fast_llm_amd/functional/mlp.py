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


class _MLPContext(typing.NamedTuple):
    """What `mlp_forward` hands `mlp_backward`, in the positional layout of the reference's context list
    (fast_llm/functional/triton/mlp.py:287-306). An intermediate that the recompute level does not keep is None."""

    input_: torch.Tensor | None  # dense tokens; kept only when the sparse copy of them is recomputed
    scores: torch.Tensor | None
    sparse_input: torch.Tensor | None  # tokens in the expert-sorted layout (the dense input itself without a map)
    layer_1_output: torch.Tensor | None
    activation_output: torch.Tensor | None
    layer_2_output: torch.Tensor | None  # always kept with a map: the score gradient reads it
    weight_1: torch.Tensor
    bias_1: torch.Tensor | None
    weight_2: torch.Tensor
    bias_2: torch.Tensor | None
    gated: bool
    activation_type: ActivationType
    group: typing.Any
    sequence_parallel: bool
    transposed_layer_2_weight: bool
    sparse_map: SparseMap | None
    input_shape: torch.Size
    use_triton: bool | None


def _fuse_forward(keep_layer_1: bool) -> bool:
    """Whether layer 1 takes the kernel with the activation in its epilogue: when asked to, and by default exactly
    where that kernel wins, i.e. where layer 1's output is not stored (see `KernelConfig.fuse_activation`)."""
    return not keep_layer_1 if KernelConfig.fuse_activation is None else bool(KernelConfig.fuse_activation)


def _fuse_backward() -> bool:
    return bool(KernelConfig.fuse_activation)  # by default never: measured slower than the two kernels


def _layer_1_and_activation(sparse_input, weight_1, bias_1, gated, activation_type, sparse_map, keep_layer_1):
    """(layer-1 output or None if it is neither kept nor needed, activation output)."""
    if _fuse_forward(keep_layer_1) and _fusable(sparse_input, weight_1.t(), gated, sparse_map, bias_1):
        try:
            return gated_layer_1_forward(sparse_input, weight_1, sparse_map, activation_type, keep_layer_1)
        except NotImplementedError:  # a shape the fused kernel does not tile
            pass
    layer_1_output, _ = output_parallel_linear_forward(sparse_input, weight_1, bias_1, None, False, False, True, sparse_map)
    activation_output, _ = mlp_activation_forward(layer_1_output, gated, activation_type, sparse_map)
    return (layer_1_output if keep_layer_1 else None), activation_output


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
    sparse = sparse_map is not None
    keep_layer_1 = training and not recompute_level.recompute_layer_1
    keep_activation = training and not recompute_level.recompute_activation

    sparse_input = copy_dense_to_sparse_forward(input_, sparse_map)[0] if sparse else input_
    layer_1_output, activation_output = _layer_1_and_activation(
        sparse_input, weight_1, bias_1, gated, activation_type, sparse_map, keep_layer_1
    )
    layer_2_output, _ = input_parallel_linear_forward(
        activation_output, weight_2, bias_2, group, False, transposed_layer_2_weight, True, sparse_map
    )
    output = copy_sparse_to_dense_forward(layer_2_output, scores, sparse_map)[0] if sparse else layer_2_output
    if not training:
        return output, None

    # Either the dense tokens or their sparse copy go to the backward, never both.
    recompute_input = recompute_level.recompute_sparse_input
    context = _MLPContext(
        input_=input_ if recompute_input else None,
        scores=scores,
        sparse_input=None if recompute_input else sparse_input,
        layer_1_output=layer_1_output,
        activation_output=activation_output if keep_activation else None,
        layer_2_output=layer_2_output if sparse else None,
        weight_1=weight_1,
        bias_1=bias_1,
        weight_2=weight_2,
        bias_2=bias_2,
        gated=gated,
        activation_type=activation_type,
        group=group,
        sequence_parallel=sequence_parallel,
        transposed_layer_2_weight=transposed_layer_2_weight,
        sparse_map=sparse_map,
        input_shape=input_.shape,
        use_triton=use_triton,
    )
    return output, list(context)


def mlp_backward(grad_output: torch.Tensor, context: list[typing.Any]) -> tuple[torch.Tensor, torch.Tensor]:
    """
    Backward of `mlp_forward`: returns (grad_input, grad_scores); weight gradients go to the grad buffers.
    Reference: fast_llm/functional/triton/mlp.py:314-415.
    """
    saved = _MLPContext(*context)
    context.clear()  # the list may outlive this call (autograd holds it): let go of the tensors now
    sparse_map, gated, activation_type = saved.sparse_map, saved.gated, saved.activation_type
    weight_2, bias_2, transposed_layer_2_weight = saved.weight_2, saved.bias_2, saved.transposed_layer_2_weight
    input_shape = saved.input_shape
    sparse = sparse_map is not None

    # Backward of the combine: the gradient of layer 2's output, and of the scores.
    grad_scores = None
    if sparse:
        grad_output, grad_scores = copy_sparse_to_dense_backward(
            grad_output, (sparse_map, saved.layer_2_output, saved.scores)
        )

    # Whatever the forward did not keep is computed again, front to back.
    sparse_input = saved.sparse_input
    if sparse_input is None:
        sparse_input = copy_dense_to_sparse_forward(saved.input_, sparse_map)[0] if sparse else saved.input_
    layer_1_context = (sparse_input, saved.weight_1, saved.bias_1, None, False, False, True, sparse_map)
    layer_1_output = saved.layer_1_output
    if layer_1_output is None:
        layer_1_output = output_parallel_linear_forward(*layer_1_context)[0]
    activation_output = saved.activation_output
    recompute_activation = activation_output is None
    del saved  # every intermediate now has one name here and is released as soon as its last reader is done

    # Gradient of layer 1's output = activation backward of (grad_output x W2^T), which also recomputes the
    # activation output if needed: one kernel where the library has one and is asked to use it, else two. (The
    # reference takes the layer-2 input gradient before its recomputations; the order does not matter.)
    weight_2_t = maybe_transpose(weight_2, transposed_layer_2_weight)
    grad_layer_1_output = None
    if _fuse_backward() and _fusable(grad_output, weight_2_t, gated, sparse_map):
        try:
            grad_layer_1_output, recomputed = gated_layer_2_input_backward(
                grad_output, weight_2_t, sparse_map, layer_1_output, activation_type, recompute_activation
            )
        except NotImplementedError:
            pass
    if grad_layer_1_output is None:
        if sparse:
            grad_activation_output = output_sparse_matmul(grad_output, weight_2_t, sparse_map)
        else:
            grad_activation_output = grad_output.matmul(weight_2_t)
        grad_layer_1_output, recomputed = mlp_activation_backward(
            grad_activation_output.contiguous(), (layer_1_output, gated, activation_type, sparse_map), recompute_activation
        )
        del grad_activation_output
    del layer_1_output
    if recompute_activation:
        activation_output = recomputed
    del recomputed

    # Layer 2's weight gradient, then layer 1's input and weight gradients.
    update_linear_gradients(activation_output, weight_2, bias_2, grad_output, transposed_layer_2_weight, sparse_map)
    del grad_output, activation_output
    grad_input = output_parallel_linear_backward(grad_layer_1_output, layer_1_context)

    # Backward of the dispatch.
    if sparse:
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
