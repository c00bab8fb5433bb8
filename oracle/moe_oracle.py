"""
CPU oracle for the dropless-MoE hot path. TEST INFRASTRUCTURE ONLY.

This module restates, in plain torch on the CPU, what the reference (ServiceNow/Fast-LLM) computes on this path. It is
the checker for the HIP kernels: only `tests/`, `__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py`
may import it. Nothing under `fast_llm_amd/` imports it, and it never runs in place of a kernel.

Every function cites the reference lines it follows. The reference itself cannot be imported here (it needs
Python >= 3.12: PEP 695 generics at fast_llm/utils.py:35 and fast_llm/functional/utils.py:13, `enum.StrEnum` at
fast_llm/functional/config.py:31), so the restatement is pinned instead by independent formulations in
`tests/test_oracle_*.py`:

| function                              | pinned by                                                                              |
|---------------------------------------|----------------------------------------------------------------------------------------|
| sparse_map                            | brute-force O(M*E) loops on small inputs; invariants (permutation, ordering, padding)  |
|                                       | on the reference's test shapes (tests/functional/test_triton_kernels.py:255-258)       |
| copy_dense_to_sparse / sparse_to_dense| explicit per-(token, slot) loops; adjointness <dispatch(x), y> == <x, combine(y)>      |
| copy_sparse_to_dense_grad_score       | torch autograd of the combine                                                          |
| output/input_inner/input_row matmul   | one dense matmul over a block-embedded operand (the docstring formulas of the          |
|                                       | reference), on the reference's hand-written fixtures (test_sparse_matmul.py:68-98)     |
| mlp_activation_forward/backward       | torch autograd of `act(x1) * x2` in float64                                            |
| mlp_forward / mlp_backward (dropless) | the per-expert looped MoE with torch autograd in float64, padding rows NaN-poisoned   |
| looped_moe                            | a per-token double loop (textbook top-k mixture) in float64                            |
| router / router_backward              | closed forms (uniform and collapsed routers), a per-token loop in Python floats,       |
|                                       | central differences of the trained objective (tests/test_oracle_router.py)             |

Arithmetic convention of the oracle: every product and sum is evaluated in `compute_dtype` (float32 by default,
float64 for pinning), and every tensor the kernels would store is rounded once to the storage dtype of its inputs.
"""

import dataclasses
import typing

import torch

MAX_DROPLESS_BLOCK_SIZE_ROW = 128  # fast_llm/functional/config.py:106


@dataclasses.dataclass
class OracleSparseMap:
    """Same fields as the reference's `SparseMap` (fast_llm/functional/triton/sparse_copy.py:10-24)."""

    sparse_rows: torch.Tensor
    expert_ends: torch.Tensor
    expert_pad_begins: torch.Tensor
    num_rows_dense: int
    num_rows: int
    num_rows_unpadded: int
    num_experts: int
    num_experts_per_token: int

    @property
    def expert_begins(self) -> torch.Tensor:
        return torch.cat([self.expert_ends.new_zeros(1), self.expert_ends[:-1]])

    def real_row_mask(self) -> torch.Tensor:
        """True for rows that hold a token; False for padding inside an expert and for the phantom tail
        (same rows as tools/benchmark/triton_kernels/bench_sparse_copy.py:30-42 marks, inverted)."""
        mask = torch.zeros(self.num_rows, dtype=torch.bool)
        for begin, pad_begin in zip(self.expert_begins.tolist(), self.expert_pad_begins.tolist()):
            mask[begin:pad_begin] = True
        return mask


# ---------------------------------------------------------------------------------------------------------
# Sparse map
# ---------------------------------------------------------------------------------------------------------
def sparse_map(
    top_experts: torch.Tensor,
    num_experts: int,
    pad_to_multiple: int = MAX_DROPLESS_BLOCK_SIZE_ROW,
    dynamic_shape: bool = False,
) -> OracleSparseMap:
    """
    Follows `sparse_map_pytorch` (fast_llm/functional/triton/sparse_copy.py:224-238) with the stable sort of
    `_compute_expert_layout` (:249-250), and the shape rules of `get_sparse_map` (:267-270, :297). int64 results.
    """
    num_rows_dense, num_experts_per_token = top_experts.shape
    num_rows_unpadded = num_rows_dense * num_experts_per_token
    max_rows = (num_rows_unpadded + num_experts * pad_to_multiple) // pad_to_multiple * pad_to_multiple
    flat = top_experts.flatten().to(torch.int64)
    expert_counts = torch.bincount(flat, minlength=num_experts)
    assert expert_counts.numel() == num_experts
    padded_expert_counts = (expert_counts + pad_to_multiple - 1) // pad_to_multiple * pad_to_multiple
    expert_ends = padded_expert_counts.cumsum(0)
    expert_begins = expert_ends - padded_expert_counts
    expert_pad_begins = expert_begins + expert_counts
    # Rank of every entry in the stable sort by expert.
    unpadded_ranks = flat.sort(stable=True)[1].sort()[1].view_as(top_experts)
    expert_begins_unpadded = expert_counts.cumsum(0) - expert_counts
    sparse_rows = unpadded_ranks - expert_begins_unpadded[top_experts] + expert_begins[top_experts]
    return OracleSparseMap(
        sparse_rows=sparse_rows,
        expert_ends=expert_ends,
        expert_pad_begins=expert_pad_begins,
        num_rows_dense=num_rows_dense,
        num_rows=int(expert_ends[-1]) if dynamic_shape else max_rows,
        num_rows_unpadded=num_rows_unpadded,
        num_experts=num_experts,
        num_experts_per_token=num_experts_per_token,
    )


# ---------------------------------------------------------------------------------------------------------
# Copies
# ---------------------------------------------------------------------------------------------------------
def copy_dense_to_sparse(
    input_: torch.Tensor,
    scores: torch.Tensor | None,
    sparse_map_: OracleSparseMap,
    fill: float = 0.0,
    compute_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """
    out[sparse_rows[t, j]] = input_[t] * (scores[t, j] or 1); product in `compute_dtype`, one rounding
    (fast_llm/functional/triton/sparse_copy.py:27-49). The reference leaves the other rows uninitialised (:56);
    here they hold `fill` (tests use NaN to prove that nothing consumes them).
    """
    out = input_.new_full((sparse_map_.num_rows, input_.size(1)), fill)
    rows = sparse_map_.sparse_rows.long()
    for j in range(sparse_map_.num_experts_per_token):
        if scores is None:
            out[rows[:, j]] = input_
        else:
            out[rows[:, j]] = (input_.to(compute_dtype) * scores[:, j, None].to(compute_dtype)).to(input_.dtype)
    return out


def copy_sparse_to_dense(
    input_: torch.Tensor,
    scores: torch.Tensor | None,
    sparse_map_: OracleSparseMap,
    compute_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """
    out[t] = sum_j input_[sparse_rows[t, j]] * (scores[t, j] or 1), slots added in order, accumulation in
    `compute_dtype`, one rounding (fast_llm/functional/triton/sparse_copy.py:69-90).
    """
    rows = sparse_map_.sparse_rows.long()
    out = torch.zeros((sparse_map_.num_rows_dense, input_.size(1)), dtype=compute_dtype)
    for j in range(sparse_map_.num_experts_per_token):
        term = input_[rows[:, j]].to(compute_dtype)
        if scores is not None:
            term = term * scores[:, j, None].to(compute_dtype)
        out = out + term
    return out.to(input_.dtype)


def copy_sparse_to_dense_grad_score(
    input_: torch.Tensor,
    grad_output: torch.Tensor,
    sparse_map_: OracleSparseMap,
    compute_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """
    grad_scores[t, j] = <input_[sparse_rows[t, j]], grad_output[t]> in `compute_dtype`, stored in the dtype of `input_`
    (fast_llm/functional/triton/sparse_copy.py:111-165, output dtype at :155).
    """
    rows = sparse_map_.sparse_rows.long()
    gathered = input_[rows].to(compute_dtype)  # [T, k, H]
    return (gathered * grad_output[:, None, :].to(compute_dtype)).sum(-1).to(input_.dtype)


# ---------------------------------------------------------------------------------------------------------
# Grouped matrix products: per-expert torch.matmul, as the reference's own tests state them
# (tests/functional/test_sparse_matmul.py:124-132, 144-152, 164-172).
# ---------------------------------------------------------------------------------------------------------
def _mm(a: torch.Tensor, b: torch.Tensor, compute_dtype: torch.dtype) -> torch.Tensor:
    return a.to(compute_dtype) @ b.to(compute_dtype)


def output_sparse_matmul(
    lhs: torch.Tensor,
    rhs: torch.Tensor,
    sparse_map_: OracleSparseMap,
    out: torch.Tensor | None = None,
    accumulate: bool = False,
    compute_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """
    out[b_e:end_e] = lhs[b_e:end_e] @ rhs[:, e*N_s:(e+1)*N_s]; padding rows are computed like real ones, rows past
    the last expert are left as they are (fast_llm/functional/triton/sparse_linear.py:185-258, 261-307).
    """
    col_sparse_dim = rhs.size(1) // sparse_map_.num_experts
    if out is None:
        out = lhs.new_zeros(lhs.size(0), col_sparse_dim)
    begin = 0
    for e, end in enumerate(sparse_map_.expert_ends.tolist()):
        result = _mm(lhs[begin:end], rhs[:, e * col_sparse_dim : (e + 1) * col_sparse_dim], compute_dtype)
        if accumulate:
            result = result + out[begin:end].to(compute_dtype)
        out[begin:end] = result.to(out.dtype)
        begin = end
    return out


def input_inner_sparse_matmul(
    lhs: torch.Tensor,
    rhs: torch.Tensor,
    sparse_map_: OracleSparseMap,
    out: torch.Tensor | None = None,
    accumulate: bool = False,
    compute_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """
    out[b_e:end_e] = lhs[b_e:end_e] @ rhs[e*K_s:(e+1)*K_s] (fast_llm/functional/triton/sparse_linear.py:310-385,
    388-434).
    """
    inner_sparse_dim = lhs.size(1)
    if out is None:
        out = lhs.new_zeros(lhs.size(0), rhs.size(1))
    begin = 0
    for e, end in enumerate(sparse_map_.expert_ends.tolist()):
        result = _mm(lhs[begin:end], rhs[e * inner_sparse_dim : (e + 1) * inner_sparse_dim], compute_dtype)
        if accumulate:
            result = result + out[begin:end].to(compute_dtype)
        out[begin:end] = result.to(out.dtype)
        begin = end
    return out


def input_row_sparse_matmul(
    lhs: torch.Tensor,
    rhs: torch.Tensor,
    sparse_map_: OracleSparseMap,
    out: torch.Tensor | None = None,
    accumulate: bool = False,
    compute_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """
    out[e*M_s:(e+1)*M_s] = lhs[:, b_e:pad_begin_e] @ rhs[b_e:pad_begin_e]: padding rows excluded, an expert without
    tokens gives zeros (fast_llm/functional/triton/sparse_linear.py:437-517, 520-570).
    """
    row_sparse_dim = lhs.size(0)
    if out is None:
        out = lhs.new_zeros(row_sparse_dim * sparse_map_.num_experts, rhs.size(1))
    begins = sparse_map_.expert_begins.tolist()
    for e, (begin, pad_begin) in enumerate(zip(begins, sparse_map_.expert_pad_begins.tolist())):
        result = _mm(lhs[:, begin:pad_begin], rhs[begin:pad_begin], compute_dtype)
        block = slice(e * row_sparse_dim, (e + 1) * row_sparse_dim)
        if accumulate:
            result = result + out[block].to(compute_dtype)
        out[block] = result.to(out.dtype)
    return out


# ---------------------------------------------------------------------------------------------------------
# Activation
# ---------------------------------------------------------------------------------------------------------
def _activation(name: str, x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """act(x), act'(x) with the formulas of fast_llm/functional/triton/mlp.py:49-67 and :100-128."""
    if name == "gelu":
        tanh_input = 0.79788456 * x * (1 + 0.044715 * x * x)
        tanh = 1 - 2 / (1 + torch.exp(2 * tanh_input))
        grad = 0.5 * x * ((1 - tanh * tanh) * (0.79788456 + 0.1070322243 * x * x)) + 0.5 * (1 + tanh)
        return x * 0.5 * (1.0 + tanh), grad
    if name == "silu":
        exp = torch.exp(-x)
        sigma = 1 / (1 + exp)
        return x * sigma, sigma * sigma + (1 + x) / (2 + exp + 1 / exp)
    if name == "relu":
        return torch.where(x > 0, x, torch.zeros_like(x)), (x > 0).to(x.dtype)
    if name == "squared_relu":
        relu = torch.where(x > 0, x, torch.zeros_like(x))
        return relu * relu, 2 * relu
    if name == "identity":
        return x, torch.ones_like(x)
    raise NotImplementedError(name)


def mlp_activation_forward(
    input_: torch.Tensor, gated: bool, activation: str, compute_dtype: torch.dtype = torch.float32
) -> torch.Tensor:
    """out = act(x[:, :n]) * x[:, n:] (gated) or act(x) (fast_llm/functional/triton/mlp.py:29-71)."""
    n_cols = input_.size(-1) // (2 if gated else 1)
    x = input_[..., :n_cols].to(compute_dtype)
    out, _ = _activation(activation, x)
    if gated:
        out = out * input_[..., n_cols:].to(compute_dtype)
    return out.to(input_.dtype)


def mlp_activation_backward(
    grad_output: torch.Tensor,
    input_: torch.Tensor,
    gated: bool,
    activation: str,
    compute_dtype: torch.dtype = torch.float32,
) -> tuple[torch.Tensor, torch.Tensor]:
    """
    (grad_input, recomputed output): grad_gate = act'(x) * up * go, grad_up = act(x) * go
    (fast_llm/functional/triton/mlp.py:74-139).
    """
    n_cols = grad_output.size(-1)
    x = input_[..., :n_cols].to(compute_dtype)
    go = grad_output.to(compute_dtype)
    out, grad = _activation(activation, x)
    if gated:
        up = input_[..., n_cols:].to(compute_dtype)
        grad_input = torch.cat([grad * up * go, out * go], dim=-1)
        out = out * up
    else:
        grad_input = grad * go
    return grad_input.to(input_.dtype), out.to(input_.dtype)


# ---------------------------------------------------------------------------------------------------------
# The composed dropless MLP
# ---------------------------------------------------------------------------------------------------------
@dataclasses.dataclass
class DroplessResult:
    output: torch.Tensor
    grad_input: torch.Tensor
    grad_scores: torch.Tensor
    grad_weight_1: torch.Tensor
    grad_weight_2: torch.Tensor
    intermediates: dict[str, torch.Tensor]


def dropless_mlp_forward_backward(
    input_: torch.Tensor,
    scores: torch.Tensor,
    weight_1: torch.Tensor,
    weight_2: torch.Tensor,
    sparse_map_: OracleSparseMap,
    grad_output: torch.Tensor,
    gated: bool = True,
    activation: str = "silu",
    padding_fill: float = float("nan"),
    grad_dtype: torch.dtype | None = None,
    compute_dtype: torch.dtype = torch.float32,
) -> DroplessResult:
    """
    Forward and backward of the dropless MoE MLP, operation by operation in the order of `mlp_forward` /
    `mlp_backward` (fast_llm/functional/triton/mlp.py:207-311, 314-415) with the operand choices of
    fast_llm/functional/linear.py:43-55, 128-132, 161, 199-201. weight_1 is [E*2F, H] (per expert [gate; up]),
    weight_2 is [E*F, H] (`transposed_layer_2_weight=True`). Padding rows of the sparse input hold `padding_fill`.
    """
    kw = {"compute_dtype": compute_dtype}
    # forward
    x_sparse = copy_dense_to_sparse(input_, None, sparse_map_, fill=padding_fill, **kw)
    layer_1 = output_sparse_matmul(x_sparse, weight_1.t(), sparse_map_, **kw)
    activated = mlp_activation_forward(layer_1, gated, activation, **kw)
    layer_2 = input_inner_sparse_matmul(activated, weight_2, sparse_map_, **kw)
    output = copy_sparse_to_dense(layer_2, scores, sparse_map_, **kw)
    # backward
    grad_layer_2 = copy_dense_to_sparse(grad_output, scores, sparse_map_, fill=padding_fill, **kw)
    grad_scores = copy_sparse_to_dense_grad_score(layer_2, grad_output, sparse_map_, **kw)
    grad_activated = output_sparse_matmul(grad_layer_2, weight_2.t(), sparse_map_, **kw)
    grad_layer_1, _ = mlp_activation_backward(grad_activated, layer_1, gated, activation, **kw)
    grad_dtype = weight_1.dtype if grad_dtype is None else grad_dtype
    grad_weight_2 = input_row_sparse_matmul(
        activated.t(), grad_layer_2, sparse_map_, out=torch.zeros(weight_2.shape, dtype=grad_dtype), **kw
    )
    grad_x_sparse = input_inner_sparse_matmul(grad_layer_1, weight_1, sparse_map_, **kw)
    grad_weight_1 = input_row_sparse_matmul(
        grad_layer_1.t(), x_sparse, sparse_map_, out=torch.zeros(weight_1.shape, dtype=grad_dtype), **kw
    )
    grad_input = copy_sparse_to_dense(grad_x_sparse, None, sparse_map_, **kw)
    return DroplessResult(
        output=output,
        grad_input=grad_input,
        grad_scores=grad_scores,
        grad_weight_1=grad_weight_1,
        grad_weight_2=grad_weight_2,
        intermediates={
            "x_sparse": x_sparse,
            "layer_1": layer_1,
            "activated": activated,
            "layer_2": layer_2,
            "grad_layer_2": grad_layer_2,
            "grad_activated": grad_activated,
            "grad_layer_1": grad_layer_1,
            "grad_x_sparse": grad_x_sparse,
        },
    )


# ---------------------------------------------------------------------------------------------------------
# The looped MoE (the reference's CPU-runnable path, and the CPU baseline of the benchmark)
# ---------------------------------------------------------------------------------------------------------
def looped_moe(
    hidden_states: torch.Tensor,
    scores: torch.Tensor,
    top_experts: torch.Tensor,
    weight_1: torch.Tensor,
    weight_2: torch.Tensor,
    num_experts: int,
    gated: bool = True,
    activation: typing.Callable[[torch.Tensor], torch.Tensor] = torch.nn.functional.silu,
) -> torch.Tensor:
    """
    One dense MLP per expert over the tokens routed to it; result scaled by the score and added into the output.
    Differentiable with torch autograd (weights and inputs are leaves), which is how the reference gets the backward
    of this path. Follows `mlp_autograd_looped` (fast_llm/functional/triton/mlp.py:480-527): one-hot mask ->
    `torch.where` per expert -> gather -> linear -> act(gate)*up -> linear -> `output[tokens] += y * score`.
    weight_1 [E*2F, H] and weight_2 [E*F, H] are chunked per expert along dim 0.
    """
    scores = scores.to(hidden_states.dtype)
    expert_mask = torch.nn.functional.one_hot(top_experts, num_classes=num_experts).permute(2, 1, 0)
    output = torch.zeros_like(hidden_states)
    for expert_idx, (weight_1_chunk, weight_2_chunk) in enumerate(
        zip(weight_1.chunk(num_experts), weight_2.chunk(num_experts))
    ):
        row, column = torch.where(expert_mask[expert_idx])
        if column.size(0) > 0:
            layer_1 = torch.nn.functional.linear(hidden_states[column], weight_1_chunk)
            if gated:
                gate, up = layer_1.chunk(2, dim=-1)
                activated = activation(gate) * up
            else:
                activated = activation(layer_1)
            layer_2 = activated @ weight_2_chunk
            output = output.index_add(0, column, layer_2 * scores[column, row, None])
    return output


def looped_moe_forward_backward(
    hidden_states: torch.Tensor,
    scores: torch.Tensor,
    top_experts: torch.Tensor,
    weight_1: torch.Tensor,
    weight_2: torch.Tensor,
    num_experts: int,
    grad_output: torch.Tensor,
    gated: bool = True,
) -> DroplessResult:
    leaves = [t.detach().clone().requires_grad_(True) for t in (hidden_states, scores, weight_1, weight_2)]
    output = looped_moe(leaves[0], leaves[1], top_experts, leaves[2], leaves[3], num_experts, gated)
    output.backward(grad_output.to(output.dtype))
    return DroplessResult(
        output=output.detach(),
        grad_input=leaves[0].grad,
        grad_scores=leaves[1].grad,
        grad_weight_1=leaves[2].grad,
        grad_weight_2=leaves[3].grad,
        intermediates={},
    )


# ---------------------------------------------------------------------------------------------------------
# Routing and workloads shared by tests and the benchmark
# ---------------------------------------------------------------------------------------------------------
def topk_routing(logits: torch.Tensor, experts_per_token: int) -> tuple[torch.Tensor, torch.Tensor]:
    """top-k experts and fp32 softmax over the selected logits
    (fast_llm/layers/decoder/mlp/mixture_of_experts.py:243-244)."""
    top_logits, top_experts = torch.topk(logits, k=experts_per_token, dim=-1)
    return torch.softmax(top_logits, dim=-1, dtype=torch.float32), top_experts


@dataclasses.dataclass
class RouterResult:
    scores: torch.Tensor  # [tokens, shared + k] fp32
    top_experts: torch.Tensor  # [tokens, shared + k] int64
    load_balancing_loss: torch.Tensor  # scalar fp32
    z_loss: torch.Tensor  # scalar fp32


def router(
    logits: torch.Tensor,
    experts_per_token: int,
    shared_experts: int = 0,
    noise: torch.Tensor | None = None,
    compute_dtype: torch.dtype = torch.float32,
) -> RouterResult:
    """What `MixtureOfExpertMLP._forward` does between the router's logits and the sparse map, for top-k routing
    (fast_llm/layers/decoder/mlp/mixture_of_experts.py:146-171), differentiable with torch autograd as there:
    z-loss on the logits as they come (:147-154; layers/language_model/loss/z_loss.py:88-92), jitter (:157-159,
    234-235: a product in the logits' own dtype), `_topk_routing` with its load-balancing loss (:243-254), then
    `_add_shared_experts` (:264-278). `logits` has one column per routed expert. The softmaxes run in
    `compute_dtype` (the reference's float32; float64 for pinning)."""
    z_loss = (torch.logsumexp(logits.to(compute_dtype), dim=-1) ** 2).mean()
    if noise is not None:
        logits = logits * noise
    top_logits, top_experts = torch.topk(logits, k=experts_per_token, dim=-1)
    scores = torch.softmax(top_logits, dim=-1, dtype=compute_dtype)
    probabilities = torch.softmax(logits, dim=-1, dtype=compute_dtype)
    mask = torch.nn.functional.one_hot(top_experts, num_classes=logits.size(-1)).sum(dim=1)
    load_balancing_loss = torch.sum(probabilities.mean(dim=0) * mask.mean(dim=0, dtype=compute_dtype))
    if shared_experts > 0:
        first = logits.size(-1)
        shared = torch.arange(first, first + shared_experts, dtype=top_experts.dtype)[None].repeat(logits.size(0), 1)
        top_experts = torch.cat((shared, top_experts), dim=1)
        scores = torch.cat((scores.new_ones(scores.size(0), shared_experts), scores), dim=1)
    return RouterResult(scores, top_experts, load_balancing_loss, z_loss)


def router_backward(
    result: RouterResult,
    logits: torch.Tensor,
    grad_scores: torch.Tensor,
    auxiliary_loss_grad: float = 0.0,
    z_loss_grad: float = 0.0,
) -> torch.Tensor:
    """Gradient of `logits` (a leaf that `result` was computed from). `AuxiliaryLoss` hands each loss a constant
    gradient when the scores (or logits) it is attached to are back-propagated (fast_llm/functional/utils.py:63-71):
    `unshared_experts * auxiliary_loss_coefficient * grad_scale` for the load-balancing loss
    (mixture_of_experts.py:257-261) and `z_loss_coefficient * grad_scale` for the z-loss (:154)."""
    total = (
        (result.scores * grad_scores.to(result.scores.dtype)).sum()
        + auxiliary_loss_grad * result.load_balancing_loss
        + z_loss_grad * result.z_loss
    )
    (grad_logits,) = torch.autograd.grad(total, logits)
    return grad_logits


def router_input(
    hidden_states: torch.Tensor,
    normalization: typing.Callable[[torch.Tensor], torch.Tensor] | None = None,
    scale: torch.Tensor | None = None,
    input_scale: float = 1.0,
) -> torch.Tensor:
    """What the router's linear layer sees (fast_llm/layers/decoder/mlp/mixture_of_experts.py:123-145): the hidden
    states through the optional router normalisation, times the optional per-feature scale, times the constant."""
    x = hidden_states if normalization is None else normalization(hidden_states)
    if scale is not None:
        x = x * scale
    if input_scale != 1.0:
        x = x * input_scale
    return x


def per_expert_scale(scores: torch.Tensor, top_experts: torch.Tensor, scale: torch.Tensor | None) -> torch.Tensor:
    """scores * scale[top_experts] (mixture_of_experts.py:174-175)."""
    return scores if scale is None else scores * scale[top_experts]


def sinkhorn(cost: torch.Tensor, tolerance: float = 1e-5, eps: float = 1e-9) -> torch.Tensor:
    """The reference's sinkhorn iteration (mixture_of_experts.py:389-403) with explicit sums: row scales
    d0[t] = (1 / T) / (sum_e d1[e] c[t, e] + eps), column scales d1[e] = (1 / E) / (sum_t d0[t] c[t, e] + eps),
    c = exp(cost), repeated until mean |d1 - d1_previous| <= tolerance; returns d0[t] c[t, e] d1[e]."""
    c = torch.exp(cost.to(torch.float32))
    tokens, experts = c.shape
    d0, d1 = torch.ones(tokens), torch.ones(experts)
    while True:
        d0 = (1.0 / tokens) / ((c * d1[None, :]).sum(dim=1) + eps)
        new_d1 = (1.0 / experts) / ((c * d0[:, None]).sum(dim=0) + eps)
        error = (new_d1 - d1).abs().mean().item()
        d1 = new_d1
        if not error > tolerance:
            break
    return d0[:, None] * c * d1[None, :]


def sinkhorn_routing(logits: torch.Tensor, experts_per_token: int, training: bool) -> tuple[torch.Tensor, torch.Tensor]:
    """(scores, top_experts) of `_sinkhorn_routing` (mixture_of_experts.py:280-296)."""
    if experts_per_token == 1:
        activated = torch.sigmoid(logits)
    else:
        activated = torch.softmax(logits, dim=-1, dtype=torch.float32).type_as(logits)
    if training:
        top_experts = torch.topk(sinkhorn(logits.detach()), k=experts_per_token, dim=-1).indices
        return torch.gather(activated, -1, top_experts), top_experts
    scores, top_experts = torch.topk(activated, k=experts_per_token, dim=-1)
    return scores, top_experts
