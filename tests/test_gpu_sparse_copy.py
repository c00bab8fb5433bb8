"""Dispatch, combine, score gradient and their autograd pairs on the GPU against the oracle."""

import pytest
import torch

from fast_llm_amd import _lib
from fast_llm_amd.functional.sparse_copy import (
    copy_dense_to_sparse,
    copy_dense_to_sparse_autograd,
    copy_sparse_to_dense,
    copy_sparse_to_dense_autograd,
    copy_sparse_to_dense_backward,
    copy_sparse_to_dense_grad_score,
    get_sparse_map,
)
from fast_llm_amd.workloads import WORKLOADS, make_inputs
from oracle import moe_oracle
from tests.helpers import REFERENCE_FIXTURES, max_rel_err, to_device_map

pytestmark = pytest.mark.gpu

# One fp32 multiply is exact against the oracle; sums may be contracted to FMAs, hence a few ulps.
_TOLERANCE = {torch.float32: 2e-6, torch.bfloat16: 1e-2, torch.float16: 2e-3}


def _problem(tokens, experts, top_k, hidden, dtype, seed=0, scores_dtype=torch.float32):
    generator = torch.Generator().manual_seed(seed)
    logits = torch.randn(tokens, experts, generator=generator)
    scores, top_experts = moe_oracle.topk_routing(logits, top_k)
    sparse_map = moe_oracle.sparse_map(top_experts, experts)
    dense = torch.randn(tokens, hidden, generator=generator).to(dtype)
    sparse = torch.randn(sparse_map.num_rows, hidden, generator=generator).to(dtype)
    return sparse_map, scores.to(scores_dtype), dense, sparse


_smoke = REFERENCE_FIXTURES["copy_smoke"]
_SHAPES = [
    (_smoke["tokens"], _smoke["experts"], _smoke["top_k"], _smoke["hidden"]),
    (300, 8, 2, 4096),
    (257, 6, 3, 1000),  # hidden not a multiple of the vector width x threads
    (50, 4, 4, 37),  # scalar path
    (129, 64, 6, 2048),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize(("tokens", "experts", "top_k", "hidden"), _SHAPES)
@pytest.mark.parametrize("scored", [False, True])
def test_dispatch_and_combine(tokens, experts, top_k, hidden, dtype, scored, device):
    oracle_map, scores, dense, sparse = _problem(tokens, experts, top_k, hidden, dtype)
    sparse_map = to_device_map(oracle_map, device, torch.int32)
    gpu_scores = scores.to(device) if scored else None
    mask = oracle_map.real_row_mask()

    dispatched = copy_dense_to_sparse(dense.to(device), gpu_scores, sparse_map).cpu()
    expected = moe_oracle.copy_dense_to_sparse(dense, scores if scored else None, oracle_map)
    assert dispatched.shape == expected.shape
    if scored and dtype == torch.float16:
        # The fp16 product is rounded once from the exact value (fused multiply-convert), the oracle rounds it to
        # fp32 first: results may differ by one fp16 ulp on rare ties.
        ulp = torch.finfo(dtype).eps * expected[mask].float().abs().clamp_min(2.0**-14)
        assert ((dispatched[mask].float() - expected[mask].float()).abs() <= ulp).all()
    else:
        # A copy, or a single fp32 product rounded once: bit-exact.
        different = dispatched[mask] != expected[mask]
        assert not different.any(), (
            f"{different.sum().item()} of {different.numel()} differ, e.g. "
            f"{dispatched[mask][different][:4].tolist()} vs {expected[mask][different][:4].tolist()}"
        )

    combined = copy_sparse_to_dense(sparse.to(device), gpu_scores, sparse_map).cpu()
    expected = moe_oracle.copy_sparse_to_dense(sparse, scores if scored else None, oracle_map)
    assert max_rel_err(combined, expected) <= _TOLERANCE[dtype]


@pytest.mark.parametrize("index_dtype", [torch.int16, torch.int32, torch.int64])
@pytest.mark.parametrize("scores_dtype", [torch.float32, torch.bfloat16])
def test_index_and_score_dtypes(index_dtype, scores_dtype, device):
    oracle_map, scores, dense, sparse = _problem(200, 8, 2, 512, torch.bfloat16, seed=1, scores_dtype=scores_dtype)
    sparse_map = to_device_map(oracle_map, device, index_dtype)
    dispatched = copy_dense_to_sparse(dense.to(device), scores.to(device), sparse_map).cpu()
    expected = moe_oracle.copy_dense_to_sparse(dense, scores, oracle_map)
    mask = oracle_map.real_row_mask()
    assert torch.equal(dispatched[mask], expected[mask])
    combined = copy_sparse_to_dense(sparse.to(device), scores.to(device), sparse_map).cpu()
    assert max_rel_err(combined, moe_oracle.copy_sparse_to_dense(sparse, scores, oracle_map)) <= 1e-2


def test_dispatch_leaves_padding_rows_untouched(device, library):
    """Through the C ABI with a caller-owned, pre-poisoned output buffer."""
    oracle_map, scores, dense, _ = _problem(100, 4, 2, 256, torch.float32, seed=2)
    rows = oracle_map.sparse_rows.to(device=device, dtype=torch.int32)
    out = torch.full((oracle_map.num_rows, 256), float("nan"), device=device)
    dense_gpu = dense.to(device)
    status = library.fm_copy_dense_to_sparse(
        dense_gpu.data_ptr(), None, rows.data_ptr(), out.data_ptr(), 100, 256, 2, oracle_map.num_rows,
        0, 0, 1, torch.cuda.current_stream().cuda_stream,
    )
    assert status == 0, library.fm_last_error()
    mask = oracle_map.real_row_mask().to(device)
    assert out[~mask].isnan().all() and not out[mask].isnan().any()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize(("tokens", "experts", "top_k", "hidden"), _SHAPES + [(64, 8, 8, 8192 + 2048)])
def test_grad_score_and_fused_backward(tokens, experts, top_k, hidden, dtype, device):
    oracle_map, scores, grad_output, sparse = _problem(tokens, experts, top_k, hidden, dtype, seed=3)
    sparse_map = to_device_map(oracle_map, device, torch.int32)
    sparse_gpu, grad_gpu, scores_gpu = sparse.to(device), grad_output.to(device), scores.to(device)

    grad_scores = copy_sparse_to_dense_grad_score(sparse_gpu, grad_gpu, sparse_map)
    assert grad_scores.dtype == dtype  # the reference returns the activation dtype (sparse_copy.py:155)
    expected = moe_oracle.copy_sparse_to_dense_grad_score(sparse, grad_output, oracle_map)
    assert max_rel_err(grad_scores.cpu(), expected) <= _TOLERANCE[dtype] * 4

    fused_input, fused_scores = copy_sparse_to_dense_backward(grad_gpu, (sparse_map, sparse_gpu, scores_gpu))
    separate_input = copy_dense_to_sparse(grad_gpu, scores_gpu, sparse_map)
    mask = oracle_map.real_row_mask().to(device)
    assert torch.equal(fused_scores, grad_scores)
    assert torch.equal(fused_input[mask], separate_input[mask])


def test_autograd_pairs(device):
    oracle_map, scores, dense, sparse = _problem(150, 8, 2, 384, torch.float32, seed=4)
    sparse_map = to_device_map(oracle_map, device, torch.int16)
    mask = oracle_map.real_row_mask()

    dense_leaf = dense.to(device).view(3, 50, 384).requires_grad_(True)
    out = copy_dense_to_sparse_autograd(dense_leaf, sparse_map)
    grad = torch.randn(oracle_map.num_rows, 384)
    out.backward(grad.to(device))
    expected = moe_oracle.copy_sparse_to_dense(grad, None, oracle_map)  # un-scored combine of the gradient
    assert dense_leaf.grad.shape == dense_leaf.shape
    assert max_rel_err(dense_leaf.grad.cpu().view(150, 384), expected) <= 2e-6

    sparse_leaf = sparse.to(device).requires_grad_(True)
    scores_leaf = scores.to(device).requires_grad_(True)
    out = copy_sparse_to_dense_autograd(sparse_leaf, scores_leaf, sparse_map)
    grad = torch.randn(150, 384)
    out.backward(grad.to(device))
    assert torch.equal(sparse_leaf.grad.cpu()[mask], moe_oracle.copy_dense_to_sparse(grad, scores, oracle_map)[mask])
    expected = moe_oracle.copy_sparse_to_dense_grad_score(sparse, grad, oracle_map)
    assert scores_leaf.grad.dtype == torch.float32
    assert max_rel_err(scores_leaf.grad.cpu(), expected) <= 1e-5


@pytest.mark.parametrize("name", ["mixtral", "fine_grained", "wide", "imbalanced"])
def test_full_size_round_trip(name, device):
    """At the benchmark sizes: un-scored dispatch then combine returns k * x exactly (fp32 sum, one rounding), scored
    dispatch then un-scored combine returns x * sum(scores), and every real row holds the token the map says."""
    workload = WORKLOADS[name]
    inputs = make_inputs(workload, seed=5, weights=False)
    x = inputs.hidden_states.to(device)
    scores = inputs.scores.to(device)
    sparse_map = get_sparse_map(inputs.top_experts.to(device), workload.experts)
    k = workload.experts_per_token

    sparse = copy_dense_to_sparse(x, None, sparse_map)
    rows = sparse_map.sparse_rows.long()
    for j in (0, k - 1):
        assert torch.equal(sparse[rows[:, j]], x)
    back = copy_sparse_to_dense(sparse, None, sparse_map)
    assert torch.equal(back, (x.float() * k).to(x.dtype))

    weighted = copy_sparse_to_dense(sparse, scores, sparse_map)
    assert max_rel_err(weighted, x.float() * scores.sum(1, keepdim=True)) <= 1e-2  # softmax scores sum to 1

    grad_scores = copy_sparse_to_dense_grad_score(sparse, x, sparse_map)
    expected = (x.float() ** 2).sum(1, keepdim=True).expand(-1, k)  # <x_t, x_t> for every slot
    assert max_rel_err(grad_scores, expected) <= 1e-2


def test_rows_outside_the_sparse_buffer_are_skipped(device, library):
    """Entries of `sparse_rows` that are negative or not below the sparse buffer's row count (a map built for another
    buffer) are skipped by all four kernels, never dereferenced: such a slot copies nothing, adds nothing to the
    combine and gets score gradient 0. The Python wrappers refuse a buffer whose row count differs from the map's."""
    tokens, hidden, k, rows = 40, 256, 3, 128
    generator = torch.Generator().manual_seed(4)
    dense = torch.randn(tokens, hidden, generator=generator).to(torch.bfloat16)
    sparse = torch.randn(rows, hidden, generator=generator).to(torch.bfloat16)
    scores = torch.rand(tokens, k, generator=generator)
    sparse_rows = torch.randperm(rows, generator=generator)[: tokens * k].view(tokens, k).to(torch.int32)
    bad = torch.rand(tokens, k, generator=generator) < 0.3
    bad_values = torch.where(torch.rand(tokens, k, generator=generator) < 0.5, -1, rows + 1000)
    bad_rows = torch.where(bad, bad_values, sparse_rows).to(torch.int32)
    valid = (~bad).float()

    dense_d, sparse_d, scores_d, rows_d = (t.to(device) for t in (dense, sparse, scores, bad_rows))
    stream = torch.cuda.current_stream(device).cuda_stream
    shape = (tokens, hidden, k, rows)
    tags = (_lib.dtype_tag(torch.bfloat16), _lib.dtype_tag(torch.float32), _lib.index_tag(torch.int32), stream)

    out = torch.full((rows, hidden), 7.0, dtype=torch.bfloat16, device=device)
    _lib.check(library.fm_copy_dense_to_sparse(dense_d.data_ptr(), scores_d.data_ptr(), rows_d.data_ptr(),
                                               out.data_ptr(), *shape, *tags))  # fmt: skip
    expected = torch.full((rows, hidden), 7.0, dtype=torch.bfloat16)
    for t in range(tokens):
        for j in range(k):
            if not bad[t, j]:
                expected[sparse_rows[t, j]] = (dense[t].float() * scores[t, j]).to(torch.bfloat16)
    assert torch.equal(out.cpu(), expected)

    combined = torch.empty(tokens, hidden, dtype=torch.bfloat16, device=device)
    _lib.check(library.fm_copy_sparse_to_dense(sparse_d.data_ptr(), scores_d.data_ptr(), rows_d.data_ptr(),
                                               combined.data_ptr(), *shape, *tags))  # fmt: skip
    gathered = sparse[sparse_rows.long()].float() * (scores * valid)[:, :, None]
    assert max_rel_err(combined.cpu(), gathered.sum(1)) <= 1e-2

    grad_scores = torch.empty(tokens, k, dtype=torch.float32, device=device)
    grad_input = torch.full((rows, hidden), 7.0, dtype=torch.bfloat16, device=device)
    _lib.check(library.fm_copy_sparse_to_dense_backward(
        sparse_d.data_ptr(), dense_d.data_ptr(), scores_d.data_ptr(), rows_d.data_ptr(), grad_input.data_ptr(),
        grad_scores.data_ptr(), *shape, tags[0], tags[1], _lib.dtype_tag(torch.float32), tags[2], stream))  # fmt: skip
    expected_scores = (sparse[sparse_rows.long()].float() * dense.float()[:, None, :]).sum(-1) * valid
    assert max_rel_err(grad_scores.cpu(), expected_scores) <= 1e-5
    assert (grad_scores.cpu()[bad] == 0).all()
    assert torch.equal(grad_input.cpu(), expected)

    plain = torch.empty(tokens, k, dtype=torch.float32, device=device)
    _lib.check(library.fm_copy_sparse_to_dense_grad_score(
        sparse_d.data_ptr(), dense_d.data_ptr(), rows_d.data_ptr(), plain.data_ptr(), *shape, tags[0],
        _lib.dtype_tag(torch.float32), tags[2], stream))  # fmt: skip
    assert torch.equal(plain, grad_scores)

    oracle_map, _, _, _ = _problem(tokens, 4, 2, hidden, torch.bfloat16)
    sparse_map = to_device_map(oracle_map, device, torch.int32)
    with pytest.raises(AssertionError):
        copy_sparse_to_dense(torch.zeros(oracle_map.num_rows - 128, hidden, dtype=torch.bfloat16, device=device), None, sparse_map)
