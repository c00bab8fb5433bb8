"""The committed golden vectors (`tests/golden/golden_small.npz`, written by `tests/golden/make_golden.py` from a
brute-force map and a float64 textbook mixture): the oracle must reproduce them on the CPU, the HIP path on the GPU."""

import numpy as np
import pytest
import torch

from oracle import moe_oracle
from tests.helpers import GOLDEN, max_rel_err

_RESULTS = ("output", "grad_input", "grad_scores", "grad_weight_1", "grad_weight_2")


@pytest.fixture(scope="module")
def golden() -> dict[str, torch.Tensor]:
    with np.load(GOLDEN / "golden_small.npz", allow_pickle=False) as data:
        return {key: torch.from_numpy(data[key]) for key in data.files}


def test_oracle_reproduces_golden_vectors(golden):
    experts = golden["expert_ends"].numel()
    sparse_map = moe_oracle.sparse_map(golden["top_experts"], experts)
    assert torch.equal(sparse_map.expert_ends, golden["expert_ends"])
    assert torch.equal(sparse_map.expert_pad_begins, golden["expert_pad_begins"])
    assert torch.equal(sparse_map.sparse_rows, golden["sparse_rows"])
    assert golden["expert_pad_begins"][2] == golden["expert_ends"][1]  # the empty expert
    result = moe_oracle.dropless_mlp_forward_backward(
        golden["hidden_states"], golden["scores"], golden["weight_1"], golden["weight_2"], sparse_map,
        golden["grad_output"],
    )
    looped = moe_oracle.looped_moe_forward_backward(
        golden["hidden_states"], golden["scores"], golden["top_experts"], golden["weight_1"], golden["weight_2"],
        experts, golden["grad_output"],
    )
    for name in _RESULTS:
        assert max_rel_err(getattr(result, name), golden[name]) <= 1e-5, name
        assert max_rel_err(getattr(looped, name), golden[name]) <= 1e-5, name


@pytest.mark.gpu
@pytest.mark.parametrize(("dtype", "tolerance"), [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)], ids=["fp32", "bf16"])
def test_hip_path_reproduces_golden_vectors(golden, dtype, tolerance, device):
    """fp32: max relative error 1e-5. bf16: the inputs themselves are rounded to bf16 (2^-9 each) before the MFMA
    path runs, so the bound against the float64 vectors is 2e-2 here; against the same-rounding oracle it is 1e-2
    (tests/test_gpu_mlp.py)."""
    from fast_llm_amd.functional.config import ActivationType, MLPRecomputeLevel
    from fast_llm_amd.functional.mlp import mlp_autograd
    from fast_llm_amd.functional.sparse_copy import get_sparse_map
    from fast_llm_amd.layers.moe import attach_grad_buffer

    experts = golden["expert_ends"].numel()
    sparse_map = get_sparse_map(golden["top_experts"].to(device), experts)
    assert torch.equal(sparse_map.expert_ends.cpu().long(), golden["expert_ends"])
    assert torch.equal(sparse_map.expert_pad_begins.cpu().long(), golden["expert_pad_begins"])
    assert torch.equal(sparse_map.sparse_rows.cpu().long(), golden["sparse_rows"])

    x = golden["hidden_states"].to(device=device, dtype=dtype).requires_grad_(True)
    scores = golden["scores"].to(device).requires_grad_(True)
    weight_1 = attach_grad_buffer(golden["weight_1"].to(device=device, dtype=dtype).requires_grad_(True))
    weight_2 = attach_grad_buffer(golden["weight_2"].to(device=device, dtype=dtype).requires_grad_(True))
    output = mlp_autograd(
        x, scores, weight_1, None, weight_2, None, True, ActivationType.silu, None, False, True,
        MLPRecomputeLevel.none, True, sparse_map,
    )
    output.backward(golden["grad_output"].to(device=device, dtype=dtype))
    actual = dict(zip(_RESULTS, (output, x.grad, scores.grad, weight_1.grad_buffer, weight_2.grad_buffer)))
    for name in _RESULTS:
        assert max_rel_err(actual[name].detach().cpu().float(), golden[name]) <= tolerance, name
