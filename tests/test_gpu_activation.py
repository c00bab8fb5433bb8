"""MLP activation kernels on the GPU: the reference's test (tests/functional/test_triton_kernels.py:167-193) plus
half precision and wide rows."""

import pytest
import torch

from fast_llm_amd.functional.config import ActivationType
from fast_llm_amd.functional.mlp import mlp_activation_backward, mlp_activation_forward, torch_mlp_activation
from oracle import moe_oracle
from tests.helpers import REFERENCE_FIXTURES, max_rel_err, rms_diff

pytestmark = pytest.mark.gpu
_FIXTURE = REFERENCE_FIXTURES["activation"]


@pytest.mark.parametrize("gated", [True, False])
@pytest.mark.parametrize("activation", _FIXTURE["activations"])
@pytest.mark.parametrize("recompute", [True, False])
def test_mlp_activation_reference_case(gated, activation, recompute, device):
    activation = ActivationType(activation)
    torch.manual_seed(0)
    rows, columns = _FIXTURE["rows"], _FIXTURE["columns"]
    input_cpu = torch.randn(rows, columns * (2 if gated else 1))
    grad_cpu = torch.randn(rows, columns)
    input_ = input_cpu.to(device).requires_grad_(True)
    output_grad = grad_cpu.to(device)

    output1, context = mlp_activation_forward(input_, gated, activation)
    input_grad1, output3 = mlp_activation_backward(output_grad, context, recompute)

    output2 = torch_mlp_activation(input_, gated, activation)
    output2.backward(output_grad)
    tolerance = _FIXTURE["rms_tolerance"]
    assert rms_diff(output1, output2.detach()) <= tolerance
    assert rms_diff(input_grad1, input_.grad) <= tolerance
    if recompute:
        assert rms_diff(output1, output3) <= tolerance
        assert torch.equal(output1, output3)  # recomputation must not change a bit
    else:
        assert output3 is None

    # and against the CPU oracle
    expected = moe_oracle.mlp_activation_forward(input_cpu, gated, activation.value)
    expected_grad, _ = moe_oracle.mlp_activation_backward(grad_cpu, input_cpu, gated, activation.value)
    assert max_rel_err(output1.cpu(), expected) <= 1e-5
    assert max_rel_err(input_grad1.cpu(), expected_grad) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize(("rows", "columns"), [(128, 14336), (257, 1408), (3, 100), (5, 7)])
def test_gated_silu_shapes_and_dtypes(rows, columns, dtype, device):
    generator = torch.Generator().manual_seed(1)
    input_cpu = (torch.randn(rows, 2 * columns, generator=generator) * 3).to(dtype)
    grad_cpu = torch.randn(rows, columns, generator=generator).to(dtype)
    output, context = mlp_activation_forward(input_cpu.to(device), True, ActivationType.silu)
    grad_input, recomputed = mlp_activation_backward(grad_cpu.to(device), context, True)
    expected = moe_oracle.mlp_activation_forward(input_cpu, True, "silu")
    expected_grad, _ = moe_oracle.mlp_activation_backward(grad_cpu, input_cpu, True, "silu")
    tolerance = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 2e-3}[dtype]
    assert max_rel_err(output.cpu(), expected) <= tolerance
    assert max_rel_err(grad_input.cpu(), expected_grad) <= tolerance
    assert torch.equal(output, recomputed)


def test_silu_extremes_are_finite(device):
    x = torch.tensor([[-200.0, -88.0, -20.0, 0.0, 20.0, 88.0, 200.0, 0.0]], device=device)
    output, context = mlp_activation_forward(x, False, ActivationType.silu)
    grad, _ = mlp_activation_backward(torch.ones_like(x), context)
    assert torch.isfinite(output).all() and torch.isfinite(grad).all()
    torch.testing.assert_close(grad[0, [0, 3, 6]].cpu(), torch.tensor([0.0, 0.5, 1.0]))


def test_sigmoid_has_no_kernel(device):
    with pytest.raises(NotImplementedError):
        mlp_activation_forward(torch.zeros(2, 4, device=device), False, ActivationType.sigmoid)


@pytest.mark.parametrize("index_dtype", [torch.int16, torch.int32, torch.int64])
@pytest.mark.parametrize("limit", [0, 1, 37, 64, 200])
def test_rows_past_the_limit_are_left_alone(limit, index_dtype, device, library):
    """With a device-side row limit (the last entry of a sparse map's `expert_ends`) the kernels neither read nor write
    the rows after it: outputs keep their sentinel there, rows before it equal the unlimited result, and NaN stored in
    the skipped input rows changes nothing."""
    from fast_llm_amd import _lib

    rows, columns = 64, 384
    generator = torch.Generator().manual_seed(limit)
    input_ = torch.randn(rows, 2 * columns, generator=generator).to(torch.bfloat16).to(device)
    grad_output = torch.randn(rows, columns, generator=generator).to(torch.bfloat16).to(device)
    expected, context = mlp_activation_forward(input_, True, ActivationType.silu)
    expected_grad, _ = mlp_activation_backward(grad_output, context)
    used = min(limit, rows)
    input_[used:] = float("nan")
    ends = torch.tensor([5, limit], dtype=index_dtype, device=device)
    limit_pointer = ends.data_ptr() + ends.element_size()
    stream = torch.cuda.current_stream(device).cuda_stream
    tags = (1, _lib.ACTIVATIONS["silu"], _lib.dtype_tag(torch.bfloat16), limit_pointer, _lib.index_tag(index_dtype), stream)

    output = torch.full((rows, columns), 3.0, dtype=torch.bfloat16, device=device)
    _lib.check(library.fm_mlp_activation_forward(input_.data_ptr(), output.data_ptr(), rows, columns, *tags))
    assert torch.equal(output[:used], expected[:used]) and (output[used:] == 3.0).all()

    grad_input = torch.full((rows, 2 * columns), 3.0, dtype=torch.bfloat16, device=device)
    recomputed = torch.full((rows, columns), 3.0, dtype=torch.bfloat16, device=device)
    _lib.check(
        library.fm_mlp_activation_backward(
            grad_output.data_ptr(), grad_input.data_ptr(), input_.data_ptr(), recomputed.data_ptr(), rows, columns, *tags
        )
    )
    assert torch.equal(grad_input[:used], expected_grad[:used]) and (grad_input[used:] == 3.0).all()
    assert torch.equal(recomputed[:used], expected[:used]) and (recomputed[used:] == 3.0).all()
