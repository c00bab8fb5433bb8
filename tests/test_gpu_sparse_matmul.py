"""The three grouped matrix products on the GPU: the reference's own fixtures and tolerances
(tests/functional/test_sparse_matmul.py), then layouts, dtypes, accumulation, padding and phantom rows."""

import pytest
import torch

from fast_llm_amd.functional.sparse_linear import (
    InputSparseLinear,
    OutputSparseLinear,
    dense_matmul,
    input_inner_sparse_matmul,
    input_row_sparse_matmul,
    output_sparse_matmul,
)
from oracle import moe_oracle
from tests.helpers import REFERENCE_FIXTURES, fixture_sparse_map, max_rel_err, rms_diff, to_device_map

pytestmark = pytest.mark.gpu

_CASES = REFERENCE_FIXTURES["sparse_matmul"]["cases"]
_STD = REFERENCE_FIXTURES["sparse_matmul"]["std"]
_RMS = REFERENCE_FIXTURES["sparse_matmul"]["rms_tolerance"]
# max|a - b| / max|b| per tensor: fp32 multiply-add vs bf16/fp16 operands with fp32 accumulation.
_MAX_REL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 2e-3}


def _normal(rows, columns, dtype, generator):
    return torch.normal(0, _STD, (rows, columns), generator=generator).to(dtype)


def _used_rows(oracle_map):
    return int(oracle_map.expert_ends[-1])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", _CASES)
@pytest.mark.parametrize("index_dtype", [torch.int64, torch.int16])
def test_output_sparse_matmul(case, dtype, index_dtype, device):
    generator = torch.Generator().manual_seed(0)
    oracle_map = fixture_sparse_map(case)
    sparse_map = to_device_map(oracle_map, device, index_dtype)
    lhs = _normal(oracle_map.num_rows, case["dense_dim"], dtype, generator)
    rhs = _normal(case["dense_dim"], case["sparse_dim"] * oracle_map.num_experts, dtype, generator)
    # Randomly initialize the output to ensure padded values have no effect.
    out = _normal(oracle_map.num_rows, case["sparse_dim"], dtype, generator).to(device)
    output = output_sparse_matmul(lhs.to(device), rhs.to(device), sparse_map, out)
    assert output is out
    expected = moe_oracle.output_sparse_matmul(lhs, rhs, oracle_map)
    assert rms_diff(output.cpu(), expected) <= _RMS
    assert max_rel_err(output.cpu(), expected) <= _MAX_REL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", _CASES)
def test_input_inner_sparse_matmul(case, dtype, device):
    generator = torch.Generator().manual_seed(1)
    oracle_map = fixture_sparse_map(case)
    sparse_map = to_device_map(oracle_map, device)
    lhs = _normal(oracle_map.num_rows, case["sparse_dim"], dtype, generator)
    rhs = _normal(case["sparse_dim"] * oracle_map.num_experts, case["dense_dim"], dtype, generator)
    output = input_inner_sparse_matmul(lhs.to(device), rhs.to(device), sparse_map)
    expected = moe_oracle.input_inner_sparse_matmul(lhs, rhs, oracle_map)
    assert rms_diff(output.cpu(), expected) <= _RMS
    assert max_rel_err(output.cpu(), expected) <= _MAX_REL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", _CASES)
def test_input_row_sparse_matmul(case, dtype, device):
    generator = torch.Generator().manual_seed(2)
    oracle_map = fixture_sparse_map(case)
    sparse_map = to_device_map(oracle_map, device)
    lhs = _normal(case["sparse_dim"], oracle_map.num_rows, dtype, generator)
    rhs = _normal(oracle_map.num_rows, case["dense_dim"], dtype, generator)
    output = input_row_sparse_matmul(lhs.to(device), rhs.to(device), sparse_map)
    expected = moe_oracle.input_row_sparse_matmul(lhs, rhs, oracle_map)
    assert rms_diff(output.cpu(), expected) <= _RMS
    assert max_rel_err(output.cpu(), expected) <= _MAX_REL[dtype]
    if 0 in case["tokens_per_expert"]:
        empty = case["tokens_per_expert"].index(0)
        assert (output[empty * case["sparse_dim"] : (empty + 1) * case["sparse_dim"]] == 0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", _CASES)
@pytest.mark.parametrize(
    ("autograd_class", "expert_axis"), [(OutputSparseLinear, 1), (InputSparseLinear, 0)], ids=["output", "input"]
)
def test_sparse_linear_autograd(case, dtype, autograd_class, expert_axis, device):
    """Mirror of the reference's `test_sparse_linear_autograd` (test_sparse_matmul.py:198-233): per-expert reference
    on the real rows, padded rows of out and grad_lhs zeroed before comparing."""
    generator = torch.Generator().manual_seed(3)
    oracle_map = fixture_sparse_map(case)
    sparse_map = to_device_map(oracle_map, device)
    experts, tokens = oracle_map.num_experts, oracle_map.num_rows
    if expert_axis == 1:
        lhs_features, out_features = case["dense_dim"], case["sparse_dim"]
        rhs_shape = (case["dense_dim"], case["sparse_dim"] * experts)
    else:
        lhs_features, out_features = case["sparse_dim"], case["dense_dim"]
        rhs_shape = (case["sparse_dim"] * experts, case["dense_dim"])
    lhs = _normal(tokens, lhs_features, dtype, generator)
    rhs = _normal(*rhs_shape, dtype, generator)
    grad_output = _normal(tokens, out_features, dtype, generator)

    lhs_ref = lhs.float().clone().requires_grad_(True)
    rhs_ref = rhs.float().clone().requires_grad_(True)
    out_ref = lhs_ref.new_zeros(tokens, out_features)
    begins = oracle_map.expert_begins.tolist()
    pad_begins = oracle_map.expert_pad_begins.tolist()
    for i, rhs_chunk in enumerate(rhs_ref.chunk(experts, dim=expert_axis)):
        out_ref[begins[i] : pad_begins[i]] = lhs_ref[begins[i] : pad_begins[i]] @ rhs_chunk
    out_ref.backward(grad_output.float())

    lhs_t = lhs.to(device).requires_grad_(True)
    rhs_t = rhs.to(device).requires_grad_(True)
    out_t = autograd_class.apply(lhs_t, rhs_t, sparse_map)
    out_t.backward(grad_output.to(device))

    def zero_padded(tensor):
        masked = tensor.detach().cpu().float().clone()
        masked[~oracle_map.real_row_mask()] = 0
        return masked

    tolerance = _MAX_REL[dtype]
    assert rms_diff(zero_padded(out_t), out_ref.detach()) <= _RMS
    assert rms_diff(zero_padded(lhs_t.grad), lhs_ref.grad) <= _RMS
    assert rms_diff(rhs_t.grad.cpu().float(), rhs_ref.grad) <= _RMS
    assert max_rel_err(zero_padded(out_t), out_ref.detach()) <= tolerance
    assert max_rel_err(zero_padded(lhs_t.grad), lhs_ref.grad) <= tolerance
    assert max_rel_err(rhs_t.grad.cpu().float(), rhs_ref.grad) <= tolerance


def _moe_layout(dtype, generator, rows_per_expert=(256, 0, 128, 384), tokens=(200, 0, 128, 300), phantom=256,
                hidden=256, ffn=384):
    """The operand layouts of the MoE layer (weights [E*N, H], transposed views) with an empty expert, a full one,
    ragged ones and a phantom tail."""
    ends, total = [], 0
    for rows in rows_per_expert:
        total += rows
        ends.append(total)
    case = {"expert_ends": ends, "tokens_per_expert": list(tokens)}
    oracle_map = fixture_sparse_map(case)
    oracle_map.num_rows = total + phantom
    experts = len(ends)
    x = _normal(oracle_map.num_rows, hidden, dtype, generator)
    y = _normal(oracle_map.num_rows, ffn, dtype, generator)
    weight = _normal(experts * ffn, hidden, dtype, generator)
    return oracle_map, x, y, weight


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_moe_layer_layouts_padding_and_phantom_rows(dtype, device):
    generator = torch.Generator().manual_seed(4)
    oracle_map, x, y, weight = _moe_layout(dtype, generator)
    sparse_map = to_device_map(oracle_map, device, torch.int16)
    used, tolerance = _used_rows(oracle_map), _MAX_REL[dtype]
    real = oracle_map.real_row_mask()
    x_gpu, y_gpu, weight_gpu = x.to(device), y.to(device), weight.to(device)

    # Layer-1-like: rhs = weight.t(), reduction-contiguous. Phantom rows of a pre-filled out must survive.
    out = torch.full((oracle_map.num_rows, weight.size(0) // 4), 7.0, dtype=dtype, device=device)
    output_sparse_matmul(x_gpu, weight_gpu.t(), sparse_map, out)
    expected = moe_oracle.output_sparse_matmul(x, weight.t(), oracle_map)
    assert max_rel_err(out[:used].cpu(), expected[:used]) <= tolerance
    assert (out[used:] == 7.0).all()

    # Layer-2-like: rhs = weight row-major, expert blocks along the reduction axis.
    out = input_inner_sparse_matmul(y_gpu, weight_gpu, sparse_map)
    expected = moe_oracle.input_inner_sparse_matmul(y, weight, oracle_map)
    assert max_rel_err(out[:used].cpu(), expected[:used]) <= tolerance

    # Weight gradient: lhs = y.t() (a transposed view), NaN/Inf in every padding and phantom row of both operands.
    y_poisoned, x_poisoned = y.clone(), x.clone()
    y_poisoned[~real] = float("nan")
    x_poisoned[~real] = float("inf")
    for out_dtype in (dtype, torch.float32):
        out = torch.full(weight.shape, 3.0, dtype=out_dtype, device=device)
        input_row_sparse_matmul(y_poisoned.to(device).t(), x_poisoned.to(device), sparse_map, out=out)
        expected = moe_oracle.input_row_sparse_matmul(y.t(), x, oracle_map, out=torch.zeros(weight.shape, dtype=out_dtype))
        assert torch.isfinite(out).all()
        assert max_rel_err(out.cpu(), expected) <= tolerance
        ffn = weight.size(0) // 4
        assert (out[ffn : 2 * ffn] == 0).all()  # the empty expert gets zeros, not stale memory
        # accumulate=True adds to what is there, including for the empty expert
        input_row_sparse_matmul(y_poisoned.to(device).t(), x_poisoned.to(device), sparse_map, out=out, accumulate=True)
        assert max_rel_err(out.cpu(), 2 * expected.float()) <= tolerance
        assert (out[ffn : 2 * ffn] == 0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_accumulate_and_wider_output(dtype, device):
    generator = torch.Generator().manual_seed(5)
    case = _CASES[0]
    oracle_map = fixture_sparse_map(case)
    sparse_map = to_device_map(oracle_map, device)
    lhs = _normal(oracle_map.num_rows, case["dense_dim"], dtype, generator)
    rhs = _normal(case["dense_dim"], case["sparse_dim"] * 3, dtype, generator)
    previous = _normal(oracle_map.num_rows, case["sparse_dim"], torch.float32, generator)
    out = previous.to(device)
    output_sparse_matmul(lhs.to(device), rhs.to(device), sparse_map, out, accumulate=True)
    expected = moe_oracle.output_sparse_matmul(lhs, rhs, oracle_map, out=previous.clone(), accumulate=True)
    assert out.dtype == torch.float32
    assert max_rel_err(out.cpu(), expected) <= _MAX_REL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize(("rows", "inner", "columns"), [(256, 128, 256), (384, 192, 128), (100, 70, 36), (1, 1, 1)])
def test_dense_matmul_and_odd_shapes(rows, inner, columns, dtype, device):
    generator = torch.Generator().manual_seed(6)
    lhs, rhs = _normal(rows, inner, dtype, generator), _normal(inner, columns, dtype, generator)
    expected = (lhs.float() @ rhs.float()).to(dtype)
    assert max_rel_err(dense_matmul(lhs.to(device), rhs.to(device)).cpu(), expected) <= _MAX_REL[dtype]
    assert max_rel_err(output_sparse_matmul(lhs.to(device), rhs.to(device), None).cpu(), expected) <= _MAX_REL[dtype]
    # transposed operands, consumed through their strides
    lhs_t, rhs_t = lhs.t().contiguous().to(device).t(), rhs.t().contiguous().to(device).t()
    assert max_rel_err(dense_matmul(lhs_t, rhs_t).cpu(), expected) <= _MAX_REL[dtype]


def test_results_are_bit_identical_from_run_to_run(device):
    generator = torch.Generator().manual_seed(7)
    oracle_map, x, y, weight = _moe_layout(torch.bfloat16, generator, hidden=512, ffn=512)
    sparse_map = to_device_map(oracle_map, device, torch.int16)
    x_gpu, y_gpu, weight_gpu = x.to(device), y.to(device), weight.to(device)
    used = _used_rows(oracle_map)
    first = (
        output_sparse_matmul(x_gpu, weight_gpu.t(), sparse_map)[:used],
        input_inner_sparse_matmul(y_gpu, weight_gpu, sparse_map)[:used],
        input_row_sparse_matmul(y_gpu.t(), x_gpu, sparse_map),
    )
    for _ in range(3):
        again = (
            output_sparse_matmul(x_gpu, weight_gpu.t(), sparse_map)[:used],
            input_inner_sparse_matmul(y_gpu, weight_gpu, sparse_map)[:used],
            input_row_sparse_matmul(y_gpu.t(), x_gpu, sparse_map),
        )
        for a, b in zip(first, again):
            assert torch.equal(a, b)


def _ragged_case(seed: int, experts: int, pad: int = 128):
    """Random expert sizes, some empty, some one token, padded to `pad`; plus phantom rows after the last expert."""
    generator = torch.Generator().manual_seed(seed)
    tokens = torch.randint(0, 700, (experts,), generator=generator)
    tokens[torch.randint(0, experts, (max(1, experts // 8),), generator=generator)] = 0
    tokens[int(torch.randint(0, experts, (1,), generator=generator))] = 1
    padded = (tokens + pad - 1) // pad * pad
    ends = torch.cumsum(padded, 0)
    return {
        "expert_ends": ends.tolist(),
        "tokens_per_expert": tokens.tolist(),
        "phantom_rows": pad * 2,
    }


# (experts, reduction size, per-expert size): more experts than a wavefront has lanes, an odd number of 64-wide
# reduction slices, partial row and column tiles, more tiles than one round of workgroups.
@pytest.mark.parametrize(("experts", "dense_dim", "sparse_dim"), [(70, 192, 264), (9, 320, 576), (130, 64, 72)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mfma_kernel_on_ragged_experts(experts, dense_dim, sparse_dim, dtype, device):
    case = _ragged_case(experts + dense_dim, experts)
    oracle_map = fixture_sparse_map(case)
    oracle_map.num_rows = case["expert_ends"][-1] + case["phantom_rows"]
    sparse_map = to_device_map(oracle_map, device, torch.int32)
    used = _used_rows(oracle_map)
    real = oracle_map.real_row_mask()
    generator = torch.Generator().manual_seed(11)
    tolerance = _MAX_REL[dtype]

    # Row-padded storage: the kernel must follow the strides.
    def strided(rows, columns):
        return _normal(rows, columns + 24, dtype, generator)[:, :columns]

    x, weight = strided(oracle_map.num_rows, dense_dim), strided(experts * sparse_dim, dense_dim)
    y = strided(oracle_map.num_rows, sparse_dim)
    x_gpu, y_gpu, weight_gpu = (
        torch.empty(t.size(0), t.size(1) + 24, dtype=dtype, device=device)[:, : t.size(1)] for t in (x, y, weight)
    )
    x_gpu.copy_(x), y_gpu.copy_(y), weight_gpu.copy_(weight)
    assert not x_gpu.is_contiguous()

    out = torch.full((oracle_map.num_rows, sparse_dim), 5.0, dtype=dtype, device=device)
    output_sparse_matmul(x_gpu, weight_gpu.t(), sparse_map, out)
    expected = moe_oracle.output_sparse_matmul(x, weight.t(), oracle_map)
    assert max_rel_err(out[:used].cpu(), expected[:used]) <= tolerance
    assert (out[used:] == 5.0).all()

    out = input_inner_sparse_matmul(y_gpu, weight_gpu, sparse_map)
    expected = moe_oracle.input_inner_sparse_matmul(y, weight, oracle_map)
    assert max_rel_err(out[:used].cpu(), expected[:used]) <= tolerance

    y_poisoned, x_poisoned = y_gpu.clone(), x_gpu.clone()
    y_poisoned[~real.to(device)] = float("nan")
    x_poisoned[~real.to(device)] = float("nan")
    for out_dtype in (dtype, torch.float32):
        out = torch.full((experts * sparse_dim, dense_dim), 3.0, dtype=out_dtype, device=device)
        input_row_sparse_matmul(y_poisoned.t(), x_poisoned, sparse_map, out=out)
        expected = moe_oracle.input_row_sparse_matmul(
            y.t(), x, oracle_map, out=torch.zeros(out.shape, dtype=out_dtype)
        )
        assert torch.isfinite(out).all()
        assert max_rel_err(out.cpu(), expected) <= tolerance
        input_row_sparse_matmul(y_poisoned.t(), x_poisoned, sparse_map, out=out, accumulate=True)
        assert max_rel_err(out.cpu(), 2 * expected.float()) <= tolerance


# The matrix-core kernel counts by hand which of its transfers have landed when a K-step reads them, with one count
# per load schedule (K-contiguous rhs, row-contiguous rhs, weight gradient) and tile kind (whole, half: an expert's last
# row tile with at most 128 valid rows). Every number of 64-wide reduction slices from 1 to 10 through all of them:
# experts of 256 + 128 rows (a whole and a half tile), of 128 rows (a half tile) and of 512 rows; one column tile, five
# whole ones followed by one of 72 columns, and the walk of a workgroup over several tiles with 40 column tiles.
@pytest.mark.parametrize(
    ("slices", "other"),
    [(slices, 256) for slices in range(1, 11)]
    + [(slices, 5 * 256 + 72) for slices in range(1, 11)]
    + [(slices, 40 * 256) for slices in (1, 2, 3, 6, 9)],
)
def test_every_slice_count_through_the_pipeline(slices, other, device):
    dtype = torch.bfloat16
    inner = 64 * slices
    case = {"expert_ends": [384, 512, 1024], "tokens_per_expert": [300, 77, 512], "phantom_rows": 128}
    oracle_map = fixture_sparse_map(case)
    oracle_map.num_rows = case["expert_ends"][-1] + case["phantom_rows"]
    sparse_map = to_device_map(oracle_map, device, torch.int32)
    used = _used_rows(oracle_map)
    experts = len(case["expert_ends"])
    generator = torch.Generator().manual_seed(slices)
    x = _normal(oracle_map.num_rows, inner, dtype, generator)
    x[~oracle_map.real_row_mask()] = 0
    x_gpu = x.to(device)

    weight = _normal(experts * other, inner, dtype, generator)  # K-contiguous rhs
    out = output_sparse_matmul(x_gpu, weight.to(device).t(), sparse_map)
    expected = moe_oracle.output_sparse_matmul(x, weight.t(), oracle_map)
    assert max_rel_err(out[:used].cpu(), expected[:used]) <= _MAX_REL[dtype]

    weight = _normal(experts * inner, other, dtype, generator)  # row-contiguous rhs
    out = input_inner_sparse_matmul(x_gpu, weight.to(device), sparse_map)
    expected = moe_oracle.input_inner_sparse_matmul(x, weight, oracle_map)
    assert max_rel_err(out[:used].cpu(), expected[:used]) <= _MAX_REL[dtype]

    if other == 256:  # the weight gradient: its reduction runs over the rows, 1 .. 8 slices here; 128 x 256 outputs
        y = _normal(oracle_map.num_rows, other, dtype, generator)
        narrow = _normal(oracle_map.num_rows, 128, dtype, generator)
        out = input_row_sparse_matmul(narrow.to(device).t(), y.to(device), sparse_map)
        expected = moe_oracle.input_row_sparse_matmul(narrow.t(), y, oracle_map)
        assert max_rel_err(out.cpu(), expected) <= _MAX_REL[dtype]


# Few tiles and a long reduction: the tiles of the last round of workgroups are cut along the reduction axis and their
# pieces added by a second kernel. (experts, reduction size, other size): 4 pieces of 18 slices with a shorter, odd last
# one; whole tiles followed by more than 256 pieces; 2 pieces.
@pytest.mark.parametrize(("experts", "inner", "other"), [(9, 4160, 320), (70, 2240, 600), (40, 4096, 256), (3, 2048, 264)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_split_reduction_of_last_round(experts, inner, other, dtype, device):
    case = _ragged_case(experts + inner, experts)
    oracle_map = fixture_sparse_map(case)
    oracle_map.num_rows = case["expert_ends"][-1] + case["phantom_rows"]
    sparse_map = to_device_map(oracle_map, device, torch.int32)
    used = _used_rows(oracle_map)
    generator = torch.Generator().manual_seed(13)
    tolerance = _MAX_REL[dtype]

    # output-sparse: [rows, inner] x per-expert [inner, other]
    x, weight = _normal(oracle_map.num_rows, inner, dtype, generator), _normal(experts * other, inner, dtype, generator)
    x_gpu, weight_gpu = x.to(device), weight.to(device)
    expected = moe_oracle.output_sparse_matmul(x, weight.t(), oracle_map)
    out = torch.full((oracle_map.num_rows, other), 5.0, dtype=dtype, device=device)
    output_sparse_matmul(x_gpu, weight_gpu.t(), sparse_map, out)
    assert max_rel_err(out[:used].cpu(), expected[:used]) <= tolerance
    assert (out[used:] == 5.0).all()
    again = torch.empty_like(out)
    output_sparse_matmul(x_gpu, weight_gpu.t(), sparse_map, again)
    assert torch.equal(out[:used], again[:used])
    # accumulation into a wider output
    previous = _normal(oracle_map.num_rows, other, torch.float32, generator)
    out = previous.to(device)
    output_sparse_matmul(x_gpu, weight_gpu.t(), sparse_map, out, accumulate=True)
    assert max_rel_err(out[:used].cpu(), (expected.float() + previous)[:used]) <= tolerance
    assert torch.equal(out[used:].cpu(), previous[used:])

    # input-inner-sparse: [rows, inner] x per-expert [inner, other], weight stored [experts * inner, other]
    weight = _normal(experts * inner, other, dtype, generator)
    out = input_inner_sparse_matmul(x_gpu, weight.to(device), sparse_map)
    expected = moe_oracle.input_inner_sparse_matmul(x, weight, oracle_map)
    assert max_rel_err(out[:used].cpu(), expected[:used]) <= tolerance
    # dense product through the same kernel
    expected = (x.float() @ weight[:inner].float()).to(dtype)
    assert max_rel_err(dense_matmul(x_gpu, weight[:inner].to(device)).cpu(), expected) <= tolerance


def test_split_does_not_depend_on_stream_or_history(device, library):
    """Whether the last round is split follows from the dimensions and the caller's choice of a workspace only: the
    same product on the default stream, on twenty fresh streams and captured into a graph on yet another stream that
    never ran it gives the same bits; without a workspace it gives the (reproducible) unsplit bits; a workspace that
    is too small is an error, never a silent change of plan."""
    from fast_llm_amd import _lib
    from fast_llm_amd.functional.config import KernelConfig

    experts, inner, other, dtype = 9, 4160, 320, torch.bfloat16
    case = _ragged_case(experts + inner, experts)
    oracle_map = fixture_sparse_map(case)
    sparse_map = to_device_map(oracle_map, device, torch.int32)
    rows = oracle_map.num_rows
    generator = torch.Generator().manual_seed(21)
    x, weight = _normal(rows, inner, dtype, generator).to(device), _normal(experts * other, inner, dtype, generator).to(device)
    split_size = library.fm_grouped_gemm_workspace_size(rows, other, inner, experts, _lib.dtype_tag(dtype))
    assert split_size > 128 << 20  # 512 partial tiles of 256 x 256 floats, then the tile table
    assert library.fm_grouped_gemm_workspace_size(rows, other, inner, experts, _lib.dtype_tag(torch.float32)) == 0
    # A short reduction is not split: the tile table only.
    assert 0 < library.fm_grouped_gemm_workspace_size(rows, other, 1024, experts, _lib.dtype_tag(dtype)) < 1 << 20

    def product():
        return output_sparse_matmul(x, weight.t(), sparse_map)

    expected = product()
    torch.cuda.synchronize()
    for _ in range(20):
        stream = torch.cuda.Stream(device=device)
        stream.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(stream):
            out = product()
        stream.synchronize()
        assert torch.equal(out, expected)

    stream = torch.cuda.Stream(device=device)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        captured = product()
    for _ in range(3):
        captured.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, expected)
        assert torch.equal(product(), expected)  # eager work between the replays

    KernelConfig.grouped_gemm_workspace = False
    try:
        unsplit = product()
        assert torch.equal(product(), unsplit)
    finally:
        KernelConfig.grouped_gemm_workspace = True
    assert not torch.equal(unsplit, expected)  # another order of the same sums
    assert max_rel_err(unsplit.cpu(), expected.cpu()) <= _MAX_REL[dtype]

    # Straight through the C ABI: a workspace one byte short.
    size = library.fm_grouped_gemm_workspace_size(rows, other, inner, experts, _lib.dtype_tag(dtype))
    small = torch.empty(size - 1, dtype=torch.uint8, device=device)
    out = torch.empty_like(expected)
    status = library.fm_output_sparse_matmul(
        x.data_ptr(), weight.data_ptr(), out.data_ptr(), sparse_map.expert_ends.data_ptr(), rows, other, inner, experts,
        x.stride(0), x.stride(1), 1, inner, other, 1, 0, _lib.dtype_tag(dtype), _lib.dtype_tag(dtype),
        _lib.index_tag(torch.int32), small.data_ptr(), size - 1, torch.cuda.current_stream(device).cuda_stream,
    )  # fmt: skip
    assert status == _lib.FM_ERR_INVALID_ARGUMENT and b"workspace" in library.fm_last_error()


def test_tile_table_changes_no_bit(device):
    """With a workspace the workgroups read where their tiles lie from a table written by a small kernel, without one
    each scans the expert map itself: the same tiles either way, so products that are not split are bit-identical
    (ragged experts with half tiles, an empty expert, all three products, accumulation into fp32)."""
    from fast_llm_amd.functional.config import KernelConfig

    experts, inner, other, dtype = 7, 192, 328, torch.bfloat16
    case = _ragged_case(1500, experts)
    oracle_map = fixture_sparse_map(case)
    sparse_map = to_device_map(oracle_map, device, torch.int32)
    rows = oracle_map.num_rows
    generator = torch.Generator().manual_seed(5)
    x = _normal(rows, inner, dtype, generator).to(device)
    y = _normal(rows, other, dtype, generator).to(device)
    weight = _normal(experts * other, inner, dtype, generator).to(device)
    previous = torch.randn(experts * other, inner, generator=generator).to(device)

    def products():
        return (
            output_sparse_matmul(x, weight.t(), sparse_map),
            input_inner_sparse_matmul(y, weight, sparse_map),
            input_row_sparse_matmul(y.t(), x, sparse_map),
            input_row_sparse_matmul(y.t(), x, sparse_map, out=previous.clone(), accumulate=True),
        )

    with_table = products()
    KernelConfig.grouped_gemm_workspace = False
    try:
        without = products()
    finally:
        KernelConfig.grouped_gemm_workspace = True
    valid = sparse_map.expert_ends[-1].item()
    for a, b in zip(with_table[:2], without[:2]):
        assert torch.equal(a[:valid], b[:valid])
    for a, b in zip(with_table[2:], without[2:]):
        assert torch.equal(a, b)


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes_through_the_matrix_core_kernel(seed, device):
    """A sweep over ragged expert layouts and sizes around the kernel's tile (256 x 256 x 64), slice-pair and
    split-reduction boundaries; all three products, random accumulation and output width."""
    generator = torch.Generator().manual_seed(1000 + seed)

    def pick(*choices):
        return choices[int(torch.randint(0, len(choices), (1,), generator=generator))]

    experts = pick(1, 3, 8, 20)
    inner = pick(64, 128, 192, 448, 2048, 2112, 4160)
    other = pick(8, 72, 256, 264, 520)
    dtype = pick(torch.bfloat16, torch.float16)
    case = _ragged_case(seed, experts)
    oracle_map = fixture_sparse_map(case)
    oracle_map.num_rows = case["expert_ends"][-1] + case["phantom_rows"]
    sparse_map = to_device_map(oracle_map, device, pick(torch.int16, torch.int32, torch.int64))
    used = _used_rows(oracle_map)
    tolerance = _MAX_REL[dtype]
    rows = oracle_map.num_rows
    x = _normal(rows, inner, dtype, generator)
    x[~oracle_map.real_row_mask()] = 0  # padding rows hold zeros here so that every product is finite
    x_gpu = x.to(device)

    # output-sparse
    weight = _normal(experts * other, inner, dtype, generator)
    out_dtype = pick(dtype, torch.float32)
    accumulate = pick(False, True)
    previous = _normal(rows, other, out_dtype, generator)
    out = previous.to(device)
    output_sparse_matmul(x_gpu, weight.to(device).t(), sparse_map, out, accumulate=accumulate)
    expected = moe_oracle.output_sparse_matmul(x, weight.t(), oracle_map, out=previous.clone(), accumulate=accumulate)
    assert max_rel_err(out[:used].cpu(), expected[:used]) <= tolerance
    assert torch.equal(out[used:].cpu(), previous[used:])

    # input-inner-sparse
    weight = _normal(experts * inner, other, dtype, generator)
    out = input_inner_sparse_matmul(x_gpu, weight.to(device), sparse_map)
    expected = moe_oracle.input_inner_sparse_matmul(x, weight, oracle_map)
    assert max_rel_err(out[:used].cpu(), expected[:used]) <= tolerance

    # input-row-sparse: the reduction runs over the (ragged) rows
    y = _normal(rows, other, dtype, generator)
    out_dtype = pick(dtype, torch.float32)
    out = torch.full((experts * inner, other), 2.0, dtype=out_dtype, device=device)
    input_row_sparse_matmul(x_gpu.t(), y.to(device), sparse_map, out=out)
    expected = moe_oracle.input_row_sparse_matmul(x.t(), y, oracle_map, out=torch.zeros(out.shape, dtype=out_dtype))
    assert max_rel_err(out.cpu(), expected) <= tolerance


@pytest.mark.parametrize("pad", [32, 8, 1])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_expert_boundaries_inside_a_tile(pad, dtype, device):
    """Expert blocks padded to less than a kernel tile (`get_sparse_map(pad_to_multiple=...)` allows any multiple):
    tiles that straddle expert boundaries are computed expert by expert, in the fp32 multiply-add kernel (64-row
    blocks) and in the matrix-core kernel (tiles enumerated per expert) alike."""
    experts, inner, other = 7, 64, 72
    case = _ragged_case(pad, experts, pad=pad)
    oracle_map = fixture_sparse_map(case)
    oracle_map.num_rows = case["expert_ends"][-1] + case["phantom_rows"]
    assert any(end % 64 for end in case["expert_ends"])
    sparse_map = to_device_map(oracle_map, device, torch.int32)
    used = _used_rows(oracle_map)
    generator = torch.Generator().manual_seed(17)
    x = _normal(oracle_map.num_rows, inner, dtype, generator)
    x[~oracle_map.real_row_mask()] = 0
    weight = _normal(experts * other, inner, dtype, generator)
    tolerance = _MAX_REL[dtype]

    out = torch.full((oracle_map.num_rows, other), 5.0, dtype=dtype, device=device)
    output_sparse_matmul(x.to(device), weight.to(device).t(), sparse_map, out)
    expected = moe_oracle.output_sparse_matmul(x, weight.t(), oracle_map)
    assert max_rel_err(out[:used].cpu(), expected[:used]) <= tolerance
    assert (out[used:] == 5.0).all()

    weight_inner = _normal(experts * inner, other, dtype, generator)
    out = input_inner_sparse_matmul(x.to(device), weight_inner.to(device), sparse_map)
    expected = moe_oracle.input_inner_sparse_matmul(x, weight_inner, oracle_map)
    assert max_rel_err(out[:used].cpu(), expected[:used]) <= tolerance

    y = _normal(oracle_map.num_rows, other, dtype, generator)
    out = input_row_sparse_matmul(x.to(device).t(), y.to(device), sparse_map)
    expected = moe_oracle.input_row_sparse_matmul(x.t(), y, oracle_map)
    assert max_rel_err(out.cpu(), expected) <= tolerance


def test_half_precision_on_the_generic_kernel_warns(device):
    """bf16 operands the matrix-core kernel cannot take (here: a reduction that is not a multiple of 64) still give the
    right product, from the multiply-add kernel, and the wrapper says so."""
    generator = torch.Generator().manual_seed(19)
    lhs, rhs = _normal(130, 100, torch.bfloat16, generator), _normal(100, 72, torch.bfloat16, generator)
    with pytest.warns(RuntimeWarning, match="generic multiply-add kernel"):
        out = dense_matmul(lhs.to(device), rhs.to(device))
    assert max_rel_err(out.cpu(), (lhs.float() @ rhs.float()).to(torch.bfloat16)) <= 1e-2
    import warnings

    with warnings.catch_warnings():
        warnings.simplefilter("error")
        dense_matmul(_normal(128, 128, torch.bfloat16, generator).to(device), _normal(128, 72, torch.bfloat16, generator).to(device))
        dense_matmul(lhs.float().to(device), rhs.float().to(device))  # fp32 belongs on that kernel: no remark


def test_one_expert_of_more_than_4_gib(device):
    """An expert whose rows span more than 4 GiB of a row-major operand (528 384 rows of 4096 bf16 values = 4.33 GB,
    after a first expert of 256 rows): byte offsets inside one expert's block exceed 32 bits in all three products,
    along the rows of the output-sparse and inner-sparse products and along the reduction of the row-sparse one
    (8256 slices of 64). Operands are drawn on the GPU and the checker is the oracle evaluated there in fp32: on the CPU
    it would take minutes."""
    dtype, wide, narrow = torch.bfloat16, 4096, 256
    case = {"expert_ends": [256, 256 + 528384], "tokens_per_expert": [200, 528300]}
    oracle_map = fixture_sparse_map(case)
    sparse_map = to_device_map(oracle_map, device)
    rows = oracle_map.num_rows
    assert (rows - 256) * wide * dtype.itemsize > 2**32
    generator = torch.Generator(device=device).manual_seed(5)

    def normal(*shape):
        return torch.empty(shape, dtype=dtype, device=device).normal_(0, _STD, generator=generator)

    x, y = normal(rows, wide), normal(rows, narrow)
    weight = normal(2 * narrow, wide)
    # Output-sparse: [rows, 4096] x [4096, 2 * 256] -> [rows, 256]; the lhs block of the second expert is the large one.
    out = output_sparse_matmul(x, weight.t(), sparse_map)
    expected = moe_oracle.output_sparse_matmul(x.float(), weight.t().float(), oracle_map)
    assert max_rel_err(out, expected) <= _MAX_REL[dtype]
    # Inner-sparse: [rows, 256] x [2 * 256, 4096] -> [rows, 4096]; the output block of the second expert.
    out = input_inner_sparse_matmul(y, weight, sparse_map)
    expected = moe_oracle.input_inner_sparse_matmul(y.float(), weight.float(), oracle_map)
    assert max_rel_err(out, expected) <= _MAX_REL[dtype]
    assert max_rel_err(out[-512:], expected[-512:]) <= _MAX_REL[dtype]
    del out, expected
    # Row-sparse: [256, rows] x [rows, 4096] -> [2 * 256, 4096]; the reduction runs down the large block, padding
    # rows (poisoned) excluded.
    real = oracle_map.real_row_mask().to(device)
    x[~real] = float("nan")
    y[~real] = float("nan")
    out = input_row_sparse_matmul(y.t(), x, sparse_map)
    x[~real] = 0
    y[~real] = 0
    expected = moe_oracle.input_row_sparse_matmul(y.t().float(), x.float(), oracle_map)
    assert torch.isfinite(out).all()
    assert max_rel_err(out, expected) <= _MAX_REL[dtype]
    assert max_rel_err(out[:narrow], expected[:narrow]) <= _MAX_REL[dtype]


@pytest.mark.parametrize("block", range(4))
def test_random_launches_of_many_rounds(block, device):
    """Random ragged layouts large enough for launches of several rounds of workgroups (hundreds to thousands of tiles:
    the tile table, a workgroup walking from tile to tile, half tiles, experts without tokens, split last rounds),
    all three products. Operands are drawn on the GPU and the checker is the oracle evaluated there in fp32."""
    for seed in range(30 * block, 30 * (block + 1)):
        generator = torch.Generator().manual_seed(5000 + seed)

        def pick(*choices):
            return choices[int(torch.randint(0, len(choices), (1,), generator=generator))]

        experts = pick(2, 5, 8, 16, 40)
        inner = pick(64, 192, 448, 768, 1408, 2048, 4096)
        other = pick(256, 520, 1024, 1408, 2112)
        dtype = pick(torch.bfloat16, torch.float16)
        tokens = torch.randint(0, pick(300, 900, 2500), (experts,), generator=generator)
        if pick(True, False):
            tokens[int(torch.randint(0, experts, (1,), generator=generator))] = 0
        ends = torch.cumsum((tokens + 127) // 128 * 128, 0)
        if int(ends[-1]) == 0:
            continue
        oracle_map = fixture_sparse_map({"expert_ends": ends.tolist(), "tokens_per_expert": tokens.tolist()})
        sparse_map = to_device_map(oracle_map, device, pick(torch.int32, torch.int64))
        device_generator = torch.Generator(device=device).manual_seed(seed)

        def normal(*shape):
            return torch.empty(shape, dtype=dtype, device=device).normal_(0, 0.5, generator=device_generator)

        x = normal(oracle_map.num_rows, inner)
        x[~oracle_map.real_row_mask().to(device)] = 0
        case = f"seed {seed}: {experts} experts, inner {inner}, other {other}, {dtype}, {oracle_map.num_rows} rows"
        weight = normal(experts * other, inner)
        out = output_sparse_matmul(x, weight.t(), sparse_map)
        expected = moe_oracle.output_sparse_matmul(x.float(), weight.t().float(), oracle_map)
        assert max_rel_err(out, expected) <= _MAX_REL[dtype], case
        weight = normal(experts * inner, other)
        out = input_inner_sparse_matmul(x, weight, sparse_map)
        expected = moe_oracle.input_inner_sparse_matmul(x.float(), weight.float(), oracle_map)
        assert max_rel_err(out, expected) <= _MAX_REL[dtype], case
        y = normal(oracle_map.num_rows, other)
        out = input_row_sparse_matmul(x.t(), y, sparse_map)
        expected = moe_oracle.input_row_sparse_matmul(x.t().float(), y.float(), oracle_map)
        assert max_rel_err(out, expected) <= _MAX_REL[dtype], case
