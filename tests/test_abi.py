"""The C-ABI boundary without a GPU: the library loads, exports every symbol the header declares, and the host side
rejects bad calls with the reference's exception types before any kernel is launched."""

import ctypes
import pathlib
import re

import pytest
import torch

from fast_llm_amd import _lib
from fast_llm_amd.functional import sparse_copy, sparse_linear
from fast_llm_amd.functional.config import ActivationType, KernelConfig, MLPRecomputeLevel
from fast_llm_amd.functional.utils import div

HEADER = pathlib.Path(__file__).resolve().parent.parent / "include" / "fastmoe_hip.h"


def _declared_symbols() -> dict[str, int]:
    """name -> number of parameters, parsed from the header."""
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    symbols = {}
    for match in re.finditer(r"\b(?:int|int64_t|size_t|const char \*)\s*(fm_\w+)\s*\(([^)]*)\)\s*;", text):
        params = match.group(2).strip()
        symbols[match.group(1)] = 0 if params in ("", "void") else params.count(",") + 1
    return symbols


def test_header_symbols_are_bound_and_exported(library):
    declared = _declared_symbols()
    assert len(declared) >= 13
    assert set(declared) == set(_lib.SIGNATURES)
    raw = ctypes.CDLL(str(_lib.LIBRARY_PATH))
    for name, num_params in declared.items():
        assert hasattr(raw, name), f"{name} not exported"
        assert len(_lib.SIGNATURES[name][1]) == num_params, name
    assert library.fm_version() == _lib.FM_VERSION
    assert library.fm_last_error() == b""


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(_lib.FastMoeLibraryError, match="only compute path"):
        _lib.load_library(tmp_path / "libfastmoe_hip.so")


def test_workspace_size_is_host_only(library):
    assert library.fm_sparse_map_workspace_size(8192, 2, 8) >= (16 + 1) * 8 * 4
    assert library.fm_sparse_map_workspace_size(0, 2, 8) > 0
    assert library.fm_sparse_map_workspace_size(-1, 2, 8) == 0


def test_argument_validation_returns_status_and_message(library):
    # Validation happens before any HIP call, so it can be exercised without a device.
    status = library.fm_sparse_map(None, 4, 2, 0, 128, 1, None, None, None, None, 0, None)
    assert status == _lib.FM_ERR_INVALID_ARGUMENT
    assert b"num_experts" in library.fm_last_error()
    with pytest.raises(ValueError, match="num_experts"):
        _lib.check(status)
    status = library.fm_mlp_activation_forward(None, None, 4, 4, 1, 99, 1, None, 0, None)
    assert status == _lib.FM_ERR_INVALID_ARGUMENT and b"activation" in library.fm_last_error()
    status = library.fm_output_sparse_matmul(None, None, None, None, 128, 128, 64, 1, 64, 1, 1, 64, 128, 1, 0, 7, 0, 1, None, 0, None)
    assert status == _lib.FM_ERR_INVALID_ARGUMENT and b"dtype" in library.fm_last_error()
    status = library.fm_output_sparse_matmul(None, None, None, None, 128, 128, 64, 1, 64, 1, 1, 64, 128, 1, 0, 1, 1, 1, None, 64, None)
    assert status == _lib.FM_ERR_INVALID_ARGUMENT and b"workspace" in library.fm_last_error()


def test_grouped_gemm_workspace_size_depends_on_the_dimensions_only(library):
    partials = 512 * 256 * 256 * 4  # the pieces of a split last round
    record = 64  # bytes of the tile table per workgroup id

    def ids(row_tiles, column_tiles, split):  # whole rounds of 256 ids, then the pieces; +4: the table's 64-byte
        return -(-row_tiles * column_tiles // 256) * 256 + (512 if split else 0) + 4  # header, rounded up to 256 bytes

    # Layer 2 forward at the Mixtral shape: 68 + 8 row tiles x 16 column tiles, reduction 14336 -> splits.
    size = library.fm_grouped_gemm_workspace_size(17408, 4096, 14336, 8, 1)
    assert size == partials + ids(76, 16, True) * record
    assert library.fm_grouped_gemm_workspace_size(17408, 4096, 14336, 8, 2) == size
    assert library.fm_grouped_gemm_workspace_size(17408, 4096, 14336, 8, 0) == 0  # fp32: generic kernel
    # Layer 1 forward (29 rounds) and a short reduction are not split: the table only.
    assert library.fm_grouped_gemm_workspace_size(17408, 28672, 4096, 8, 1) == ids(76, 112, False) * record
    assert library.fm_grouped_gemm_workspace_size(17408, 4096, 1984, 8, 1) == ids(76, 16, False) * record
    # Dimensions the matrix-core kernel refuses whatever the strides (reduction not in whole 64-element slices, columns
    # not in whole 16-byte vectors): the generic kernel takes no workspace.
    assert library.fm_grouped_gemm_workspace_size(17408, 4096, 1000, 8, 1) == 0
    assert library.fm_grouped_gemm_workspace_size(17408, 4100, 4096, 8, 1) == 0
    assert library.fm_input_row_sparse_matmul_workspace_size(14340, 4096, 17408, 8, 1) == 0
    assert library.fm_grouped_gemm_workspace_size(0, 4096, 14336, 8, 1) == 0
    # The row-sparse product never splits: 8 experts x 56 row tiles x 16 column tiles.
    assert library.fm_input_row_sparse_matmul_workspace_size(14336, 4096, 17408, 8, 1) == ids(8 * 56, 16, False) * record
    assert library.fm_input_row_sparse_matmul_workspace_size(14336, 4096, 17408, 8, 0) == 0


def test_router_and_fused_entry_points_validate_before_launching(library):
    assert library.fm_router_workspace_size(8192, 8) >= 4 * (2 * 8 + 1)
    assert library.fm_router_workspace_size(0, 8) == 0
    fake = 256  # a non-null "pointer" that validation must never dereference
    args = dict(tokens=16, experts=8, k=2, shared=0)

    def forward(workspace_size=1 << 20, dtype=0, **overrides):
        a = {**args, **overrides}
        return library.fm_router_forward(fake, None, fake, fake, fake, fake, fake, fake, workspace_size, a["tokens"],
                                         a["experts"], a["k"], a["shared"], dtype, None)  # fmt: skip

    assert forward(experts=2000) == _lib.FM_ERR_INVALID_ARGUMENT and b"experts" in library.fm_last_error()
    assert forward(k=60, shared=10, experts=64) == _lib.FM_ERR_INVALID_ARGUMENT
    assert forward(k=9) == _lib.FM_ERR_INVALID_ARGUMENT and b"experts_per_token" in library.fm_last_error()
    assert forward(workspace_size=8) == _lib.FM_ERR_INVALID_ARGUMENT and b"workspace" in library.fm_last_error()
    assert forward(dtype=9) == _lib.FM_ERR_INVALID_ARGUMENT
    status = library.fm_router_backward(fake, fake, fake, fake, None, fake, fake, None, 0.0, 0.0, 16, 8, 2, 0, 0, None)
    assert status == _lib.FM_ERR_INVALID_ARGUMENT and b"null" in library.fm_last_error()

    # The fused products exist for the matrix-core kernel only: anything else is reported, not emulated.
    def fused(dtype=1, activation_dim=256, inner=128, activation=1, lhs_stride_inner=1):
        return library.fm_output_sparse_matmul_gated_activation(
            fake, fake, fake, fake, None, 256, activation_dim, inner, 1, inner, lhs_stride_inner, 1, inner, activation,
            dtype, 1, None,
        )  # fmt: skip

    assert fused(dtype=0) == _lib.FM_ERR_UNSUPPORTED and b"separately" in library.fm_last_error()
    with pytest.raises(NotImplementedError):
        _lib.check(_lib.FM_ERR_UNSUPPORTED)
    assert fused(activation_dim=200) == _lib.FM_ERR_UNSUPPORTED  # not a multiple of 128
    assert fused(inner=100) == _lib.FM_ERR_UNSUPPORTED  # reduction not in whole 64-element slices
    assert fused(lhs_stride_inner=2) == _lib.FM_ERR_UNSUPPORTED
    assert fused(activation=42) == _lib.FM_ERR_INVALID_ARGUMENT and b"activation" in library.fm_last_error()
    status = library.fm_output_sparse_matmul_gated_activation_backward(
        fake, fake, None, fake, None, None, 256, 256, 128, 1, 128, 1, 1, 128, 1, 1, 1, None
    )
    assert status == _lib.FM_ERR_INVALID_ARGUMENT and b"null" in library.fm_last_error()


def test_cpu_tensors_are_refused_not_emulated(library):
    top_experts = torch.zeros(4, 2, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="GPU"):
        sparse_copy.get_sparse_map(top_experts, 8)
    with pytest.raises(NotImplementedError):
        sparse_copy.get_sparse_map(top_experts, 8, use_triton=False)
    with pytest.raises(RuntimeError, match="GPU only"):
        sparse_linear.dense_matmul(torch.zeros(4, 4), torch.zeros(4, 4))


def test_shape_errors_follow_the_reference_conventions():
    sparse_map = sparse_copy.SparseMap(None, torch.tensor([128, 256]), torch.tensor([100, 200]), None, 256, None, 3, None)
    with pytest.raises(AssertionError):  # row_dim != num_rows
        sparse_linear.output_sparse_matmul(torch.zeros(128, 8), torch.zeros(8, 6), sparse_map)
    with pytest.raises(ValueError):  # columns not divisible by the expert count
        sparse_linear.output_sparse_matmul(torch.zeros(256, 8), torch.zeros(8, 8), sparse_map)
    with pytest.raises(AssertionError):  # accumulate without out
        sparse_linear.input_row_sparse_matmul(torch.zeros(8, 256), torch.zeros(256, 8), sparse_map, accumulate=True)
    with pytest.raises(ValueError):
        div(7, 2)


def test_enums_mirror_the_reference():
    assert [level.value for level in MLPRecomputeLevel] == ["none", "activation", "activation_and_input", "full"]
    assert MLPRecomputeLevel.full.recompute_layer_1 and not MLPRecomputeLevel.activation.recompute_sparse_input
    assert MLPRecomputeLevel("activation_and_input").recompute_sparse_input
    assert ActivationType.silu.value == "silu" and f"{ActivationType.gelu}" == "gelu"
    assert KernelConfig.POINTWISE_BLOCK_SIZE == 1024
