"""
Constants and enums of the MoE hot path (reference: fast_llm/functional/config.py:8-60,106).
"""

import enum
import typing

if typing.TYPE_CHECKING:
    import torch


class KernelConfig:
    """
    Counterpart of the reference's `TritonConfig` switch (fast_llm/functional/config.py:8-28). The reference chooses
    between Triton kernels and a torch path; here the HIP kernels are the only path, so the switch can only confirm
    that or refuse.
    """

    POINTWISE_BLOCK_SIZE = 1024
    # Whether a gated sparse MLP's activation runs in the epilogue of the neighbouring grouped product (layer 1 forward;
    # layer 2 input gradient) where the shapes allow. Results are bit-identical either way. None (default): chosen per
    # call, fused exactly where it was measured faster on MI355X, which is the layer 1 forward whose own output is not
    # stored (inference, `MLPRecomputeLevel.full`: 3.27 ms against 3.14 + 0.24 ms at the Mixtral shape). Where layer
    # 1's output is kept the fused kernels are slower (forward 3.45 ms against 3.06 + 0.24 ms, layer 2 input gradient
    # 2.15 ms against 1.56 + 0.40 ms): the matrix-core kernel runs one wavefront per SIMD, so the exponentials and
    # reciprocals of the epilogue run with nothing to overlap them, while the separate streaming kernel does the same
    # arithmetic at full occupancy behind its memory traffic. True: fuse both wherever possible; False: never.
    fuse_activation: bool | None = None
    # Hand the grouped products their scratch: a table of where every tile of a launch lies, written by a small
    # kernel before the product (the product's workgroups then look their tiles up instead of each scanning the expert
    # map), and the space with which a launch of few, long tiles (layer 2 forward and the layer 1 input gradient at
    # the Mixtral shape: 4.1 rounds of tiles on 256 CUs) cuts the reductions of its last round's tiles into pieces
    # that fill the idle CUs. Split and unsplit sums differ in the last bits; with a fixed setting results are
    # reproducible whatever the stream or allocator state.
    grouped_gemm_workspace = True

    @classmethod
    def enabled(cls, device: "torch.device|None" = None, default: bool | None = None) -> bool:
        if default is False:
            raise NotImplementedError(
                "use_triton=False asks for the reference's torch path; this package only has the HIP kernel path"
            )
        if device is not None and device.type != "cuda":
            raise RuntimeError(f"the HIP kernels need a GPU tensor, got device `{device}`")
        return True


# The reference's name for the switch, kept so call sites read the same.
TritonConfig = KernelConfig


class MLPRecomputeLevel(str, enum.Enum):
    none = "none"
    activation = "activation"
    activation_and_input = "activation_and_input"
    full = "full"

    def __str__(self) -> str:
        return self.value

    @property
    def recompute_layer_1(self) -> bool:
        return self == MLPRecomputeLevel.full

    @property
    def recompute_activation(self) -> bool:
        return self != MLPRecomputeLevel.none

    @property
    def recompute_sparse_input(self) -> bool:
        return self in (MLPRecomputeLevel.full, MLPRecomputeLevel.activation_and_input)


class ActivationType(str, enum.Enum):
    gelu = "gelu"
    silu = "silu"
    relu = "relu"
    sigmoid = "sigmoid"
    squared_relu = "squared_relu"
    identity = "identity"

    def __str__(self) -> str:
        return self.value

    @property
    def activation_fn(self) -> typing.Callable[["torch.Tensor"], "torch.Tensor"]:
        import torch

        return {
            ActivationType.gelu: lambda x: torch.nn.functional.gelu(x, approximate="tanh"),
            ActivationType.silu: torch.nn.functional.silu,
            ActivationType.relu: torch.nn.functional.relu,
            ActivationType.sigmoid: torch.nn.functional.sigmoid,
            ActivationType.squared_relu: lambda x: torch.pow(torch.nn.functional.relu(x), 2),
            ActivationType.identity: lambda x: x,
        }[self]


# Expert blocks of the sparse layout are padded to this many rows; the grouped GEMMs rely on it.
MAX_DROPLESS_BLOCK_SIZE_ROW = 128
