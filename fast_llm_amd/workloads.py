"""
The synthetic workloads of the MoE hot path: the five benchmark/parity configurations and their seeded inputs.

Inputs are generated on the CPU from a seed (so a CPU checker and the GPU see identical bits) and router logits are
computed once in fp32: top-k is discontinuous, and recomputing the logits per device flips experts for near-tie tokens.
"""

import dataclasses

import torch


@dataclasses.dataclass(frozen=True)
class MoEWorkload:
    name: str
    tokens: int
    hidden: int
    ffn: int
    experts: int
    experts_per_token: int
    dtype: torch.dtype
    zipf_exponent: float | None = None  # per-expert logit bias log(p_e), p_e ~ (e + 1) ** -s
    empty_experts: tuple[int, ...] = ()  # experts masked out of the routing (forced-empty blocks)

    @property
    def sparse_rows_unpadded(self) -> int:
        return self.tokens * self.experts_per_token

    @property
    def gemm_flops(self) -> int:
        """Forward + backward of the gated MLP on the unpadded rows: 18 * M * H * F."""
        return 18 * self.sparse_rows_unpadded * self.hidden * self.ffn

    @property
    def copy_bytes(self) -> int:
        """Algorithmic bytes of one dispatch or combine: (1 + k) * T * H * itemsize."""
        return (1 + self.experts_per_token) * self.tokens * self.hidden * self.dtype.itemsize


WORKLOADS: dict[str, MoEWorkload] = {
    workload.name: workload
    for workload in (
        MoEWorkload("tiny", 512, 256, 512, 8, 2, torch.float32),
        MoEWorkload("mixtral", 8192, 4096, 14336, 8, 2, torch.bfloat16),
        MoEWorkload("fine_grained", 16384, 2048, 1408, 64, 6, torch.bfloat16),
        MoEWorkload("wide", 16384, 2048, 768, 128, 8, torch.bfloat16),
        MoEWorkload("imbalanced", 8192, 4096, 14336, 8, 2, torch.bfloat16, zipf_exponent=1.2),
    )
}


@dataclasses.dataclass
class MoEInputs:
    hidden_states: torch.Tensor  # [T, H]
    grad_output: torch.Tensor  # [T, H]
    weight_1: torch.Tensor  # [E * 2F, H], per expert [gate; up]
    weight_2: torch.Tensor  # [E * F, H]
    logits: torch.Tensor  # [T, E] fp32
    scores: torch.Tensor  # [T, k] fp32
    top_experts: torch.Tensor  # [T, k] int64

    def to(self, device: torch.device | str) -> "MoEInputs":
        return MoEInputs(**{field.name: getattr(self, field.name).to(device) for field in dataclasses.fields(self)})


def make_inputs(
    workload: MoEWorkload, seed: int = 0, weights: bool = True, weight_device: torch.device | None = None
) -> MoEInputs:
    """
    x, grad ~ N(0, 1); router and expert weights ~ N(0, 0.02); top-k routing with fp32 softmax over the top logits.
    Everything is drawn on the CPU unless `weight_device` is given: then the (large) expert weights are drawn there
    from a generator of that device, which is much faster but not bit-reproducible on another device.
    """
    generator = torch.Generator().manual_seed(seed)

    def normal(shape, std):
        return torch.empty(shape, dtype=torch.float32).normal_(0, std, generator=generator)

    hidden_states = normal((workload.tokens, workload.hidden), 1.0)
    grad_output = normal((workload.tokens, workload.hidden), 1.0)
    router_weight = normal((workload.experts, workload.hidden), 0.02)
    logits = hidden_states @ router_weight.t()
    if workload.zipf_exponent is not None:
        probabilities = torch.arange(1, workload.experts + 1, dtype=torch.float32) ** -workload.zipf_exponent
        logits = logits + (probabilities / probabilities.sum()).log()
    for expert in workload.empty_experts:
        logits[:, expert] = float("-inf")
    top_logits, top_experts = torch.topk(logits, k=workload.experts_per_token, dim=-1)
    scores = torch.softmax(top_logits, dim=-1, dtype=torch.float32)
    if weights and weight_device is not None:
        device_generator = torch.Generator(device=weight_device).manual_seed(seed)
        weight_1, weight_2 = (
            torch.empty((workload.experts * width, workload.hidden), dtype=workload.dtype, device=weight_device).normal_(
                0, 0.02, generator=device_generator
            )
            for width in (2 * workload.ffn, workload.ffn)
        )
    elif weights:
        weight_1 = torch.empty((workload.experts * 2 * workload.ffn, workload.hidden), dtype=workload.dtype)
        weight_2 = torch.empty((workload.experts * workload.ffn, workload.hidden), dtype=workload.dtype)
        # Filled in slabs so the fp32 staging buffer stays small next to the 1.9 GB bf16 weight.
        for weight in (weight_1, weight_2):
            for slab in weight.chunk(max(1, weight.numel() // (1 << 26))):
                slab.copy_(normal(slab.shape, 0.02))
    else:
        weight_1 = weight_2 = torch.empty(0, dtype=workload.dtype)
    return MoEInputs(
        hidden_states=hidden_states.to(workload.dtype),
        grad_output=grad_output.to(workload.dtype),
        weight_1=weight_1,
        weight_2=weight_2,
        logits=logits,
        scores=scores,
        top_experts=top_experts,
    )
