"""
A single-GPU dropless mixture-of-experts MLP block built on the HIP kernel path.

Covers what `MixtureOfExpertMLP` does between the router input and the block output for top-k routing
(reference: fast_llm/layers/decoder/mlp/mixture_of_experts.py:130-213, 237-278): router logits, z-loss, jitter, top-k
experts, fp32 softmax over the selected logits, load-balancing loss, shared experts, sparse map, dropless MLP.
Weight layout as in the reference: `layer_1.weight` [experts * 2 * ffn, hidden] with each expert's block ordered
[gate; up] (layers/decoder/mlp/mlp.py:81-87), `layer_2.weight` [experts * ffn, hidden] (stored transposed, :70-79).
"""

import torch

from fast_llm_amd.functional.config import ActivationType, MLPRecomputeLevel
from fast_llm_amd.functional.mlp import mlp_autograd
from fast_llm_amd.functional.sparse_copy import get_sparse_map


def attach_grad_buffer(weight: torch.Tensor, dtype: torch.dtype | None = None) -> torch.Tensor:
    """Give a weight the `grad_buffer` / `param_grad_is_zero` pair the hot path writes its gradient through
    (in the reference the training engine does this: fast_llm/engine/multi_stage/fsdp.py:258-260, 364-372)."""
    weight.grad_buffer = torch.empty_like(weight, dtype=dtype or weight.dtype)
    weight.param_grad_is_zero = True
    return weight


from fast_llm_amd.functional.routing import router, sinkhorn_routing, topk_routing  # noqa: E402, F401  (re-exported)
from fast_llm_amd.functional.utils import AuxiliaryLoss  # noqa: E402

LOAD_BALANCING_LOSS, ROUTER_Z_LOSS = "load_balancing_loss", "router_z_loss"  # layers/decoder/mlp/config.py:24-26
ROUTING_TOPK, ROUTING_SINKHORN = "aux_loss", "sinkhorn"  # `RoutingType`, layers/decoder/mlp/config.py:29-31


class DroplessMoEMLP(torch.nn.Module):
    def __init__(
        self,
        hidden_size: int,
        intermediate_size: int,
        experts: int,
        experts_per_token: int,
        *,
        gated: bool = True,
        activation: ActivationType = ActivationType.silu,
        recompute_level: MLPRecomputeLevel = MLPRecomputeLevel.none,
        dropless_dynamic_shape: bool = False,
        shared_experts: int = 0,
        auxiliary_loss_coefficient: float = 0.01,
        z_loss_coefficient: float = 0.0,
        jitter_eps: float = 0.0,
        routing: str = ROUTING_TOPK,
        router_normalization: torch.nn.Module | None = None,
        router_scale: bool = False,
        router_input_scale: float = 1.0,
        router_per_expert_scale: bool = False,
        full_precision_gradients: bool = False,
        init_std: float = 0.02,
        dtype: torch.dtype = torch.bfloat16,
        device: torch.device | str = "cuda",
    ):
        super().__init__()
        # `experts` counts the shared experts, which every token visits on top of its `experts_per_token` routed ones
        # (layers/decoder/mlp/config.py:127-133, 181-187).
        if not 0 <= shared_experts <= experts - experts_per_token:
            raise ValueError(f"shared_experts={shared_experts} with {experts} experts, {experts_per_token} per token")
        self.experts, self.experts_per_token, self.shared_experts = experts, experts_per_token, shared_experts
        self.unshared_experts = experts - shared_experts
        self.auxiliary_loss_coefficient, self.z_loss_coefficient = auxiliary_loss_coefficient, z_loss_coefficient
        self.jitter_eps = jitter_eps
        if routing not in (ROUTING_TOPK, ROUTING_SINKHORN):
            raise NotImplementedError(routing)
        if routing == ROUTING_SINKHORN and shared_experts:
            # The reference appends the shared experts on the top-k branch only (mixture_of_experts.py:163-168).
            raise ValueError("sinkhorn routing has no shared experts")
        self.routing = routing
        # The router's own view of the input (layers/decoder/mlp/config.py:101-122; mixture_of_experts.py:83-105,
        # 130-145): an optional normalisation layer, a learnable per-feature scale, a constant, and after the
        # routing a learnable per-expert scale on the scores. All upstream of the kernels: plain torch modules.
        self.router_normalization = router_normalization
        self.router_input_scale = router_input_scale
        self.router_scale = (
            torch.nn.Parameter(torch.ones(hidden_size, dtype=dtype, device=device)) if router_scale else None
        )
        self.router_per_expert_scale = (
            torch.nn.Parameter(torch.ones(experts, dtype=dtype, device=device)) if router_per_expert_scale else None
        )
        self.gated, self.activation = gated, activation
        self.recompute_level, self.dropless_dynamic_shape = recompute_level, dropless_dynamic_shape
        layer_1_rows = experts * intermediate_size * (2 if gated else 1)
        self.router = torch.nn.Parameter(torch.empty(self.unshared_experts, hidden_size, dtype=dtype, device=device))
        self.layer_1 = torch.nn.Parameter(torch.empty(layer_1_rows, hidden_size, dtype=dtype, device=device))
        self.layer_2 = torch.nn.Parameter(
            torch.empty(experts * intermediate_size, hidden_size, dtype=dtype, device=device)
        )
        with torch.no_grad():
            for parameter in (self.router, self.layer_1, self.layer_2):
                parameter.normal_(0, init_std)
        grad_dtype = torch.float32 if full_precision_gradients else None
        attach_grad_buffer(self.layer_1, grad_dtype)
        attach_grad_buffer(self.layer_2, grad_dtype)

    def route(
        self, hidden_states: torch.Tensor, grad_scale: float | None = None, losses: dict | None = None
    ) -> tuple[torch.Tensor, torch.Tensor]:
        """Router logits to (scores, top_experts), shared experts included. `grad_scale` (the reference's
        `kwargs["grad_output"]`) makes the two auxiliary losses train the router; `losses` collects their values
        (mixture_of_experts.py:146-171, 237-262)."""
        return self.route_with_counts(hidden_states, grad_scale, losses)[:2]

    def route_with_counts(
        self, hidden_states: torch.Tensor, grad_scale: float | None = None, losses: dict | None = None
    ) -> tuple:
        """`route`, followed by what the router's kernel counted on its way (the `RouterCounts` for `get_sparse_map`
        together with the returned `top_experts`; None for sinkhorn routing, which does not count)."""
        router_input = hidden_states if self.router_normalization is None else self.router_normalization(hidden_states)
        if self.router_scale is not None:
            router_input = router_input * self.router_scale
        if self.router_input_scale != 1.0:
            router_input = router_input * self.router_input_scale
        logits = torch.nn.functional.linear(router_input, self.router)
        noise = None
        if self.training and self.jitter_eps > 0.0:
            noise = torch.empty_like(logits).uniform_(1.0 - self.jitter_eps, 1.0 + self.jitter_eps)
        trained = self.training and grad_scale is not None
        if self.routing == ROUTING_SINKHORN:
            routed = self._route_sinkhorn(logits, noise, grad_scale if trained else None, losses)
            return (*self._scale_per_expert(*routed), None)
        scores, top_experts, load_balancing_loss, z_loss, router_counts = router(
            logits,
            self.experts_per_token,
            shared_experts=self.shared_experts,
            noise=noise,
            auxiliary_loss_grad=self.unshared_experts * self.auxiliary_loss_coefficient * grad_scale if trained else None,
            z_loss_grad=self.z_loss_coefficient * grad_scale if trained else None,
            return_counts=True,
        )
        if losses is not None:
            losses.setdefault(LOAD_BALANCING_LOSS, []).append(load_balancing_loss)
            if self.z_loss_coefficient > 0.0:
                losses.setdefault(ROUTER_Z_LOSS, []).append(z_loss)
        return (*self._scale_per_expert(scores, top_experts), router_counts)

    def _scale_per_expert(self, scores: torch.Tensor, top_experts: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        if self.router_per_expert_scale is not None:  # mixture_of_experts.py:174-175
            scores = scores * self.router_per_expert_scale[top_experts]
        return scores, top_experts

    def _route_sinkhorn(
        self, logits: torch.Tensor, noise: torch.Tensor | None, grad_scale: float | None, losses: dict | None
    ) -> tuple[torch.Tensor, torch.Tensor]:
        """z-loss, jitter and sinkhorn routing as the reference orders them (mixture_of_experts.py:146-171)."""
        if self.z_loss_coefficient > 0.0 and (grad_scale is not None or losses is not None):
            loss = torch.mean(torch.logsumexp(logits.float(), dim=-1) ** 2)
            if losses is not None:
                losses.setdefault(ROUTER_Z_LOSS, []).append(loss.detach())
            if grad_scale is not None:
                logits = AuxiliaryLoss.apply(logits, loss, self.z_loss_coefficient * grad_scale)
        if noise is not None:
            logits = logits * noise
        return sinkhorn_routing(logits, self.experts_per_token, self.training)

    def forward(
        self,
        input_: torch.Tensor,
        scores: torch.Tensor | None = None,
        top_experts: torch.Tensor | None = None,
        *,
        grad_scale: float | None = None,
        losses: dict | None = None,
    ) -> torch.Tensor:
        """`scores`/`top_experts` may be passed to bypass the router (tests pin the routing that way)."""
        hidden_states = input_.flatten(0, -2)
        router_counts = None
        if top_experts is None:
            # The router has counted the tokens of every expert on its way: the map need not count them again.
            scores, top_experts, router_counts = self.route_with_counts(hidden_states, grad_scale, losses)
        sparse_map = get_sparse_map(
            top_experts, self.experts, dynamic_shape=self.dropless_dynamic_shape, router_counts=router_counts
        )
        output = mlp_autograd(
            hidden_states,
            scores,
            self.layer_1,
            None,
            self.layer_2,
            None,
            gated=self.gated,
            activation_type=self.activation,
            group=None,
            sequence_parallel=False,
            training=self.training,
            recompute_level=self.recompute_level,
            transposed_layer_2_weight=True,
            sparse_map=sparse_map,
        )
        return output.view_as(input_)

    # ---- Hugging Face Mixtral layout ----------------------------------------------------------------------
    # The reference's Mixtral converter (fast_llm/models/gpt/conversion/mixtral.py:65-82) maps, per block,
    #   router.weight  <- block_sparse_moe.gate.weight                                   [experts, hidden]
    #   layer_1.weight <- cat over experts i of (experts.i.w1.weight, experts.i.w3.weight), dim 0
    #                     (`SplitWeightConverter`, engine/checkpoint/external.py:847-859): [gate_i; up_i] per expert
    #   layer_2.weight <- cat over i of experts.i.w2.weight along the last dim, transposed
    #                     (`TransposeSplitWeightConverter`, :862-879): [experts * ffn, hidden]
    @torch.no_grad()
    def import_mixtral_weights(self, state_dict: dict[str, torch.Tensor], prefix: str = "") -> None:
        """Load the weights of one `block_sparse_moe` module of a Hugging Face Mixtral checkpoint (keys
        `gate.weight`, `experts.{i}.w1|w2|w3.weight` after `prefix`)."""
        if not self.gated or self.shared_experts != 0:
            raise ValueError("the Mixtral layout has gated experts and no shared experts")

        def get(name: str) -> torch.Tensor:
            return state_dict[f"{prefix}{name}"]

        layer_1 = torch.cat(
            [get(f"experts.{i}.{name}.weight") for i in range(self.experts) for name in ("w1", "w3")], dim=0
        )
        layer_2 = torch.cat([get(f"experts.{i}.w2.weight") for i in range(self.experts)], dim=-1).t()
        for parameter, value in ((self.router, get("gate.weight")), (self.layer_1, layer_1), (self.layer_2, layer_2)):
            if parameter.shape != value.shape:
                raise ValueError(f"shape mismatch: {tuple(parameter.shape)} here, {tuple(value.shape)} in the checkpoint")
            parameter.copy_(value)

    @torch.no_grad()
    def export_mixtral_weights(self, prefix: str = "") -> dict[str, torch.Tensor]:
        """The inverse of `import_mixtral_weights`."""
        if not self.gated or self.shared_experts != 0:
            raise ValueError("the Mixtral layout has gated experts and no shared experts")
        out = {f"{prefix}gate.weight": self.router.detach().clone()}
        for i, (gate_up, down) in enumerate(zip(self.layer_1.chunk(self.experts), self.layer_2.chunk(self.experts))):
            gate, up = gate_up.chunk(2)
            out[f"{prefix}experts.{i}.w1.weight"] = gate.clone()
            out[f"{prefix}experts.{i}.w3.weight"] = up.clone()
            out[f"{prefix}experts.{i}.w2.weight"] = down.t().contiguous()
        return out
