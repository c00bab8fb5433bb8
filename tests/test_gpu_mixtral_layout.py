"""The block with weights in the Hugging Face Mixtral checkpoint layout against `transformers`' own Mixtral MoE block
run on the CPU in fp32: an implementation of the same layer that shares no code with this package or its oracle."""

import pytest
import torch

from fast_llm_amd.layers.moe import DroplessMoEMLP

pytestmark = pytest.mark.gpu


def _huggingface_block(hidden, ffn, experts, k):
    transformers = pytest.importorskip("transformers")
    from transformers.models.mixtral import modeling_mixtral

    config = transformers.MixtralConfig(
        hidden_size=hidden, intermediate_size=ffn, num_local_experts=experts, num_experts_per_tok=k,
        num_hidden_layers=1, num_attention_heads=4, num_key_value_heads=4, vocab_size=32,
    )  # fmt: skip
    block = modeling_mixtral.MixtralSparseMoeBlock(config).float()
    state = block.state_dict()
    if "experts.gate_up_proj" not in state:
        pytest.skip("this transformers version stores the experts in another layout")
    generator = torch.Generator().manual_seed(0)
    with torch.no_grad():
        for parameter in block.parameters():
            parameter.copy_(torch.randn(parameter.shape, generator=generator) * 0.1)
    # The checkpoint format (one w1/w3/w2 per expert), from the fused in-memory layout of this transformers version:
    # gate_up_proj [experts, 2 * ffn, hidden] holds w1 (gate) then w3 (up), down_proj [experts, hidden, ffn] is w2.
    state = block.state_dict()
    checkpoint = {"gate.weight": state["gate.weight"]}
    for i in range(experts):
        checkpoint[f"experts.{i}.w1.weight"] = state["experts.gate_up_proj"][i, :ffn]
        checkpoint[f"experts.{i}.w3.weight"] = state["experts.gate_up_proj"][i, ffn:]
        checkpoint[f"experts.{i}.w2.weight"] = state["experts.down_proj"][i]
    return block, checkpoint


@pytest.mark.parametrize(("hidden", "ffn", "experts", "k"), [(64, 128, 4, 2), (128, 192, 8, 2)])
def test_block_matches_the_transformers_mixtral_block(hidden, ffn, experts, k, device):
    block, checkpoint = _huggingface_block(hidden, ffn, experts, k)
    layer = DroplessMoEMLP(hidden, ffn, experts, k, dtype=torch.float32, device=device)
    layer.import_mixtral_weights({f"model.layers.0.block_sparse_moe.{key}": v for key, v in checkpoint.items()},
                                 prefix="model.layers.0.block_sparse_moe.")  # fmt: skip
    generator = torch.Generator().manual_seed(1)
    x = torch.randn(3, 50, hidden, generator=generator)
    grad_output = torch.randn(3, 50, hidden, generator=generator)

    x_cpu = x.clone().requires_grad_()
    expected = block(x_cpu)
    expected = expected[0] if isinstance(expected, tuple) else expected
    expected.backward(grad_output)

    x_gpu = x.to(device).requires_grad_()
    out = layer(x_gpu)
    out.backward(grad_output.to(device))

    def close(actual, reference):
        return (actual.cpu() - reference).abs().max() <= 1e-4 * reference.abs().max()

    assert close(out.detach(), expected.detach())
    assert close(x_gpu.grad, x_cpu.grad)
    assert close(layer.router.grad, block.gate.weight.grad)
    gate_up_grad = block.experts.gate_up_proj.grad  # [experts, 2 * ffn, hidden]
    assert close(layer.layer_1.grad_buffer, gate_up_grad.reshape(experts * 2 * ffn, hidden))
    down_grad = block.experts.down_proj.grad  # [experts, hidden, ffn]
    assert close(layer.layer_2.grad_buffer, down_grad.transpose(1, 2).reshape(experts * ffn, hidden))

    exported = layer.export_mixtral_weights()
    assert exported.keys() == checkpoint.keys()
    assert all(torch.equal(exported[key].cpu(), checkpoint[key]) for key in checkpoint)
