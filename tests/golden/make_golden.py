"""
Writes `tests/golden/golden_small.npz`: inputs and expected outputs of small cases of the hot path.

Expected values do not come from the oracle's own formulas: the sparse map is computed by the brute-force O(M*E)
python loops of `tests/helpers.py`, the MoE outputs and gradients by a token-by-token textbook mixture in float64
differentiated by torch autograd. (The reference itself cannot be imported under this Python: it needs 3.12's
PEP 695 generics and `enum.StrEnum`, fast_llm/utils.py:35, fast_llm/functional/config.py:31.)

Run from the repository root: `python tests/golden/make_golden.py`.
"""

import pathlib
import sys

import numpy as np
import torch

ROOT = pathlib.Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT))

from tests.helpers import brute_force_sparse_map  # noqa: E402

TOKENS, HIDDEN, FFN, EXPERTS, TOP_K = 48, 64, 64, 4, 2


def textbook_moe(x, scores, top_experts, weight_1, weight_2):
    out = torch.zeros_like(x)
    for t in range(x.size(0)):
        for j in range(top_experts.size(1)):
            e = int(top_experts[t, j])
            w1 = weight_1[e * 2 * FFN : (e + 1) * 2 * FFN]
            gate, up = w1[:FFN] @ x[t], w1[FFN:] @ x[t]
            hidden = torch.nn.functional.silu(gate) * up
            out[t] = out[t] + scores[t, j] * (hidden @ weight_2[e * FFN : (e + 1) * FFN])
    return out


def main() -> None:
    generator = torch.Generator().manual_seed(1234)
    normal = lambda *shape: torch.randn(*shape, generator=generator)  # noqa: E731
    x, grad_output = normal(TOKENS, HIDDEN), normal(TOKENS, HIDDEN)
    weight_1, weight_2 = normal(EXPERTS * 2 * FFN, HIDDEN) / 8, normal(EXPERTS * FFN, HIDDEN) / 8
    logits = normal(TOKENS, EXPERTS)
    logits[:, 2] = float("-inf")  # expert 2 receives no token
    top_logits, top_experts = torch.topk(logits, TOP_K, dim=-1)
    scores = torch.softmax(top_logits, dim=-1, dtype=torch.float32)

    ends, pad_begins, rows = brute_force_sparse_map(top_experts.tolist(), EXPERTS, 128)

    leaves = [t.double().requires_grad_(True) for t in (x, scores, weight_1, weight_2)]
    output = textbook_moe(leaves[0], leaves[1], top_experts, leaves[2], leaves[3])
    output.backward(grad_output.double())

    np.savez_compressed(
        ROOT / "tests" / "golden" / "golden_small.npz",
        hidden_states=x.numpy(),
        grad_output=grad_output.numpy(),
        weight_1=weight_1.numpy(),
        weight_2=weight_2.numpy(),
        scores=scores.numpy(),
        top_experts=top_experts.numpy(),
        expert_ends=np.array(ends, dtype=np.int64),
        expert_pad_begins=np.array(pad_begins, dtype=np.int64),
        sparse_rows=np.array(rows, dtype=np.int64),
        output=output.detach().float().numpy(),
        grad_input=leaves[0].grad.float().numpy(),
        grad_scores=leaves[1].grad.float().numpy(),
        grad_weight_1=leaves[2].grad.float().numpy(),
        grad_weight_2=leaves[3].grad.float().numpy(),
    )


if __name__ == "__main__":
    main()
