"""
Benchmark of the dropless-MoE hot path on one MI355X.

A step is one forward + backward of the MoE MLP over one batch of synthetic tokens: sparse map, dispatch, layer 1,
gated SiLU, layer 2, combine, and the whole backward including both weight gradients. Inputs, weights and routing
(top-k experts, fp32 scores) are resident in HBM before the timed region. The default workload is the Mixtral-like
configuration (8192 tokens, hidden 4096, ffn 14336, 8 experts, top-2, bf16 with fp32 accumulation).

Prints one JSON line: whole-step tokens/s, the roofline of the grouped-GEMM kernel (six launches per step, algorithmic
FLOPs 18*M*H*F over their summed device time from HIP events on the launch stream), per-kernel figures for the
bandwidth-bound kernels, and a CPU baseline (the looped torch MoE on the host cores, on a bounded token sample).
"""

import argparse
import json
import os
import pathlib
import sys
import time

import torch

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA peak, TFLOP/s
PEAK_HBM_GBS = 8000.0  # MI355X HBM3E peak, GB/s
# HBM traffic per GEMM launch cannot be measured from inside the process; it comes from the committed summary of two
# `rocprofv3 --pmc` runs of this script (FETCH_SIZE, WRITE_SIZE, calibrated on the copy kernel below).
TRAFFIC_SUMMARY = pathlib.Path(__file__).resolve().parent / "profiles" / "bench_mixtral_hbm_traffic.json"


def measured_traffic(workload_name: str) -> tuple[int | None, str | None]:
    try:
        summary = json.loads(TRAFFIC_SUMMARY.read_text())
    except (OSError, ValueError):
        return None, None
    if summary.get("workload") != workload_name:
        return None, None
    return summary["traffic_bytes_per_launch"], summary["source"]


def parse_args() -> argparse.Namespace:
    parser = argparse.ArgumentParser(description=__doc__)
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=10)
    parser.add_argument("--warmup", type=int, default=3)
    parser.add_argument("--workload", default="mixtral", help="tiny | mixtral | fine_grained | wide | imbalanced")
    parser.add_argument("--recompute", default="none", help="none | activation | activation_and_input | full")
    parser.add_argument("--cpu-tokens", type=int, default=8192, help="tokens in the CPU baseline sample (0: skip)")
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument(
        "--grad-dtype",
        default="same",
        choices=("same", "fp32"),
        help="dtype of the weight-gradient buffers: the weights' own (what the reference's kernel benchmarks and "
        "functional tests attach: torch.empty_like(param)) or float32 (the training engine's full_precision_gradients)",
    )
    parser.add_argument(
        "--calibration-mib",
        type=int,
        default=1024,
        help="size of a plain device copy done once before the warm-up; hardware counters (FETCH_SIZE, WRITE_SIZE) "
        "read for it calibrate the counters read for the kernels of the timed region (0: skip)",
    )
    return parser.parse_args()


def cpu_baseline(workload, inputs, tokens: int) -> dict:
    """The looped torch MoE (per-expert gather -> linear -> silu*up -> linear -> scaled scatter-add, autograd
    backward) in fp32 on the host cores, over the first `tokens` tokens of the same batch with all experts' weights."""
    from oracle import moe_oracle

    torch.set_num_threads(max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "1024")))))
    weight_1, weight_2 = inputs.weight_1.float().cpu(), inputs.weight_2.float().cpu()
    x, grad = inputs.hidden_states[:tokens].float().cpu(), inputs.grad_output[:tokens].float().cpu()
    scores, top_experts = inputs.scores[:tokens].cpu(), inputs.top_experts[:tokens].cpu()

    def run(count: int) -> float:
        start = time.perf_counter()
        moe_oracle.looped_moe_forward_backward(
            x[:count], scores[:count], top_experts[:count], weight_1, weight_2, workload.experts, grad[:count]
        )
        return time.perf_counter() - start

    run(min(tokens, 32))  # thread pool and allocator warm-up
    seconds = run(tokens)
    return {
        "value": tokens / seconds,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"first {tokens} of {workload.tokens} tokens, full {workload.experts}-expert weights, fp32, "
        f"looped torch MoE fwd+bwd, 1 warm-up + 1 timed pass ({seconds:.2f} s)",
    }


def main() -> None:
    args = parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print(
            "bench.py measures one GPU: the dropless-MoE path keeps the whole expert set on a single MI355X and has no "
            "collectives. Run it with --gpus 1.",
            file=sys.stderr,
        )
        sys.exit(2)

    from fast_llm_amd import _lib
    from fast_llm_amd.functional.config import ActivationType, MLPRecomputeLevel
    from fast_llm_amd.functional.mlp import mlp_autograd
    from fast_llm_amd.functional.sparse_copy import get_sparse_map
    from fast_llm_amd.layers.moe import attach_grad_buffer
    from fast_llm_amd.workloads import WORKLOADS, make_inputs

    if not _lib.LIBRARY_PATH.is_file():
        from fast_llm_amd.build import build_library

        build_library()

    workload = WORKLOADS[args.workload]
    recompute_level = MLPRecomputeLevel(args.recompute)
    device = torch.device("cuda:0")
    inputs = make_inputs(workload, seed=args.seed, weight_device=device).to(device)
    x = inputs.hidden_states.requires_grad_(True)
    scores = inputs.scores.requires_grad_(True)
    grad_dtype = torch.float32 if args.grad_dtype == "fp32" else None
    weight_1 = attach_grad_buffer(inputs.weight_1.requires_grad_(True), grad_dtype)
    weight_2 = attach_grad_buffer(inputs.weight_2.requires_grad_(True), grad_dtype)

    def step() -> None:
        x.grad = scores.grad = None
        weight_1.param_grad_is_zero = weight_2.param_grad_is_zero = True
        sparse_map = get_sparse_map(inputs.top_experts, workload.experts)
        output = mlp_autograd(
            x, scores, weight_1, None, weight_2, None, True, ActivationType.silu, None, False, True,
            recompute_level, True, sparse_map,
        )
        output.backward(inputs.grad_output)

    if args.calibration_mib > 0:
        # One read and one write of a known size, outside the timed region: an elementwise add kernel (a plain
        # `copy_` would go through the runtime's blit path, for which no counters are reported).
        source = torch.ones(args.calibration_mib << 18, dtype=torch.float32, device=device)
        torch.add(source, 1.0, out=torch.empty_like(source))
        del source
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    with _lib.KernelTimer() as timer:
        start = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        seconds = time.perf_counter() - start
    ms_per_step = seconds / args.steps * 1e3
    tokens_per_second = workload.tokens * args.steps / seconds

    # Per-kernel device time, averaged over the timed steps.
    durations = {label: sum(values) / len(values) for label, values in timer.durations_ms().items()}
    calls_per_step = {label: len(values) / args.steps for label, values in timer.durations_ms().items()}
    rows, hidden, ffn = workload.sparse_rows_unpadded, workload.hidden, workload.ffn
    itemsize = workload.dtype.itemsize
    gemm_ms = sum(durations[label] * calls_per_step[label] for label in durations if "matmul" in label)
    gemm_launches = sum(calls_per_step[label] for label in durations if "matmul" in label)
    gemm_flops = workload.gemm_flops * (4 / 3 if recompute_level.recompute_layer_1 else 1)
    gemm_tflops = gemm_flops / (gemm_ms * 1e-3) / 1e12
    index_size = 2 if rows + workload.experts * 128 < 32768 else 4
    copy_bytes = workload.copy_bytes + rows * (index_size + 4)  # rows + indices + fp32 scores
    kernels = {}
    for label, ms in sorted(durations.items()):
        entry = {"ms": round(ms, 4), "calls_per_step": calls_per_step[label]}
        if "matmul" in label:
            m, n, k = (int(v) for v in label[label.index("[") + 1 : -1].split("x"))
            # Dimensions are padded/static; algorithmic FLOPs use the unpadded row count.
            per_launch = 2 * rows * (n if "row_sparse" not in label else m) * (k if "row_sparse" not in label else n)
            entry["tflops"] = round(per_launch / (ms * 1e-3) / 1e12, 1)
            entry["frac_of_mfma_peak"] = round(entry["tflops"] / PEAK_BF16_TFLOPS, 4)
        elif label in ("fm_copy_dense_to_sparse", "fm_copy_sparse_to_dense"):
            entry["gbs"] = round(copy_bytes / (ms * 1e-3) / 1e9, 1)
            entry["frac_of_hbm_peak"] = round(entry["gbs"] / PEAK_HBM_GBS, 4)
        elif label == "fm_copy_sparse_to_dense_backward":
            fused_bytes = (1 + 2 * workload.experts_per_token) * workload.tokens * hidden * itemsize
            entry["gbs"] = round(fused_bytes / (ms * 1e-3) / 1e9, 1)
            entry["frac_of_hbm_peak"] = round(entry["gbs"] / PEAK_HBM_GBS, 4)
        elif label.startswith("fm_mlp_activation"):
            factor = 3 if label.endswith("forward") else (6 if recompute_level.recompute_activation else 5)
            entry["gbs"] = round(factor * rows * ffn * itemsize / (ms * 1e-3) / 1e9, 1)
            entry["frac_of_hbm_peak"] = round(entry["gbs"] / PEAK_HBM_GBS, 4)
        kernels[label] = entry

    traffic, traffic_source = measured_traffic(workload.name)
    result = {
        "metric": "MoE fwd+bwd tokens/s at Mixtral shape; grouped-GEMM % bf16 MFMA peak",
        "value": tokens_per_second,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {torch.bfloat16: "bf16", torch.float32: "f32", torch.float16: "f16"}[workload.dtype],
        "data": "synthetic",
        "config": {
            "workload": f"{workload.name}: dropless MoE MLP fwd+bwd, {workload.tokens} tokens, hidden {hidden}, "
            f"ffn {ffn}, {workload.experts} experts, top-{workload.experts_per_token}, gated SiLU, "
            f"recompute={recompute_level.value}",
            "tokens": workload.tokens,
            "hidden": hidden,
            "ffn": ffn,
            "experts": workload.experts,
            "experts_per_token": workload.experts_per_token,
        },
        "roofline": {
            "bound": "mfma",
            "kernel": "grouped_gemm_mfma_kernel (all grouped-GEMM launches of a step; figures are per launch, averaged over them)",
            "achieved": gemm_tflops,
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": gemm_tflops / PEAK_BF16_TFLOPS,
            "traffic": traffic,
            "traffic_source": traffic_source,
            "launches_per_step": gemm_launches,
            "flops_per_launch": gemm_flops / gemm_launches,
            "ms_per_launch": gemm_ms / gemm_launches,
        },
        "gemm_frac_of_step": gemm_ms / ms_per_step,
        "kernels": kernels,
    }
    if args.cpu_tokens > 0:
        result["cpu_baseline"] = cpu_baseline(workload, inputs, min(args.cpu_tokens, workload.tokens))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
