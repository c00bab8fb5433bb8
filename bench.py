"""
Benchmark of the dropless-MoE hot path on one MI355X.

A step is one forward + backward of the MoE MLP over one batch of synthetic tokens: sparse map, dispatch, layer 1,
gated SiLU, layer 2, combine, and the whole backward including both weight gradients. Inputs, weights and routing
(top-k experts, fp32 scores) are resident in HBM before the timed region. The headline workload is the Mixtral-like
configuration (8192 tokens, hidden 4096, ffn 14336, 8 experts, top-2, bf16 with fp32 accumulation).

Prints one JSON line: whole-step tokens/s, the roofline of the grouped-GEMM kernel (six launches per step, algorithmic
FLOPs 18*M*H*F over their summed device time from HIP events on the launch stream), per-kernel figures for the
bandwidth-bound kernels (mean, median and minimum over the timed steps), `box` (what this very device sustains in the
same run: a register-only MFMA loop on random operands and the shader clock it holds), `isolated` (every kernel of the
step launched on its own with the caches flushed in between: median and minimum of 20 launches), the same step with
fp32 gradient buffers and with full recomputation, the other four configurations (`configs`), and a CPU baseline (the
looped torch MoE on the host cores over the whole batch).

`python bench.py --ceilings` prints, instead, what the device sustains: back-to-back MFMAs on zero and on random
operands, the vendor BLAS on dense products of the same sizes, the library's grouped products on normal and on all-zero
operands, a plain streaming copy, and the rate at which the CUs fill LDS from L2.

The probes behind `box` and `--ceilings` are not part of the kernel library: they are `bench_probes.hip` beside this
file, built into `libbench_probes.so` by `build_probes()` (which `__graft_entry__.build()` calls).
"""

import argparse
import contextlib
import ctypes
import json
import os
import pathlib
import statistics
import sys
import time

import torch

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA peak, TFLOP/s
PEAK_FP32_TFLOPS = 157.3  # MI355X fp32 (matrix) peak, TFLOP/s
PEAK_HBM_GBS = 8000.0  # MI355X HBM3E peak, GB/s
ROOT = pathlib.Path(__file__).resolve().parent
PROFILES = ROOT / "profiles"
PROBE_SOURCE, PROBE_LIBRARY = ROOT / "bench_probes.hip", ROOT / "libbench_probes.so"
FLUSH_BYTES = 512 << 20  # read between isolated launches: twice the 256 MiB Infinity Cache
HEADLINE = "mixtral"
_ISOLATED_KEYS = ("ms_median", "ms_min", "tflops", "frac_of_mfma_peak", "gbs", "frac_of_hbm_peak")
OTHER_WORKLOADS = ("tiny", "fine_grained", "wide", "imbalanced")


def measured_traffic(workload_name: str) -> tuple[int | None, str | None]:
    """HBM traffic per GEMM launch cannot be measured from inside the process; it comes from the committed summary of
    two `rocprofv3 --pmc` runs of this script (FETCH_SIZE, WRITE_SIZE, calibrated on the add kernel below)."""
    try:
        summary = json.loads((PROFILES / f"bench_{workload_name}_hbm_traffic.json").read_text())
    except (OSError, ValueError):
        return None, None
    if summary.get("workload") != workload_name:
        return None, None
    return summary["traffic_bytes_per_launch"], summary["source"]


def build_probes(verbose: bool = True) -> pathlib.Path:
    """Compile `bench_probes.hip` for gfx950 into `libbench_probes.so` (no GPU needed)."""
    if str(ROOT) not in sys.path:
        sys.path.insert(0, str(ROOT))
    from fast_llm_amd.build import build_shared

    return build_shared([PROBE_SOURCE], PROBE_LIBRARY, verbose)


_probes: ctypes.CDLL | None = None


def probes() -> ctypes.CDLL:
    """The probe library, built first if it is not there."""
    global _probes
    if _probes is None:
        if not PROBE_LIBRARY.is_file():
            build_probes()
        library = ctypes.CDLL(str(PROBE_LIBRARY))
        i64, ptr = ctypes.c_int64, ctypes.c_void_p
        library.probe_mfma.argtypes = [ptr, ptr, i64, i64, ctypes.c_int, ctypes.c_float, ptr]
        library.probe_mfma_flops.argtypes, library.probe_mfma_flops.restype = [i64, i64], i64
        library.probe_copy.argtypes = [ptr, ptr, i64, i64, ptr]
        library.probe_l2.argtypes = [ptr, i64, i64, i64, i64, i64, ptr, ptr]
        _probes = library
    return _probes


def probe_ok(status: int) -> None:
    if status != 0:
        raise RuntimeError(f"probe launch failed with status {status}")


def box_probe(device: torch.device, launches: int = 3) -> dict:
    """What this device sustains right now: a register-only loop of the grouped products' MFMA instruction on
    normal(0, 0.02) bf16 operands on every CU (about 40 ms per launch), and the shader clock it holds meanwhile. The
    chip is power-limited, boxes differ by a few per cent, and this is the ceiling of the one the figures come from."""
    library = probes()
    stream = torch.cuda.current_stream(device)
    compute_units = torch.cuda.get_device_properties(device).multi_processor_count
    iterations = 40000
    sink = torch.empty(compute_units * 256, dtype=torch.float32, device=device)
    cycles = torch.zeros(compute_units, dtype=torch.int64, device=device)

    def launch() -> None:
        probe_ok(library.probe_mfma(sink.data_ptr(), cycles.data_ptr(), compute_units, iterations, 1, 0.02, stream.cuda_stream))

    launch()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record(stream)
    for _ in range(launches):
        launch()
    end.record(stream)
    torch.cuda.synchronize()
    ms = start.elapsed_time(end) / launches
    tflops = library.probe_mfma_flops(compute_units, iterations) / ms / 1e9
    return {
        "mfma_loop_tflops_random": round(tflops, 1),
        "mfma_loop_frac_of_peak": round(tflops / PEAK_BF16_TFLOPS, 4),
        "shader_clock_mhz": round(cycles.double().mean().item() / ms / 1e3),
        "what": f"{launches} launches of {iterations} x 32 back-to-back v_mfma_f32_32x32x16_bf16 per wavefront, 4 "
        f"wavefronts on each of {compute_units} CUs, normal(0, 0.02) operands in registers, right after the timed steps",
    }


def parse_args() -> argparse.Namespace:
    parser = argparse.ArgumentParser(description=__doc__)
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=20)
    parser.add_argument("--warmup", type=int, default=3)
    parser.add_argument("--workload", default=HEADLINE, help="tiny | mixtral | fine_grained | wide | imbalanced")
    parser.add_argument("--recompute", default="none", help="none | activation | activation_and_input | full")
    parser.add_argument(
        "--cpu-tokens", type=int, default=1 << 30,
        help="tokens in the CPU baseline sample of the headline, at most the whole batch (the default; 0: skip)",
    )  # fmt: skip
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument(
        "--grad-dtype",
        default="same",
        choices=("same", "fp32"),
        help="dtype of the weight-gradient buffers of the headline: the weights' own (what the reference's kernel "
        "benchmarks and functional tests attach: torch.empty_like(param)) or float32 (the training engine's "
        "full_precision_gradients); the other one is reported under `other_grad_dtype`",
    )
    parser.add_argument(
        "--only", action="store_true", help="time the chosen workload only (no other configurations, no second "
        "gradient dtype): what the profiler runs use"
    )  # fmt: skip
    parser.add_argument(
        "--calibration-mib",
        type=int,
        default=1024,
        help="size of a plain device add done once before the warm-up; hardware counters (FETCH_SIZE, WRITE_SIZE) "
        "read for it calibrate the counters read for the kernels of the timed region (0: skip)",
    )
    parser.add_argument("--ceilings", action="store_true", help="measure the device's ceilings instead of the path")
    return parser.parse_args()


def cpu_baseline(workload, inputs, tokens: int, repetitions: int = 3) -> dict:
    """The looped torch MoE (per-expert gather -> linear -> silu*up -> linear -> scaled scatter-add, autograd
    backward) in fp32 on the host cores, over the first `tokens` tokens of the same batch with all experts' weights:
    one warm-up pass, then the median of `repetitions` timed passes."""
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

    run(min(tokens, 256))  # thread pool, allocator and page-fault warm-up
    seconds = [run(tokens) for _ in range(repetitions)]
    median = statistics.median(seconds)
    return {
        "value": tokens / median,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{workload.name}: first {tokens} of {workload.tokens} tokens, full {workload.experts}-expert weights, "
        f"fp32, looped torch MoE fwd+bwd, 1 warm-up + {repetitions} timed passes, median "
        f"({', '.join(f'{s:.2f}' for s in seconds)} s)",
    }


def time_workload(
    workload, args, steps: int, warmup: int, grad_dtype_name: str, recompute_level, device, events: bool = True
) -> dict:
    """Warm up, time `steps` steps of `workload` and return the step time and the per-kernel figures. Without `events`
    the timed steps carry no HIP events at all (for a step that is bound by the host's launches) and every kernel
    figure comes from the pass that follows them."""
    from fast_llm_amd import _lib
    from fast_llm_amd.functional.config import ActivationType
    from fast_llm_amd.functional.mlp import mlp_autograd
    from fast_llm_amd.functional.sparse_copy import get_sparse_map
    from fast_llm_amd.layers.moe import attach_grad_buffer
    from fast_llm_amd.workloads import make_inputs

    inputs = make_inputs(workload, seed=args.seed, weight_device=device).to(device)
    x = inputs.hidden_states.requires_grad_(True)
    scores = inputs.scores.requires_grad_(True)
    grad_dtype = torch.float32 if grad_dtype_name == "fp32" else None
    weight_1 = attach_grad_buffer(inputs.weight_1.requires_grad_(True), grad_dtype)
    weight_2 = attach_grad_buffer(inputs.weight_2.requires_grad_(True), grad_dtype)

    def step() -> None:
        x.grad = scores.grad = None
        weight_1.param_grad_is_zero = weight_2.param_grad_is_zero = True
        sparse_map = get_sparse_map(inputs.top_experts, workload.experts)
        output = mlp_autograd(
            x, scores, weight_1, None, weight_2, None, True, ActivationType.silu, None, False, True,
            recompute_level, True, sparse_map,
        )  # fmt: skip
        output.backward(inputs.grad_output)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # The timed region. HIP events bracket the grouped products only (the kernel the roofline figure is about): every
    # event record is a marker that the next kernel waits behind, and bracketing all ~22 calls of a step costs 0.06-0.1
    # ms per step (0.6 % of the Mixtral-like step, 1.6 % of the wide one, a third of the 512-token one).
    timer = _lib.KernelTimer(only="matmul") if events else None
    with timer or contextlib.nullcontext():
        start = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        seconds = time.perf_counter() - start
    ms_per_step = seconds / steps * 1e3
    all_durations = timer.durations_ms() if timer else {}
    calls_per_step = {label: len(values) / steps for label, values in all_durations.items()}
    # The other kernels of the step: a second, shorter pass with events around every call.
    other_steps = min(steps, 10)
    with _lib.KernelTimer() as timer:
        for _ in range(other_steps):
            step()
    for label, values in timer.durations_ms().items():
        if label not in all_durations:
            all_durations[label] = values
            calls_per_step[label] = len(values) / other_steps
    kernels = {
        label: kernel_figures(label, values, workload, recompute_level) | {"calls_per_step": calls_per_step[label]}
        for label, values in sorted(all_durations.items())
    }
    # Whole-step GEMM rate: algorithmic FLOPs of a step over the summed mean launch times.
    peak_tflops = PEAK_FP32_TFLOPS if workload.dtype == torch.float32 else PEAK_BF16_TFLOPS
    gemm_ms = sum(kernels[label]["ms"] * calls_per_step[label] for label in kernels if "matmul" in label)
    gemm_launches = sum(calls_per_step[label] for label in kernels if "matmul" in label)
    gemm_flops = workload.gemm_flops * (4 / 3 if recompute_level.recompute_layer_1 else 1)
    gemm_tflops = gemm_flops / (gemm_ms * 1e-3) / 1e12
    return {
        "inputs": inputs,
        "step": step,
        "state": (x, scores, weight_1, weight_2),
        "ms_per_step": ms_per_step,
        "tokens_per_s": workload.tokens * steps / seconds,
        "gemm_ms": gemm_ms,
        "gemm_launches": gemm_launches,
        "gemm_flops": gemm_flops,
        "gemm_tflops": gemm_tflops,
        "gemm_peak_tflops": peak_tflops,
        "kernels": kernels,
    }


def kernel_figures(label: str, durations_ms: list[float], workload, recompute_level) -> dict:
    """Mean, median and minimum device time of the launches of one kernel-library call, and the rate its algorithmic
    work (unpadded rows) gives at the mean, as a fraction of the matrix peak or of the HBM peak."""
    ms = sum(durations_ms) / len(durations_ms)
    entry = {
        "ms": round(ms, 4),
        "ms_median": round(statistics.median(durations_ms), 4),
        "ms_min": round(min(durations_ms), 4),
    }
    rows, hidden, ffn = workload.sparse_rows_unpadded, workload.hidden, workload.ffn
    itemsize = workload.dtype.itemsize
    peak_tflops = PEAK_FP32_TFLOPS if workload.dtype == torch.float32 else PEAK_BF16_TFLOPS
    index_size = 2 if rows + workload.experts * 128 < 32768 else 4
    work_bytes = None
    if "matmul" in label:
        m, n, k = (int(v) for v in label[label.index("[") + 1 : -1].split("x"))
        # Dimensions are padded/static; algorithmic FLOPs use the unpadded row count.
        per_launch = 2 * rows * (n if "row_sparse" not in label else m) * (k if "row_sparse" not in label else n)
        entry["tflops"] = round(per_launch / (ms * 1e-3) / 1e12, 1)
        entry["frac_of_mfma_peak"] = round(entry["tflops"] / peak_tflops, 4)
        entry["tflops_best"] = round(per_launch / (entry["ms_min"] * 1e-3) / 1e12, 1)
    elif label in ("fm_copy_dense_to_sparse", "fm_copy_sparse_to_dense"):
        work_bytes = workload.copy_bytes + rows * (index_size + 4)  # rows + indices + fp32 scores
    elif label == "fm_copy_sparse_to_dense_backward":
        work_bytes = (1 + 2 * workload.experts_per_token) * workload.tokens * hidden * itemsize
    elif label.startswith("fm_mlp_activation"):
        factor = 3 if label.endswith("forward") else (6 if recompute_level.recompute_activation else 5)
        work_bytes = factor * rows * ffn * itemsize
    if work_bytes is not None:
        entry["gbs"] = round(work_bytes / (ms * 1e-3) / 1e9, 1)
        entry["frac_of_hbm_peak"] = round(entry["gbs"] / PEAK_HBM_GBS, 4)
        entry["gbs_best"] = round(work_bytes / (entry["ms_min"] * 1e-3) / 1e9, 1)
    return entry


def isolated_kernels(workload, inputs, device, recompute_level, repetitions: int = 20) -> dict:
    """Every kernel of the step launched on its own, on the step's own operands, with the caches flushed before each
    launch: a 512 MiB buffer (twice the Infinity Cache) is read, so operands and whatever an earlier kernel left
    behind come from HBM. Median and minimum of `repetitions` launches, HIP events around the library call. The
    method of the reference's kernel benchmarks (tools/benchmark/triton_kernels/runner.py:211-276), except that the
    buffer is read where the reference zeroes it: a written buffer leaves the Infinity Cache full of dirty lines
    whose write-back is then charged to the kernel measured (the dispatch at the Mixtral shape, a 36 us kernel,
    measures 0.46 of the HBM peak after a write, 0.70 after a read and 0.69 inside the step)."""
    from fast_llm_amd import _lib
    from fast_llm_amd.functional import sparse_copy, sparse_linear
    from fast_llm_amd.functional.config import ActivationType
    from fast_llm_amd.functional.mlp import mlp_activation_backward, mlp_activation_forward

    silu = ActivationType.silu
    x, scores, grad_output = inputs.hidden_states, inputs.scores, inputs.grad_output
    weight_1, weight_2 = inputs.weight_1.detach(), inputs.weight_2.detach()
    sparse_map = sparse_copy.get_sparse_map(inputs.top_experts, workload.experts)
    # The operands of every kernel, computed once in the order of a step.
    x_sparse = sparse_copy.copy_dense_to_sparse(x, None, sparse_map)
    layer_1 = sparse_linear.output_sparse_matmul(x_sparse, weight_1.t(), sparse_map)
    activation = mlp_activation_forward(layer_1, True, silu, sparse_map)[0]
    layer_2 = sparse_linear.input_inner_sparse_matmul(activation, weight_2, sparse_map)
    grad_layer_2 = sparse_copy.copy_sparse_to_dense_backward(grad_output, (sparse_map, layer_2, scores))[0]
    grad_activation = sparse_linear.output_sparse_matmul(grad_layer_2, weight_2.t(), sparse_map)
    grad_layer_1 = mlp_activation_backward(grad_activation, (layer_1, True, silu, sparse_map))[0]
    grad_x_sparse = sparse_linear.input_inner_sparse_matmul(grad_layer_1, weight_1, sparse_map)
    grad_weight_1, grad_weight_2 = torch.empty_like(weight_1), torch.empty_like(weight_2)
    launches = [
        lambda: sparse_copy.get_sparse_map(inputs.top_experts, workload.experts),
        lambda: sparse_copy.copy_dense_to_sparse(x, None, sparse_map),
        lambda: sparse_linear.output_sparse_matmul(x_sparse, weight_1.t(), sparse_map),
        lambda: mlp_activation_forward(layer_1, True, silu, sparse_map),
        lambda: sparse_linear.input_inner_sparse_matmul(activation, weight_2, sparse_map),
        lambda: sparse_copy.copy_sparse_to_dense(layer_2, scores, sparse_map),
        lambda: sparse_copy.copy_sparse_to_dense_backward(grad_output, (sparse_map, layer_2, scores)),
        lambda: sparse_linear.output_sparse_matmul(grad_layer_2, weight_2.t(), sparse_map),
        lambda: mlp_activation_backward(grad_activation, (layer_1, True, silu, sparse_map)),
        lambda: sparse_linear.input_row_sparse_matmul(activation.t(), grad_layer_2, sparse_map, out=grad_weight_2),
        lambda: sparse_linear.input_inner_sparse_matmul(grad_layer_1, weight_1, sparse_map),
        lambda: sparse_linear.input_row_sparse_matmul(grad_layer_1.t(), x_sparse, sparse_map, out=grad_weight_1),
    ]
    flush = torch.ones(FLUSH_BYTES // 4, dtype=torch.int32, device=device)
    durations: dict[str, list[float]] = {}
    for launch in launches:
        with _lib.KernelTimer() as timer:
            for repetition in range(repetitions + 1):
                flush.sum()
                launch()
        for label, values in timer.durations_ms().items():
            durations.setdefault(label, []).extend(values[1:])  # the first launch warms up
    figures = {}
    for label, values in sorted(durations.items()):
        entry = kernel_figures(label, values, workload, recompute_level)
        # Here the median is the figure: rate and fraction at the median instead of the mean.
        for rate, peak_key in (("tflops", "frac_of_mfma_peak"), ("gbs", "frac_of_hbm_peak")):
            if rate in entry:
                entry[rate] = round(entry[rate] * entry["ms"] / entry["ms_median"], 1)
                peak = PEAK_HBM_GBS if rate == "gbs" else (PEAK_FP32_TFLOPS if workload.dtype == torch.float32 else PEAK_BF16_TFLOPS)
                entry[peak_key] = round(entry[rate] / peak, 4)
        del entry["ms"]
        figures[label] = entry
    return {
        "method": f"each kernel on its own, a {FLUSH_BYTES >> 20} MiB buffer read before every launch (caches hold "
        f"none of the operands, and no dirty lines), median and minimum of {repetitions} launches after one warm-up; "
        "rates and fractions at the median",
        "kernels": figures,
    }


def graph_replay(timed: dict, device: torch.device, replays: int = 200) -> dict:
    """The step captured once in a HIP graph and replayed: what is left of a launch-bound step when the host is out of
    the way. The replayed step writes the same gradient as the eager one (checked)."""
    step = timed["step"]
    x = timed["state"][0]
    step()
    torch.cuda.synchronize()
    eager_grad = x.grad.clone()
    stream = torch.cuda.Stream(device=device)
    stream.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(stream):
        step()
    torch.cuda.current_stream(device).wait_stream(stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        step()
    graph.replay()
    torch.cuda.synchronize()
    matches = bool(torch.equal(x.grad, eager_grad))
    start = time.perf_counter()
    for _ in range(replays):
        graph.replay()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - start) / replays * 1e3
    return {"ms_per_step": round(ms, 4), "replays": replays, "matches_eager": matches}


def summary_of(workload, timed: dict) -> dict:
    """The per-configuration record: absolute throughput, TFLOP/s and GB/s, and each as a fraction of its roofline."""
    kernels = timed["kernels"]

    def hbm(label: str) -> dict | None:
        entry = kernels.get(label)
        return None if entry is None else {"gbs": entry["gbs"], "frac": entry["frac_of_hbm_peak"]}

    return {
        "workload": f"{workload.tokens} tokens, hidden {workload.hidden}, ffn {workload.ffn}, {workload.experts} "
        f"experts, top-{workload.experts_per_token}, {str(workload.dtype).removeprefix('torch.')}",
        "ms_per_step": round(timed["ms_per_step"], 4),
        "tokens_per_s": round(timed["tokens_per_s"], 1),
        "gemm_tflops": round(timed["gemm_tflops"], 1),
        "gemm_peak_tflops": timed["gemm_peak_tflops"],
        "gemm_frac": round(timed["gemm_tflops"] / timed["gemm_peak_tflops"], 4),
        "gemm_frac_of_step": round(timed["gemm_ms"] / timed["ms_per_step"], 4),
        "dispatch": hbm("fm_copy_dense_to_sparse"),
        "combine": hbm("fm_copy_sparse_to_dense"),
        "combine_backward": hbm("fm_copy_sparse_to_dense_backward"),
        "activation_forward": hbm("fm_mlp_activation_forward"),
        "activation_backward": hbm("fm_mlp_activation_backward"),
        "sparse_map_ms": kernels.get("fm_sparse_map", {}).get("ms"),
    }


def release(timed: dict) -> None:
    for key in ("inputs", "step", "state"):
        timed.pop(key, None)
    torch.cuda.empty_cache()


def measure_ceilings(device: torch.device) -> dict:
    """What the device sustains, for setting the kernels' figures against: see the module docstring."""
    library = probes()
    stream = torch.cuda.current_stream(device)
    compute_units = torch.cuda.get_device_properties(device).multi_processor_count

    def timed(function, repetitions: int) -> float:
        function()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for _ in range(repetitions):
            function()
        end.record(stream)
        torch.cuda.synchronize()
        return start.elapsed_time(end) / repetitions  # ms

    result: dict = {"compute_units": compute_units}
    sink = torch.empty(compute_units * 256, dtype=torch.float32, device=device)
    iterations = 40000  # about 30 ms per launch at the published peak
    flops = library.probe_mfma_flops(compute_units, iterations)
    for name, random_operands, sigma in (("zeros", 0, 0.0), ("normal_sigma_0.02", 1, 0.02), ("normal_sigma_1", 1, 1.0)):
        ms = timed(
            lambda: probe_ok(
                library.probe_mfma(sink.data_ptr(), None, compute_units, iterations, random_operands, sigma, stream.cuda_stream)
            ),
            10,
        )
        result[f"mfma_loop_tflops_{name}"] = round(flops / ms / 1e9, 1)

    # The vendor BLAS (torch.matmul) on dense products of the grouped products' sizes and operand layouts.
    generator = torch.Generator(device=device).manual_seed(0)

    def normal(*shape):
        return torch.empty(*shape, dtype=torch.bfloat16, device=device).normal_(0, 0.02, generator=generator)

    rows, hidden, wide = 16384, 4096, 28672
    x, weight, y = normal(rows, hidden), normal(wide, hidden), normal(rows, wide)
    gemm_flops = 2 * rows * hidden * wide
    for name, function in (
        ("blas_dense_tflops_x_wT", lambda: torch.matmul(x, weight.t())),
        ("blas_dense_tflops_y_w", lambda: torch.matmul(y, weight)),
        ("blas_dense_tflops_yT_x", lambda: torch.matmul(y.t(), x)),
    ):
        result[name] = round(gemm_flops / timed(function, 10) / 1e9, 1)
    x_zero, weight_zero = torch.zeros_like(x), torch.zeros_like(weight)
    result["blas_dense_tflops_x_wT_zeros"] = round(gemm_flops / timed(lambda: torch.matmul(x_zero, weight_zero.t()), 10) / 1e9, 1)
    del x, weight, y, x_zero, weight_zero

    # The library's three grouped products at the Mixtral shape, launched back to back on their own, on normal and on
    # all-zero operands: on zeros the clock stays up, so the rate shows how far the kernels' structure alone would go.
    from fast_llm_amd.functional.sparse_copy import get_sparse_map
    from fast_llm_amd.functional.sparse_linear import (
        input_inner_sparse_matmul,
        input_row_sparse_matmul,
        output_sparse_matmul,
    )
    from fast_llm_amd.workloads import WORKLOADS, make_inputs

    workload = WORKLOADS[HEADLINE]
    sparse_map = get_sparse_map(make_inputs(workload, weights=False).top_experts.to(device), workload.experts)
    padded_rows, wide = sparse_map.num_rows, 2 * workload.ffn
    grouped_flops = 2 * workload.sparse_rows_unpadded * workload.hidden * wide
    for name, fill in (("normal_sigma_0.02", lambda t: t.normal_(0, 0.02, generator=generator)), ("zeros", lambda t: t.zero_())):
        x = fill(torch.empty(padded_rows, workload.hidden, dtype=torch.bfloat16, device=device))
        y = fill(torch.empty(padded_rows, wide, dtype=torch.bfloat16, device=device))
        weight = fill(torch.empty(workload.experts * wide, workload.hidden, dtype=torch.bfloat16, device=device))
        gradient = torch.empty_like(weight)
        for product, function in (
            ("output_sparse_x_wT", lambda: output_sparse_matmul(x, weight.t(), sparse_map)),
            ("input_inner_sparse_y_w", lambda: input_inner_sparse_matmul(y, weight, sparse_map)),
            ("input_row_sparse_yT_x", lambda: input_row_sparse_matmul(y.t(), x, sparse_map, out=gradient)),
        ):
            result[f"grouped_tflops_{product}_{name}"] = round(grouped_flops / timed(function, 10) / 1e9, 1)
        del x, y, weight, gradient

    # Plain copies: 1 GiB read + 1 GiB written.
    size = 1 << 30
    source = torch.empty(size, dtype=torch.uint8, device=device).random_(0, 255)
    target = torch.empty_like(source)
    for workgroups in (compute_units * 8, compute_units * 32, size // 16 // 256):
        ms = timed(
            lambda: probe_ok(
                library.probe_copy(source.data_ptr(), target.data_ptr(), size, workgroups, stream.cuda_stream)
            ),
            20,
        )
        result[f"copy_kernel_gbs_{workgroups}_workgroups"] = round(2 * size / ms / 1e6, 1)
    assert torch.equal(source, target)
    result["torch_copy_gbs"] = round(2 * size / timed(lambda: target.copy_(source), 20) / 1e6, 1)
    result["torch_add_gbs"] = round(2 * size / timed(lambda: torch.add(source, 1, out=target), 20) / 1e6, 1)
    del source, target

    # L2 -> LDS: every CU streams 64 KiB per iteration (one 256 x 256 x 64 bf16 slice) from a region that stays in its
    # XCD's 4 MiB L2 (groups of 4 CUs share 256 KiB: 2 MiB per XCD; or all 32 CUs of an XCD share 1 MiB), and, for
    # comparison, from regions that do not fit in L2 (4 MiB per CU).
    iterations = 4000
    cycles = torch.zeros(compute_units, dtype=torch.int64, device=device)
    for name, region_bytes, shared_by, in_flight in (
        ("l2_16_loads_in_flight", 256 << 10, 4, 1),
        ("l2_32_loads_in_flight", 256 << 10, 4, 2),
        ("l2_48_loads_in_flight", 256 << 10, 4, 3),
        ("l2_shared_by_32_48_loads_in_flight", 1 << 20, 32, 3),
        ("l2_48_loads_in_flight_64_cus", 256 << 10, 4, 3),
        ("beyond_l2_48_loads_in_flight", 4 << 20, 1, 3),
    ):
        workgroups = 64 if name.endswith("64_cus") else compute_units
        groups = 8 * -(-(workgroups // 8) // shared_by)
        region = torch.empty(groups * region_bytes, dtype=torch.uint8, device=device).random_(0, 255)
        ms = timed(
            lambda: probe_ok(
                library.probe_l2(
                    region.data_ptr(), region_bytes, shared_by, workgroups, iterations, in_flight, cycles.data_ptr(),
                    stream.cuda_stream,
                )
            ),
            3,
        )
        mean_cycles = cycles[:workgroups].double().mean().item()
        result[f"lds_fill_from_{name}"] = {
            "tbs": round(workgroups * iterations * 65536 / ms / 1e9, 2),
            "bytes_per_cycle_per_cu": round(iterations * 65536 / mean_cycles, 1),
            "shader_clock_mhz": round(mean_cycles / ms / 1e3),
            "cycles_per_64_kib": round(mean_cycles / iterations),
        }
        del region
    result["peaks"] = {"bf16_mfma_tflops": PEAK_BF16_TFLOPS, "hbm_gbs": PEAK_HBM_GBS}
    return result


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
    from fast_llm_amd.functional.config import MLPRecomputeLevel
    from fast_llm_amd.workloads import WORKLOADS

    if not _lib.LIBRARY_PATH.is_file():
        from fast_llm_amd.build import build_library

        build_library()

    device = torch.device("cuda:0")
    if args.ceilings:
        print(json.dumps({"ceilings": measure_ceilings(device)}))
        return

    workload = WORKLOADS[args.workload]
    recompute_level = MLPRecomputeLevel(args.recompute)
    dtype_names = {torch.bfloat16: "bf16", torch.float32: "f32", torch.float16: "f16"}

    if args.calibration_mib > 0:
        # One read and one write of a known size, outside the timed region: an elementwise add kernel (a plain
        # `copy_` would go through the runtime's blit path, for which no counters are reported).
        source = torch.ones(args.calibration_mib << 18, dtype=torch.float32, device=device)
        torch.add(source, 1.0, out=torch.empty_like(source))
        del source

    timed = time_workload(workload, args, args.steps, args.warmup, args.grad_dtype, recompute_level, device)
    hidden, ffn = workload.hidden, workload.ffn
    grad_dtype_name = "f32" if args.grad_dtype == "fp32" else dtype_names[workload.dtype]
    traffic, traffic_source = measured_traffic(workload.name)
    result = {
        "metric": "MoE fwd+bwd tokens/s at Mixtral shape; grouped-GEMM % bf16 MFMA peak",
        "value": timed["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": timed["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype_names[workload.dtype],
        "data": "synthetic",
        "config": {
            "workload": f"{workload.name}: dropless MoE MLP fwd+bwd, {workload.tokens} tokens, hidden {hidden}, "
            f"ffn {ffn}, {workload.experts} experts, top-{workload.experts_per_token}, gated SiLU, "
            f"recompute={recompute_level.value}, weight-gradient buffers {grad_dtype_name}",
            "tokens": workload.tokens,
            "hidden": hidden,
            "ffn": ffn,
            "experts": workload.experts,
            "experts_per_token": workload.experts_per_token,
            "grad_dtype": grad_dtype_name,
        },
        "roofline": {
            "bound": "mfma",
            "kernel": "grouped_gemm_mfma_kernel (all grouped-GEMM launches of a step; figures are per launch, averaged over them)",
            "achieved": timed["gemm_tflops"],
            "peak": timed["gemm_peak_tflops"],
            "unit": "TFLOP/s",
            "frac": timed["gemm_tflops"] / timed["gemm_peak_tflops"],
            "traffic": traffic,
            "traffic_source": traffic_source,
            "launches_per_step": timed["gemm_launches"],
            "flops_per_launch": timed["gemm_flops"] / timed["gemm_launches"],
            "ms_per_launch": timed["gemm_ms"] / timed["gemm_launches"],
        },
        "gemm_frac_of_step": timed["gemm_ms"] / timed["ms_per_step"],
        "kernels": timed["kernels"],
    }
    headline_inputs = timed["inputs"]
    # Same run, same device, right after the timed steps: the MFMA rate and clock this box holds under load.
    result["box"] = box_probe(device)
    result["roofline"]["frac_of_box_mfma_loop"] = round(timed["gemm_tflops"] / result["box"]["mfma_loop_tflops_random"], 4)

    if not args.only:
        result["isolated"] = isolated_kernels(workload, timed["inputs"], device, recompute_level)
        # The same step with the other gradient-buffer layout.
        other = "same" if args.grad_dtype == "fp32" else "fp32"
        headline_inputs = None if args.cpu_tokens <= 0 else timed["inputs"].to("cpu")
        release(timed)
        other_timed = time_workload(workload, args, args.steps, args.warmup, other, recompute_level, device)
        release(other_timed)
        result["other_grad_dtype"] = {
            "grad_dtype": "f32" if other == "fp32" else dtype_names[workload.dtype],
            "ms_per_step": round(other_timed["ms_per_step"], 4),
            "tokens_per_s": round(other_timed["tokens_per_s"], 1),
            "gemm_tflops": round(other_timed["gemm_tflops"], 1),
            "gemm_frac": round(other_timed["gemm_tflops"] / other_timed["gemm_peak_tflops"], 4),
        }
        # The same step with full recomputation (layer 1 runs a second time in the backward; its forward takes the
        # kernel with the activation in its epilogue, since its output is not stored).
        if recompute_level != MLPRecomputeLevel.full:
            full_timed = time_workload(workload, args, min(args.steps, 10), min(args.warmup, 2), args.grad_dtype,
                                       MLPRecomputeLevel.full, device)  # fmt: skip
            release(full_timed)
            result["recompute_full"] = {
                "ms_per_step": round(full_timed["ms_per_step"], 4),
                "tokens_per_s": round(full_timed["tokens_per_s"], 1),
                "gemm_tflops": round(full_timed["gemm_tflops"], 1),
                "gemm_frac": round(full_timed["gemm_tflops"] / full_timed["gemm_peak_tflops"], 4),
                "kernels": {label: entry["ms"] for label, entry in full_timed["kernels"].items()},
            }
        # The other configurations: a few steps each, figures per configuration.
        configs = {workload.name: summary_of(workload, timed)}
        tiny_inputs = None
        for name in (HEADLINE,) + OTHER_WORKLOADS:
            if name == workload.name:
                continue
            other_workload = WORKLOADS[name]
            # A few steps each; the 512-token one is bound by the host's launches and needs more to be steady.
            config_steps, config_warmup = (200, 20) if name == "tiny" else (min(args.steps, 10), min(args.warmup, 2))
            config_timed = time_workload(other_workload, args, config_steps, config_warmup, "same",
                                         recompute_level, device, events=name != "tiny")  # fmt: skip
            configs[name] = summary_of(other_workload, config_timed)
            if name != "imbalanced":  # same shapes as the Mixtral-like configuration
                isolated = isolated_kernels(other_workload, config_timed["inputs"], device, recompute_level)
                configs[name]["isolated"] = {
                    label: {key: value for key, value in entry.items() if key in _ISOLATED_KEYS}
                    for label, entry in isolated["kernels"].items()
                }
            if name == "tiny":
                # Launch-bound (a dozen kernels of 5 to 150 us per step): the step replayed from a HIP graph.
                configs[name]["graph_replay"] = graph_replay(config_timed, device)
                if args.cpu_tokens > 0:
                    tiny_inputs = config_timed["inputs"].to("cpu")
            release(config_timed)
        result["configs"] = configs
        if tiny_inputs is not None:
            result["cpu_baseline_tiny"] = cpu_baseline(WORKLOADS["tiny"], tiny_inputs, WORKLOADS["tiny"].tokens)
    if args.cpu_tokens > 0:
        result["cpu_baseline"] = cpu_baseline(workload, headline_inputs, min(args.cpu_tokens, workload.tokens))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
