"""
ctypes binding of `libfastmoe_hip.so` (C ABI declared in `include/fastmoe_hip.h`).

The library is the only compute path of this package: if it is missing or a symbol is absent, importing this module
raises. Build it with `python -m fast_llm_amd.build`.
"""

import ctypes
import pathlib
import warnings

import torch

LIBRARY_PATH = pathlib.Path(__file__).resolve().parent / "csrc" / "libfastmoe_hip.so"

FM_VERSION = 10

_c_i64, _c_int, _c_ptr, _c_size = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t

# name -> (restype, argtypes). Mirrors include/fastmoe_hip.h one to one; tests check that every declared symbol
# is listed here and exported by the library.
SIGNATURES: dict[str, tuple] = {
    "fm_version": (_c_int, []),
    "fm_last_error": (ctypes.c_char_p, []),
    "fm_sparse_map_workspace_size": (_c_size, [_c_i64] * 3),
    "fm_sparse_map": (_c_int, [_c_ptr] + [_c_i64] * 4 + [_c_int] + [_c_ptr] * 4 + [_c_size, _c_ptr]),
    "fm_sparse_map_static_scratch_size": (_c_size, []),
    "fm_sparse_map_static": (_c_int, [_c_ptr] + [_c_i64] * 4 + [_c_int] + [_c_ptr] * 3 + [_c_ptr]),
    "fm_copy_dense_to_sparse": (_c_int, [_c_ptr] * 4 + [_c_i64] * 4 + [_c_int] * 3 + [_c_ptr]),
    "fm_copy_sparse_to_dense": (_c_int, [_c_ptr] * 4 + [_c_i64] * 4 + [_c_int] * 3 + [_c_ptr]),
    "fm_copy_sparse_to_dense_grad_score": (_c_int, [_c_ptr] * 4 + [_c_i64] * 4 + [_c_int] * 3 + [_c_ptr]),
    "fm_copy_sparse_to_dense_backward": (_c_int, [_c_ptr] * 6 + [_c_i64] * 4 + [_c_int] * 4 + [_c_ptr]),
    "fm_topk_routing": (_c_int, [_c_ptr] * 3 + [_c_i64] * 3 + [_c_int, _c_ptr]),
    "fm_topk_routing_backward": (_c_int, [_c_ptr] * 4 + [_c_i64] * 3 + [_c_int, _c_ptr]),
    "fm_router_workspace_size": (_c_size, [_c_i64] * 2),
    "fm_router_forward": (_c_int, [_c_ptr] * 8 + [_c_size] + [_c_i64] * 4 + [_c_int, _c_ptr]),
    "fm_sparse_map_from_router_workspace_size": (_c_size, [_c_i64] * 2),
    "fm_sparse_map_from_router": (
        _c_int,
        [_c_ptr, _c_ptr, _c_size] + [_c_i64] * 5 + [_c_int] + [_c_ptr] * 4 + [_c_size, _c_ptr],
    ),
    "fm_router_backward": (_c_int, [_c_ptr] * 8 + [ctypes.c_double] * 2 + [_c_i64] * 4 + [_c_int, _c_ptr]),
    "fm_mlp_activation_forward": (_c_int, [_c_ptr] * 2 + [_c_i64] * 2 + [_c_int] * 3 + [_c_ptr, _c_int, _c_ptr]),
    "fm_mlp_activation_backward": (_c_int, [_c_ptr] * 4 + [_c_i64] * 2 + [_c_int] * 3 + [_c_ptr, _c_int, _c_ptr]),
    "fm_grouped_gemm_workspace_size": (_c_size, [_c_i64] * 4 + [_c_int]),
    "fm_input_row_sparse_matmul_workspace_size": (_c_size, [_c_i64] * 4 + [_c_int]),
    "fm_output_sparse_matmul": (_c_int, [_c_ptr] * 4 + [_c_i64] * 10 + [_c_int] * 4 + [_c_ptr, _c_size, _c_ptr]),
    "fm_input_inner_sparse_matmul": (_c_int, [_c_ptr] * 4 + [_c_i64] * 10 + [_c_int] * 4 + [_c_ptr, _c_size, _c_ptr]),
    "fm_input_row_sparse_matmul": (_c_int, [_c_ptr] * 5 + [_c_i64] * 10 + [_c_int] * 4 + [_c_ptr, _c_size, _c_ptr]),
    "fm_output_sparse_matmul_gated_activation": (_c_int, [_c_ptr] * 5 + [_c_i64] * 8 + [_c_int] * 3 + [_c_ptr]),
    "fm_output_sparse_matmul_gated_activation_backward": (
        _c_int,
        [_c_ptr] * 6 + [_c_i64] * 8 + [_c_int] * 3 + [_c_ptr],
    ),
}

FM_ERR_INVALID_ARGUMENT, FM_ERR_UNSUPPORTED, FM_ERR_LAUNCH = -1, -2, -3
FM_NOTE_GENERIC_KERNEL = 1

DTYPES = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
INDEX_DTYPES = {torch.int16: 0, torch.int32: 1, torch.int64: 2}
ACTIVATIONS = {"gelu": 0, "silu": 1, "relu": 2, "squared_relu": 3, "identity": 4}


class FastMoeLibraryError(ImportError):
    pass


def load_library(path: pathlib.Path = LIBRARY_PATH) -> ctypes.CDLL:
    if not path.is_file():
        raise FastMoeLibraryError(
            f"{path} is missing: the HIP kernel library is the only compute path of fast_llm_amd. "
            "Build it with `python -m fast_llm_amd.build` (needs hipcc; no GPU required to compile)."
        )
    library = ctypes.CDLL(str(path))
    for name, (restype, argtypes) in SIGNATURES.items():
        try:
            function = getattr(library, name)
        except AttributeError as e:
            raise FastMoeLibraryError(f"{path} does not export `{name}`; rebuild it") from e
        function.restype = restype
        function.argtypes = argtypes
    version = library.fm_version()
    if version != FM_VERSION:
        raise FastMoeLibraryError(f"{path} has ABI version {version}, this package needs {FM_VERSION}; rebuild it")
    return library


_library: ctypes.CDLL | None = None


def lib() -> ctypes.CDLL:
    global _library
    if _library is None:
        _library = load_library()
    return _library


def check(status: int) -> None:
    """Turn a negative `fm_status` into the exception the reference's Python code would raise; a positive one (the
    call went through, with a remark) into a warning."""
    if status == 0:
        return
    if status == FM_NOTE_GENERIC_KERNEL:
        warnings.warn(
            "a grouped product with half-precision operands ran on the generic multiply-add kernel, not on the matrix "
            "cores (operands need a unit stride on one axis, 16-byte aligned rows, a reduction that is a multiple of 64)",
            RuntimeWarning,
            stacklevel=3,
        )
        return
    message = lib().fm_last_error().decode()
    if status == FM_ERR_LAUNCH:
        raise RuntimeError(message)
    if status == FM_ERR_UNSUPPORTED:
        raise NotImplementedError(message)
    raise ValueError(message)


class KernelTimer:
    """
    Device-time of every kernel-library call made while the timer is active, from HIP events recorded on the launch
    stream right before and after the call. Used by the benchmark; costs two event records per call (each one a
    marker in the stream that the next kernel waits behind: some 3 us of device time per timed call). `only` restricts
    the timer to the entry points whose name contains it.
    """

    def __init__(self, only: str | None = None):
        self.only = only
        self.records: list[tuple[str, torch.cuda.Event, torch.cuda.Event]] = []

    def __enter__(self) -> "KernelTimer":
        global _active_timer
        self._previous, _active_timer = _active_timer, self
        return self

    def __exit__(self, *exc) -> None:
        global _active_timer
        _active_timer = self._previous

    def durations_ms(self) -> dict[str, list[float]]:
        """label -> device milliseconds of each call, in call order. Synchronises."""
        torch.cuda.synchronize()
        out: dict[str, list[float]] = {}
        for label, start, end in self.records:
            out.setdefault(label, []).append(start.elapsed_time(end))
        return out


_active_timer: KernelTimer | None = None


def _current_raw_stream(device_index: int) -> int:
    """The `hipStream_t` of torch's current stream on that device, as an integer. `torch.cuda.current_stream()` builds
    a Python stream object and resolves the device on the way (some 9 us per call, most of the host time of a small
    launch); torch's own kernel launchers use this accessor instead."""
    try:
        return torch._C._cuda_getCurrentRawStream(device_index)
    except AttributeError:
        return torch.cuda.current_stream(device_index).cuda_stream


def call(name: str, device: torch.device, *args, label: str | None = None) -> None:
    """Launch entry point `name` on the current stream of `device` (appended as the last argument) and raise on a
    non-zero status."""
    current = torch.cuda.current_device()
    if device.index is not None and device.index != current:
        with torch.cuda.device(device):  # the kernels run on the device that is current
            return call(name, torch.device("cuda", torch.cuda.current_device()), *args, label=label)
    function = getattr(lib(), name)
    stream = _current_raw_stream(current)
    timer = _active_timer
    if timer is None or (timer.only is not None and timer.only not in name):
        status = function(*args, stream)
    else:
        # `record()` without an argument records on the current stream of the current device: the launch stream.
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        status = function(*args, stream)
        end.record()
        timer.records.append((label or name, start, end))
    if status != 0:
        check(status)


def require_device(*tensors: torch.Tensor | None) -> torch.device:
    """All tensors must live on one HIP device; there is no host implementation to fall back to."""
    device = None
    for tensor in tensors:
        if tensor is None:
            continue
        if tensor.device.type != "cuda":
            raise RuntimeError(
                f"fast_llm_amd kernels run on the GPU only, got a tensor on `{tensor.device}` (there is no CPU path)"
            )
        if device is None:
            device = tensor.device
        elif tensor.device != device:
            raise RuntimeError(f"tensors on different devices: {device} and {tensor.device}")
    assert device is not None
    return device


def ptr(tensor: torch.Tensor | None) -> int | None:
    return None if tensor is None else tensor.data_ptr()


def stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def dtype_tag(dtype: torch.dtype) -> int:
    try:
        return DTYPES[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {dtype} (supported: float32, bfloat16, float16)") from None


def index_tag(dtype: torch.dtype) -> int:
    try:
        return INDEX_DTYPES[dtype]
    except KeyError:
        raise ValueError(f"unsupported index dtype {dtype} (supported: int16, int32, int64)") from None
