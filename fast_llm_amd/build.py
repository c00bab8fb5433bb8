"""
Build `libfastmoe_hip.so` (the gfx950 kernel library behind the C ABI in `include/fastmoe_hip.h`) in-tree with hipcc.

`python -m fast_llm_amd.build` compiles every `csrc/*.hip` for gfx950 and links them into
`fast_llm_amd/csrc/libfastmoe_hip.so`. hipcc cross-compiles, so no GPU is needed to build.
"""

import concurrent.futures
import pathlib
import shutil
import subprocess
import sys

CSRC = pathlib.Path(__file__).resolve().parent / "csrc"
LIBRARY = CSRC / "libfastmoe_hip.so"

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # Packed-fp32 instructions are kept out of the generated code.
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


def _hipcc() -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not pathlib.Path(hipcc).exists():
        raise RuntimeError("hipcc not found; the kernel library can only be built with the ROCm toolchain")
    return hipcc


def _compile(source: pathlib.Path) -> pathlib.Path:
    obj = source.with_suffix(".o")
    command = [_hipcc(), *HIPCC_FLAGS, "-c", str(source), "-o", str(obj)]
    result = subprocess.run(command, capture_output=True, text=True)
    # The host pass does not know the device-only target feature; that warning is noise.
    stderr = "\n".join(line for line in result.stderr.splitlines() if "packed-fp32-ops" not in line)
    if result.returncode != 0:
        raise RuntimeError(f"hipcc failed for {source.name}:\n{stderr}")
    if stderr.strip():
        print(stderr, file=sys.stderr)
    return obj


def build_shared(sources: list[pathlib.Path], library: pathlib.Path, verbose: bool = True) -> pathlib.Path:
    """Compile `sources` for gfx950 (in parallel) and link them into the shared library `library`."""
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        objects = list(pool.map(_compile, sources))
    command = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objects), "-o", str(library)]
    result = subprocess.run(command, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError(f"link failed:\n{result.stderr}")
    if verbose:
        print(f"built {library} from {len(sources)} sources")
    return library


def build_library(verbose: bool = True) -> pathlib.Path:
    sources = sorted(CSRC.glob("*.hip"))
    if not sources:
        raise RuntimeError(f"no HIP sources in {CSRC}")
    return build_shared(sources, LIBRARY, verbose)


if __name__ == "__main__":
    build_library()
