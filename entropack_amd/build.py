"""Builds the native libraries of this package in-tree with hipcc (gfx950 only).

    python -m entropack_amd.build          # compile everything
"""
import os
import subprocess
import sys
import tempfile

PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PACKAGE_DIR, "csrc")
INCLUDE = os.path.join(os.path.dirname(PACKAGE_DIR), "include")
HIP_LIBRARY = os.path.join(PACKAGE_DIR, "libentropack_hip.so")
HIP_SOURCES = ("ep_plan.hip", "ep_decode.hip", "ep_decode_lds.hip", "ep_decode_rank.hip", "ep_decode_dot.hip", "ep_decode_sym.hip", "ep_decode_mfma.hip", "ep_tile_ans.hip", "ep_linear.hip", "ep_encode.hip")
HOST_LIBRARY = os.path.join(PACKAGE_DIR, "libentropack_host.so")
HOST_SOURCES = ("host_codec.c",)
HOST_FLAGS = ("-O2", "-std=c11", "-fPIC", "-shared", "-fopenmp", "-ffp-contract=off", "-Wall", "-Wextra")

HIPCC_FLAGS = (
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
    # Packed FP32 VALU forms are kept out of every kernel of this library.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
)


def hipcc() -> str:
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _run(command, verbose):
    if verbose:
        print(" ".join(command), flush=True)
    done = subprocess.run(command, capture_output=True, text=True)
    if done.returncode != 0:
        raise RuntimeError(f"{command[0]} failed ({done.returncode}):\n{done.stdout}\n{done.stderr}")
    if verbose and done.stderr.strip():
        print(done.stderr, file=sys.stderr)


def build_hip(verbose: bool = False, extra_flags=(), jobs: int = 4) -> str:
    """Compiles every translation unit (in parallel) and links libentropack_hip.so."""
    from concurrent.futures import ThreadPoolExecutor
    compile_flags = [flag for flag in HIPCC_FLAGS if flag != "-shared"]
    with tempfile.TemporaryDirectory(prefix="entropack_hip_") as scratch:
        objects = [os.path.join(scratch, name.replace(".hip", ".o")) for name in HIP_SOURCES]
        commands = [[hipcc(), *compile_flags, *extra_flags, "-I", INCLUDE, "-I", CSRC, "-c", os.path.join(CSRC, name), "-o", target]
                    for name, target in zip(HIP_SOURCES, objects)]
        with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
            list(pool.map(lambda command: _run(command, verbose), commands))
        _run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", HIP_LIBRARY, *objects], verbose)
    return HIP_LIBRARY


def build_host(verbose: bool = False) -> str:
    """The CPU encoder kernels (plain C)."""
    sources = [os.path.join(CSRC, name) for name in HOST_SOURCES]
    command = [os.environ.get("CC", "gcc"), *HOST_FLAGS, "-o", HOST_LIBRARY, *sources, "-lm"]
    if verbose:
        print(" ".join(command), flush=True)
    done = subprocess.run(command, capture_output=True, text=True)
    if done.returncode != 0:
        raise RuntimeError(f"gcc failed ({done.returncode}):\n{done.stdout}\n{done.stderr}")
    return HOST_LIBRARY


def build_all(verbose: bool = False) -> None:
    build_host(verbose)
    build_hip(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
