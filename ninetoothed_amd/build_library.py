"""Builds ``libnt_hip.so`` (the gfx950 kernels behind the C ABI) and ``libnt_probe.so`` (measurement kernels
that only bench.py loads) in-tree with hipcc.

Usage: ``python -m ninetoothed_amd.build_library`` or ``build_library()``.  The library
is written to ``ninetoothed_amd/lib/libnt_hip.so``; object files go to
``ninetoothed_amd/csrc/build/``.  Cross-compiling needs no GPU.
"""

import concurrent.futures
import pathlib
import shutil
import subprocess
import sys

PACKAGE_DIR = pathlib.Path(__file__).resolve().parent
CSRC_DIR = PACKAGE_DIR / "csrc"
LIBRARY_PATH = PACKAGE_DIR / "lib" / "libnt_hip.so"

SOURCES = ("gemm_api.hip", "conv2d.hip", "softmax.hip", "attention.hip", "map.hip", "workspace.hip", "tune.hip")

# Measurement aids (MFMA issue-rate kernels that bench.py times next to the programs) are no part of the C ABI:
# they are built into a library of their own that only bench.py loads.
PROBE_LIBRARY_PATH = PACKAGE_DIR / "lib" / "libnt_probe.so"
PROBE_SOURCES = ("probe.hip",)

OFFLOAD_ARCH = "gfx950"

# packed FP32 instructions are switched off for all device code of this library
DEVICE_FLAGS = (
    f"--offload-arch={OFFLOAD_ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
)


def _hipcc():
    path = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not pathlib.Path(path).exists():
        raise RuntimeError("hipcc not found; libnt_hip.so cannot be built")
    return path


def _run(command):
    result = subprocess.run(command, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError(
            "command failed: " + " ".join(map(str, command)) + "\n" + result.stdout + result.stderr
        )
    return result


def build_library(verbose=False, extra_flags=()):
    """Compiles every source for gfx950 and links the shared library.

    Always recompiles (it doubles as the "does it build" check)."""
    hipcc = _hipcc()
    build_dir = CSRC_DIR / "build"
    build_dir.mkdir(parents=True, exist_ok=True)
    LIBRARY_PATH.parent.mkdir(parents=True, exist_ok=True)

    def compile_one(source):
        obj = build_dir / (pathlib.Path(source).stem + ".o")
        command = [hipcc, *DEVICE_FLAGS, *extra_flags, "-c", str(CSRC_DIR / source), "-o", str(obj)]
        if verbose:
            print(" ".join(command), flush=True)
        _run(command)
        return obj

    def link(objects, path):
        temporary = path.with_suffix(".so.tmp")
        command = [hipcc, f"--offload-arch={OFFLOAD_ARCH}", "-shared", "-fPIC", *map(str, objects), "-o", str(temporary)]
        if verbose:
            print(" ".join(command), flush=True)
        _run(command)
        temporary.replace(path)

    with concurrent.futures.ThreadPoolExecutor(max_workers=4) as pool:
        objects = list(pool.map(compile_one, SOURCES + PROBE_SOURCES))

    link(objects[: len(SOURCES)], LIBRARY_PATH)
    link(objects[len(SOURCES) :], PROBE_LIBRARY_PATH)
    return LIBRARY_PATH


if __name__ == "__main__":
    print(build_library(verbose="-v" in sys.argv))
