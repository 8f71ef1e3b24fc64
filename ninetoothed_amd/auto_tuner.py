"""Tile selection for matmul / addmm launches with tunable block sizes.

The reference wraps a generated kernel whose arrangement has meta symbols in
``triton.autotune`` (src/ninetoothed/generation.py:372-516): the first call
with a new problem times every candidate and later calls reuse the winner; its
AOT path persists winners in a line-pair CSV file
(src/ninetoothed/build.py:683-703, templates/auto_tuning_cache.h:27-75) and
its ``AutoTuner`` keeps timings on disk between processes
(src/ninetoothed/auto_tuner.py:11-95).  Here the candidates are the GEMM
instances of ``libnt_hip.so``: ``nt_tune_gemm`` times them on the caller's
tensors, the library caches the winner per device and problem, and this module
keeps that cache on disk in the reference's CSV format so that a new process
starts tuned.

``NINETOOTHED_AMD_AUTOTUNE=0`` switches tuning off (launches then use the
library's fixed preference order).
"""

import ctypes
import hashlib
import os
import pathlib
import threading

from ninetoothed_amd import runtime

CACHE_DIR = pathlib.Path.home() / ".ninetoothed_amd" / "auto_tuning"

_lock = threading.Lock()
_loaded = False


def enabled():
    return os.environ.get("NINETOOTHED_AMD_AUTOTUNE", "1") != "0"


def cache_path():
    """One file per build of the library (a rebuilt library may number its instances differently)."""
    lib = runtime.library()
    names = "|".join(runtime.gemm_config_names()) + "|" + lib.nt_version().decode()
    return CACHE_DIR / ("gemm_" + hashlib.sha256(names.encode()).hexdigest()[:16] + ".csv")


def load_once():
    """Reads the on-disk cache into the library the first time a tuned launch is prepared."""
    global _loaded
    with _lock:
        if _loaded:
            return
        _loaded = True
        path = cache_path()
        if path.exists():
            entries = ctypes.c_int(0)
            runtime.library().nt_tune_cache_load(str(path).encode(), ctypes.byref(entries))


def lookup(dtype, out_dtype, m, n, k, addmm):
    return runtime.library().nt_tune_cache_lookup(dtype, out_dtype, m, n, k, int(addmm))


def tune(input, mat1, mat2, beta, alpha, output, dtype, out_dtype, iters=5):
    """Times the instances on these arguments (:class:`runtime.ArgumentTensor`), records the
    winner in the library and on disk.  Returns ``(instance, milliseconds)``."""
    lib = runtime.library()
    best, best_ms = ctypes.c_int(-1), ctypes.c_float(0.0)
    runtime.check(
        lib.nt_tune_gemm(runtime.current_stream(), input, mat1, mat2, beta, alpha, output, dtype, out_dtype, iters, ctypes.byref(best), ctypes.byref(best_ms))
    )
    try:
        CACHE_DIR.mkdir(parents=True, exist_ok=True)
        lib.nt_tune_cache_save(str(cache_path()).encode())
    except OSError:
        pass  # a read-only home directory only costs the persistence
    return best.value, best_ms.value
