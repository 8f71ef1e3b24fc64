"""Tile selection for matmul / addmm launches with tunable block sizes.

The reference wraps a generated kernel whose arrangement has meta symbols in
``triton.autotune`` (src/ninetoothed/generation.py:372-516): the first call
with a new problem times every candidate and later calls reuse the winner; its
AOT path persists winners in a line-pair CSV file
(src/ninetoothed/build.py:683-703, templates/auto_tuning_cache.h:27-75) and
its ``AutoTuner`` keeps timings on disk between processes
(src/ninetoothed/auto_tuner.py:11-95).  Here the candidates are the
kernel variants of ``libnt_hip.so`` -- GEMM instances, attention loop forms,
conv2d paths: ``nt_tune_gemm`` / ``nt_tune_attention`` / ``nt_tune_conv2d`` time
them on the caller's tensors, the library caches the winner per device and
problem, and this module keeps that cache on disk in the reference's CSV format
so that a new process starts tuned.

``NINETOOTHED_AMD_AUTOTUNE=0`` switches tuning off (launches then use the
library's fixed preference order).
"""

import ctypes
import hashlib
import os
import pathlib
import threading

from ninetoothed_amd import runtime

# where tuned choices are kept between processes; NINETOOTHED_AMD_CACHE_DIR moves it (and make's kernel
# descriptions) away from the home directory
CACHE_DIR = pathlib.Path(os.environ.get("NINETOOTHED_AMD_CACHE_DIR") or pathlib.Path.home() / ".ninetoothed_amd") / "auto_tuning"

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


def lookup_problem(kind, values):
    """The recorded choice for a problem of program ``kind`` (``runtime.TUNE_*``), or -1."""
    array = (ctypes.c_int * len(values))(*[int(v) for v in values])
    return runtime.library().nt_tune_lookup(kind, array, len(values))


def lookup(dtype, out_dtype, m, n, k, addmm, rhs_layout=0):
    """The tuned GEMM instance, or -1.  ``rhs_layout``: 0 row-major ``[K, N]``, 1 transposed (``[N, K]`` storage), 2 other strides."""
    return lookup_problem(runtime.TUNE_GEMM, (dtype, out_dtype, m, n, k, int(addmm), rhs_layout))


def _save():
    try:
        CACHE_DIR.mkdir(parents=True, exist_ok=True)
        runtime.library().nt_tune_cache_save(str(cache_path()).encode())
    except OSError:
        pass  # a read-only home directory only costs the persistence


def tune_attention(q, k, v, is_causal, scale, o, dtype, iters=5):
    """Times the loop variants of the attention kernel on these arguments.  Returns the variant, -1 when nothing
    was timed (graph capture), -2 when the problem has no alternatives."""
    best, best_ms = ctypes.c_int(-2), ctypes.c_float(0.0)
    runtime.check(runtime.library().nt_tune_attention(runtime.current_stream(), q, k, v, is_causal, scale, o, dtype, iters, ctypes.byref(best), ctypes.byref(best_ms)))
    if best.value >= 0:
        _save()
    return best.value


def tune_conv2d(x, w, y, dtype, padding_h, padding_w, iters=5):
    """Times the ways to run this convolution (one launch on the tensors as they lie, repacking pass plus GEMM loop,
    gather kernel).  Returns the path (``block_size_m`` value that selects it), or -1 when nothing was timed."""
    best, best_ms = ctypes.c_int(-1), ctypes.c_float(0.0)
    runtime.check(runtime.library().nt_tune_conv2d(runtime.current_stream(), x, w, y, dtype, padding_h, padding_w, iters, ctypes.byref(best), ctypes.byref(best_ms)))
    if best.value >= 0:
        _save()
    return best.value


def tune(input, mat1, mat2, beta, alpha, output, dtype, out_dtype, iters=5):
    """Times the instances on these arguments (:class:`runtime.ArgumentTensor`), records the
    winner in the library and on disk.  Returns ``(instance, milliseconds)``; the instance is -1
    when the stream is being captured into a graph (nothing is timed or recorded then) and -2
    when a single instance takes the problem (nothing to time)."""
    lib = runtime.library()
    best, best_ms = ctypes.c_int(-1), ctypes.c_float(0.0)
    runtime.check(
        lib.nt_tune_gemm(runtime.current_stream(), input, mat1, mat2, beta, alpha, output, dtype, out_dtype, iters, ctypes.byref(best), ctypes.byref(best_ms))
    )
    if best.value < 0:  # nothing was timed: the stream is being captured into a graph
        return best.value, best_ms.value
    _save()
    return best.value, best_ms.value


class AutoTuner:
    """Picks the fastest of several callables per argument signature and keeps the timings on
    disk, in the files the reference's ``AutoTuner`` writes (src/ninetoothed/auto_tuner.py:11-118):

    * ``<sha256(str(key))>.json`` per callable: ``{argument key: milliseconds}``;
    * ``<sha256(str(tuple(keys)))>.json`` for the tuner: ``{argument key: [milliseconds per callable]}``
      (plus one empty object per callable key, as the reference initialises it).

    An argument key is ``"tensor(shape=(..), dtype=float16), 3, name=value"``.  A callable that
    raises :class:`runtime.KernelLaunchError` is timed as infinity.  Timing is wall clock around
    repeated calls, each batch closed by a device synchronisation when a GPU is in use.
    """

    def __init__(self, funcs, keys, cache_dir=None, repetitions=5):
        import json

        self._json = json
        self._funcs = tuple(funcs)
        self._keys = tuple(keys)
        self._func_to_key = dict(zip(self._funcs, self._keys))
        self._repetitions = repetitions
        self._cache_dir = pathlib.Path(cache_dir) if cache_dir is not None else CACHE_DIR / _project_key()
        self._cache_dir.mkdir(parents=True, exist_ok=True)
        self._cache_path = self._cache_dir / (hashlib.sha256(str(self._keys).encode()).hexdigest() + ".json")
        if self._cache_path.exists():
            self._timings = json.loads(self._cache_path.read_text())
        else:
            self._timings = {key: {} for key in self._keys}
        self._best_func = {}

    def __call__(self, *args, **kwargs):
        arg_key = self._make_arg_key(args, kwargs)
        if arg_key not in self._best_func:
            timings = self._get_timings(args, kwargs)
            self._best_func[arg_key] = self._funcs[timings.index(min(timings))]
        return self._best_func[arg_key](*args, **kwargs)

    def _get_timings(self, args, kwargs):
        arg_key = self._make_arg_key(args, kwargs)
        if arg_key in self._timings:
            return self._timings[arg_key]
        timings = [self._get_timing(func, args, kwargs) for func in self._funcs]
        self._timings[arg_key] = timings
        self._cache_path.write_text(self._json.dumps(self._timings))
        return timings

    def _get_timing(self, func, args, kwargs):
        data = self._timings.setdefault(self._func_to_key[func], {})
        arg_key = self._make_arg_key(args, kwargs)
        cache_path = self._get_func_cache_path(func)
        if arg_key not in data and cache_path.exists():
            data.update(self._json.loads(cache_path.read_text()))
        if arg_key in data:
            return data[arg_key]
        try:
            timing = self._measure(lambda: func(*args, **kwargs))
        except runtime.KernelLaunchError:
            timing = float("inf")
        data[arg_key] = timing
        cache_path.write_text(self._json.dumps(data))
        return timing

    def _measure(self, call):
        import time

        try:
            import torch

            synchronize = torch.cuda.synchronize if torch.cuda.is_available() else (lambda: None)
        except ImportError:
            synchronize = lambda: None  # noqa: E731
        call()  # warm-up: first-launch work (plans, specialisation) is not the kernel's time
        synchronize()
        best = float("inf")
        for _ in range(self._repetitions):
            start = time.perf_counter()
            call()
            synchronize()
            best = min(best, (time.perf_counter() - start) * 1e3)
        return best

    def _get_func_cache_path(self, func):
        return self._cache_dir / (hashlib.sha256(str(self._func_to_key[func]).encode()).hexdigest() + ".json")

    @staticmethod
    def _make_arg_key(args, kwargs):
        def make_key(arg):
            if hasattr(arg, "shape") and hasattr(arg, "dtype"):
                return f"tensor(shape={tuple(arg.shape)}, dtype={str(arg.dtype).split('.')[-1]})"
            return str(arg)

        return ", ".join([make_key(arg) for arg in args] + [f"{name}={make_key(arg)}" for name, arg in sorted(kwargs.items())])


def _project_key():
    """Timings belong to one build of the kernels: the key is the library's instance list and version."""
    try:
        names = "|".join(runtime.gemm_config_names()) + "|" + runtime.library().nt_version().decode()
    except Exception:
        names = "no-library"
    return "timings_" + hashlib.sha256(names.encode()).hexdigest()[:16]
