"""The C ABI library: it loads, exports every symbol include/ninetoothed_hip.h
declares, and rejects bad requests without touching a GPU."""

import ctypes
import pathlib
import re

import pytest

from ninetoothed_amd import runtime

ROOT = pathlib.Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "ninetoothed_hip.h"


def _declared_functions():
    text = HEADER.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(launch_nt_\w+|nt_\w+)\s*\(", text)
    return sorted(set(names))


def test_header_declares_the_entry_points():
    names = _declared_functions()
    for expected in ("launch_nt_matmul", "launch_nt_addmm", "launch_nt_softmax", "launch_nt_attention", "launch_nt_conv2d", "nt_tune_gemm"):
        assert expected in names


def test_library_exports_every_declared_symbol():
    library = ctypes.CDLL(str(runtime.LIBRARY_PATH))
    for name in _declared_functions():
        assert hasattr(library, name), f"{name} is declared in the header but not exported"


def test_python_binding_covers_the_header():
    assert set(_declared_functions()) == set(runtime.exported_symbols())


def test_version_and_instance_table():
    library = runtime.library()
    assert library.nt_version().decode().startswith("nt_hip")
    names = runtime.gemm_config_names()
    assert len(names) >= 3 and any("any-stride" in name for name in names)
    buffer = ctypes.create_string_buffer(8)
    assert library.nt_gemm_config_name(10_000, buffer, 8) == runtime.NO_KERNEL


def test_struct_layout_matches_the_header():
    # {void *data; uint64_t *shape; int64_t *strides;} passed by value
    assert ctypes.sizeof(runtime.ArgumentTensor) == 3 * ctypes.sizeof(ctypes.c_void_p)
    assert [name for name, _ in runtime.ArgumentTensor._fields_] == ["data", "shape", "strides"]
    scalar = runtime.ArgumentTensor.from_scalar(0.25)
    assert ctypes.cast(scalar.data, ctypes.POINTER(ctypes.c_double))[0] == 0.25
    flag = runtime.ArgumentTensor.from_scalar(True)
    assert ctypes.cast(flag.data, ctypes.POINTER(ctypes.c_int64))[0] == 1


def test_launch_error_class():
    with pytest.raises(runtime.KernelLaunchError, match="error code: 1"):
        runtime.check(1)
    runtime.check(0)


def test_requests_without_a_kernel_are_refused_on_the_host():
    # validation happens before any device call, so this runs without a GPU
    library = runtime.library()
    a = runtime.ArgumentTensor.from_layout(0, (4, 4), (4, 1))
    fp64 = runtime.DATA_TYPE_INDEX["fp64"]
    assert library.launch_nt_matmul(None, a, a, a, fp64, fp64, 0, 0, 0) == runtime.NO_KERNEL
    assert library.launch_nt_softmax(None, a, a, runtime.DATA_TYPE_INDEX["i32"], 0) == runtime.NO_KERNEL
    mismatched = runtime.ArgumentTensor.from_layout(0, (5, 4), (4, 1))
    assert library.launch_nt_matmul(None, a, mismatched, a, runtime.DATA_TYPE_INDEX["fp16"], runtime.DATA_TYPE_INDEX["fp16"], 0, 0, 0) != 0  # hipErrorInvalidValue
    empty = runtime.ArgumentTensor.from_layout(0, (0, 4), (4, 1))
    assert library.launch_nt_softmax(None, empty, empty, runtime.DATA_TYPE_INDEX["fp32"], 0) == 0


def test_tuning_cache_reads_and_writes_the_reference_csv_format(tmp_path):
    # the file layout of src/ninetoothed/build.py:683-703 (csv.writer rows: an empty row and the
    # default first, then problem / choice pairs), read by templates/auto_tuning_cache.h:27-75;
    # a problem row starts with the program (0 matmul / addmm, 1 attention, 2 conv2d)
    import csv
    import ctypes

    from ninetoothed_amd import auto_tuner, runtime

    lib = runtime.library()
    names = runtime.gemm_config_names()
    fast = next(index for index, name in enumerate(names) if name.startswith("256x256x32"))
    fp16 = runtime.DATA_TYPE_INDEX["fp16"]
    file_format = lib.nt_tune_file_format()
    path = tmp_path / "cache.csv"
    with open(path, "w") as handle:
        writer = csv.writer(handle)
        writer.writerow(())
        writer.writerow((file_format,))
        writer.writerow((runtime.TUNE_GEMM, fp16, fp16, 4096, 2048, 1024, 1, 0))
        writer.writerow((fast, 256, 256, 32))
        writer.writerow((runtime.TUNE_GEMM, fp16, fp16, 4096, 2048, 1024, 1, 1))  # the same sizes with a transposed rhs
        writer.writerow((fast + 1, 256, 256, 64))
        writer.writerow((runtime.TUNE_GEMM, fp16, fp16, 1024, 1024, 1024, 0, 0))
        writer.writerow((fast, 128, 128, 64))  # block sizes of another instance: a file from another numbering, dropped
        writer.writerow((runtime.TUNE_GEMM, fp16, fp16, 2048, 1024, 1024, 0, 0))
        writer.writerow((fast,))  # no block sizes: dropped
        writer.writerow((runtime.TUNE_ATTENTION, fp16, 4, 32, 2048, 2048, 128, 1))
        writer.writerow((99,))  # no such variant: dropped
        writer.writerow((runtime.TUNE_CONV2D, fp16, 32, 256, 28, 28, 256, 3, 3, 1, 1, 1))
        writer.writerow((0,))  # no such path: dropped
        writer.writerow((runtime.TUNE_ATTENTION, fp16, 4, 32, 4096, 4096, 128, 1))
        writer.writerow((3,))
        writer.writerow((runtime.TUNE_CONV2D, fp16, 32, 256, 56, 56, 256, 3, 3, 1, 1, 1))
        writer.writerow((2,))
        writer.writerow((7, 1, 2, 3))  # a program this build does not have: skipped
        writer.writerow((1,))
        writer.writerow((runtime.TUNE_GEMM, fp16, fp16, 64, 64, 64, 0, 0))
        writer.writerow((-5,))  # no choice: skipped
    entries = ctypes.c_int(-1)
    assert lib.nt_tune_cache_load(str(path).encode(), ctypes.byref(entries)) == 0
    assert entries.value == 4
    assert lib.nt_tune_cache_lookup(fp16, fp16, 4096, 2048, 1024, 1) == fast
    assert auto_tuner.lookup(fp16, fp16, 4096, 2048, 1024, True, rhs_layout=1) == fast + 1
    assert lib.nt_tune_cache_lookup(fp16, fp16, 64, 64, 64, 0) == -1
    assert lib.nt_tune_cache_lookup(fp16, fp16, 1024, 1024, 1024, 0) == -1
    assert lib.nt_tune_cache_lookup(fp16, fp16, 2048, 1024, 1024, 0) == -1
    assert auto_tuner.lookup_problem(runtime.TUNE_ATTENTION, (fp16, 4, 32, 2048, 2048, 128, 1)) == -1
    assert auto_tuner.lookup_problem(runtime.TUNE_CONV2D, (fp16, 32, 256, 28, 28, 256, 3, 3, 1, 1, 1)) == -1
    assert lib.nt_tune_cache_lookup(fp16, fp16, 4096, 2048, 1024, 0) == -1
    assert auto_tuner.lookup_problem(runtime.TUNE_ATTENTION, (fp16, 4, 32, 4096, 4096, 128, 1)) == 3
    assert auto_tuner.lookup_problem(runtime.TUNE_ATTENTION, (fp16, 4, 32, 4096, 4096, 128, 0)) == -1
    assert auto_tuner.lookup_problem(runtime.TUNE_CONV2D, (fp16, 32, 256, 56, 56, 256, 3, 3, 1, 1, 1)) == 2

    saved = tmp_path / "saved.csv"
    assert lib.nt_tune_cache_save(str(saved).encode()) == 0
    rows = list(csv.reader(open(saved)))
    assert rows[0] == [] and rows[1] == [str(file_format)]  # the default pair carries the numbering's format
    pairs = {tuple(rows[i]): tuple(rows[i + 1]) for i in range(2, len(rows) - 1, 2)}
    assert pairs[tuple(str(v) for v in (0, fp16, fp16, 4096, 2048, 1024, 1, 0))] == (str(fast), "256", "256", "32")
    assert pairs[tuple(str(v) for v in (1, fp16, 4, 32, 4096, 4096, 128, 1))] == ("3",)
    assert pairs[tuple(str(v) for v in (2, fp16, 32, 256, 56, 56, 256, 3, 3, 1, 1, 1))] == ("2",)
    assert lib.nt_tune_cache_load(str(tmp_path / "missing.csv").encode(), None) != 0

    # a file written under another numbering of the variants is ignored whole
    other = tmp_path / "other_format.csv"
    with open(other, "w") as handle:
        writer = csv.writer(handle)
        writer.writerow(())
        writer.writerow((file_format - 1,))
        writer.writerow((runtime.TUNE_GEMM, fp16, fp16, 512, 1024, 2048, 0, 0))
        writer.writerow((fast, 256, 256, 32))
    assert lib.nt_tune_cache_load(str(other).encode(), ctypes.byref(entries)) == 0
    assert entries.value == 0
    assert lib.nt_tune_cache_lookup(fp16, fp16, 512, 1024, 2048, 0) == -1


def test_auto_tuner_json_caches(tmp_path):
    """The reference's tests/test_auto_tuner.py:9-80: callables with known delays, the two kinds of
    JSON files, and a second call that no longer measures."""
    import json
    import time

    from ninetoothed_amd.auto_tuner import AutoTuner

    def delay_foo(*args, **kwargs):
        return 0.001 * (2 * len(args) + len(kwargs))

    def delay_bar(*args, **kwargs):
        return 0.001 * (len(args) + 2 * len(kwargs))

    def foo(*args, **kwargs):
        time.sleep(delay_foo(*args, **kwargs))

    def bar(*args, **kwargs):
        time.sleep(delay_bar(*args, **kwargs))

    for args, kwargs in (((1,), {"a": 2, "b": 4, "c": 6, "d": 8}), ((1, 3, 5), {"a": 2})):
        tuner = AutoTuner((foo, bar), ("foo", "bar"), cache_dir=tmp_path / f"cache{len(args)}")
        assert not tuner._cache_path.exists() and not tuner._get_func_cache_path(foo).exists()
        start = time.perf_counter()
        tuner(*args, **kwargs)
        first = time.perf_counter() - start
        assert tuner._cache_path.exists() and tuner._get_func_cache_path(foo).exists() and tuner._get_func_cache_path(bar).exists()
        start = time.perf_counter()
        tuner(*args, **kwargs)
        assert time.perf_counter() - start < first
        key = tuner._make_arg_key(args, kwargs)
        assert key == ", ".join([str(a) for a in args] + [f"{k}={v}" for k, v in sorted(kwargs.items())])
        expected = foo if delay_foo(*args, **kwargs) < delay_bar(*args, **kwargs) else bar
        assert tuner._best_func[key] is expected
        # the files hold what the reference's reader expects
        per_func = json.loads(tuner._get_func_cache_path(foo).read_text())
        assert list(per_func) == [key] and per_func[key] >= delay_foo(*args, **kwargs) * 1e3
        whole = json.loads(tuner._cache_path.read_text())
        assert set(whole) == {"foo", "bar", key} and len(whole[key]) == 2
        # a new tuner over the same directory starts from the files and measures nothing
        again = AutoTuner((foo, bar), ("foo", "bar"), cache_dir=tmp_path / f"cache{len(args)}")
        assert again._get_timings(args, kwargs) == whole[key]


def test_auto_tuner_tensor_keys_and_failed_launches(tmp_path):
    import torch

    from ninetoothed_amd.auto_tuner import AutoTuner
    from ninetoothed_amd.runtime import KernelLaunchError

    def refuses(x):
        raise KernelLaunchError(1)

    def works(x):
        return x

    tuner = AutoTuner((refuses, works), ("refuses", "works"), cache_dir=tmp_path)
    x = torch.zeros(3, 4, dtype=torch.float16)
    assert tuner(x) is x
    assert tuner._make_arg_key((x,), {}) == "tensor(shape=(3, 4), dtype=float16)"
    assert tuner._timings["tensor(shape=(3, 4), dtype=float16)"][0] == float("inf")
