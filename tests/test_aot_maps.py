"""Ahead-of-time packaging of element-wise / reducing programs (tile maps).

The reference packages such programs like any other (tests/test_aot.py:24-60 `test_add`,
:306-343 `test_fp32_scalar`, :346-378 static non-power-of-two sizes; tests/test_aot_auto_tuning.py).
Here the lowering runs once on sample sizes made of `SymInt`s; the C launch function re-checks
the recorded decisions and recomputes the size-dependent fields.

CPU: the symbolic integers themselves; the packaged lowering instantiated in Python for many
sizes and executed by the numpy machine of ``oracle.map_machine`` against numpy; the generated C
code linked against a stand-in `launch_nt_map` that captures the program, compared byte for byte
with the Python instantiation.  GPU: the packaged libraries called like the reference's tests do.
"""

import ctypes
import functools
import subprocess

import numpy as np
import pytest
import torch

import ninetoothed_amd as ninetoothed
import ninetoothed_amd.language as ntl
from ninetoothed_amd import Tensor, aot, mapping
from ninetoothed_amd.recognition import UnsupportedProgram
from ninetoothed_amd.symbolic_int import CWriter, Recorder, SymInt, constant_difference, evaluate, holds, is_symbolic, plain
from oracle.map_machine import Machine

# ---- symbolic integers ---------------------------------------------------------------------


def test_symbolic_integers_carry_their_expression():
    n = SymInt.symbol("x.shape[0]", 1000)
    tiles = (n + 255) // 256
    assert tiles == 4 and is_symbolic(tiles) and type(plain(tiles)) is int
    for size in (1, 255, 256, 257, 10**9):
        assert evaluate(tiles.expr, {"x.shape[0]": size}) == (size + 255) // 256
    assert evaluate((7 - n * 3).expr, {"x.shape[0]": 5}) == -8
    assert evaluate((-n % 7).expr, {"x.shape[0]": 5}) == 2      # floor semantics
    assert evaluate((-n // 7).expr, {"x.shape[0]": 5}) == -1
    # neutral operations keep the value, constants of nested sums fold
    assert (n * 1) is n and (n + 0) is n and (0 + n) is n and n * 0 == 0 and not is_symbolic(n * 0)
    assert ((n - 255) - 1 + 256).expr == n.expr
    assert constant_difference(tiles - 1, tiles) == -1 and constant_difference(n * 2 + 3, n + n) == 3
    assert constant_difference(n, tiles) is None


def test_decisions_on_symbolic_integers_become_guards():
    with Recorder() as recorder:
        n = SymInt.symbol("n", 1000)
        m = SymInt.symbol("m", 1000)
        assert n > 3 and not (n < 3) and max(n, 1) is n and n == m and bool(n)
        assert (n - 998) ** 2 == 4               # no symbolic form: pins the value
        assert float(m) == 1000.0
        assert n == n                            # same expression: nothing to record
        assert (n // m) == 1                     # divisor recorded as non-zero
    guards = recorder.guards
    assert guards[(">", n.expr, ("const", 3))] is True and guards[("<", n.expr, ("const", 3))] is False
    assert guards[("==", n.expr, m.expr)] is True
    assert guards[("==", (n - 998).expr, ("const", 2))] is True
    assert guards[("==", m.expr, ("const", 1000))] is True
    assert guards[("!=", m.expr, ("const", 0))] is True
    assert all(holds(key, outcome, {"n": 1000, "m": 1000}) for key, outcome in guards.items())
    assert not all(holds(key, outcome, {"n": 1001, "m": 1000}) for key, outcome in guards.items())
    # outside a recorder nothing is kept, values still propagate
    assert SymInt.symbol("k", 5) + 1 == 6


def test_expressions_as_c_code():
    n = SymInt.symbol("x.shape[0]", 10)
    writer = CWriter()
    name = writer.value(((n - 1) // 4 + 1).expr)
    lines = writer.take_lines()
    assert lines[0] == "const int64_t t0 = (int64_t)(x.shape[0]);"
    assert "t0 - INT64_C(1)" in lines[1] and "nt_floordiv(t1, INT64_C(4))" in lines[2] and name == "t3"
    assert writer.failure(("<", n.expr, ("const", 1)), False) == "t0 < INT64_C(1)"
    assert writer.failure(("!=", n.expr, ("const", 0)), True) == "!(t0 != INT64_C(0))"


# ---- programs ------------------------------------------------------------------------------


def add_arrangement(input, other, alpha, output, block_size=256):
    return input.tile((block_size,)), other.tile((block_size,)), alpha, output.tile((block_size,))


def add_application(input, other, alpha, output):
    output = input + alpha * other  # noqa: F841


def add_tensors(dtype, size=None):
    shape = {} if size is None else {"shape": (size,)}
    vector = functools.partial(Tensor, **shape) if size is not None else functools.partial(Tensor, 1)
    return vector(dtype=dtype), vector(dtype=dtype), Tensor(0, dtype=ninetoothed.float64), vector(dtype=dtype)


def scale_arrangement(input, scale, output):
    return input.tile((256,)), scale, output.tile((256,))


def scale_application(input, scale, output):
    output = input * scale  # noqa: F841


def copy_arrangement(input, output):
    return input.tile((3,)), output.tile((3,))


def copy_application(input, output):
    output = input  # noqa: F841


def bias_arrangement(x, bias, output):
    tile = (4, 32)
    return x.tile(tile), bias.tile((32,)).unsqueeze(0).expand((x.tile(tile).shape[0], -1)), output.tile(tile)


def bias_application(x, bias, output):
    output = ntl.maximum(x + bias[None, :], 0)  # noqa: F841


def row_softmax_arrangement(input, output):
    return input.tile((1, -1)), output.tile((1, -1))


def row_softmax_application(input, output):
    shifted = input - ntl.max(input)
    numerator = ntl.exp(shifted)
    output = numerator / ntl.sum(numerator)  # noqa: F841


def _kernel(arrangement, application, tensors):
    from ninetoothed_amd.make import Kernel

    types = arrangement(*tensors)
    return Kernel(application, types if isinstance(types, tuple) else (types,))


def _instantiate_and_run(package, arrays, scalars):
    """Runs the packaged lowering for these numpy arrays on the numpy machine; returns False
    when a guard rejects the call.  ``arrays``: parameter name -> array (contiguous or a view)."""
    shapes = {name: array.shape for name, array in arrays.items()}
    strides = {name: tuple(s // array.itemsize for s in array.strides) for name, array in arrays.items()}
    programs = package.instantiate(shapes, strides, scalars)
    if programs is None:
        return False
    for program, (_, _, operand_params) in zip(programs, package.launches):
        flat = {}
        for slot, param in enumerate(operand_params):
            array = arrays[package.parameters[param]]
            base = array.base if array.base is not None else array
            assert array.__array_interface__["data"][0] == base.__array_interface__["data"][0]
            flat[slot] = base.reshape(-1)
        Machine(program, flat).run()
    return True


@pytest.mark.parametrize("size", (1, 3, 255, 256, 257, 1000, 4096, 70001))
def test_packaged_add_for_sizes_unknown_at_packaging(size):
    package = aot.MapPackage(_kernel(add_arrangement, add_application, add_tensors(ninetoothed.float32)), {})
    assert not package.declared and package.guards
    rng = np.random.default_rng(size)
    input, other = rng.standard_normal(size, dtype=np.float32), rng.standard_normal(size, dtype=np.float32)
    output = np.full(size, np.nan, dtype=np.float32)
    assert _instantiate_and_run(package, {"input": input, "other": other, "output": output}, {"alpha": 0.375})
    expected = (input.astype(np.float64) + 0.375 * other.astype(np.float64)).astype(np.float32)
    np.testing.assert_array_equal(output, expected)


def test_packaged_add_takes_strided_views_and_rejects_what_the_lowering_did_not_see():
    package = aot.MapPackage(_kernel(add_arrangement, add_application, add_tensors(ninetoothed.float32)), {})
    rng = np.random.default_rng(0)
    storage = rng.standard_normal(2000, dtype=np.float32)
    input, other = storage[::2], rng.standard_normal(1000, dtype=np.float32)
    output_storage = np.full(3000, np.nan, dtype=np.float32)
    output = output_storage[::3]
    assert _instantiate_and_run(package, {"input": input, "other": other, "output": output}, {"alpha": 2.0})
    np.testing.assert_array_equal(output, (input.astype(np.float64) + 2.0 * other).astype(np.float32))
    assert np.isnan(output_storage[1::3]).all() and np.isnan(output_storage[2::3]).all()
    # operands with different numbers of tiles, a broadcast (stride 0) operand: guards say no; an empty call launches nothing
    shapes = {"input": (1000,), "other": (700,), "output": (1000,)}
    unit = {name: (1,) for name in shapes}
    assert package.instantiate(shapes, unit, {"alpha": 1.0}) is None
    assert package.instantiate({name: (0,) for name in shapes}, unit, {"alpha": 1.0}) == []  # empty tensors: nothing to launch
    assert package.instantiate({name: (1000,) for name in shapes}, dict(unit, other=(0,)), {"alpha": 1.0}) is None


def test_declared_sizes_are_checked_and_leave_no_size_guards():
    package = aot.MapPackage(_kernel(add_arrangement, add_application, add_tensors(ninetoothed.float16, size=1127)), {})
    assert package.declared == [("input", 0, 1127), ("other", 0, 1127), ("output", 0, 1127)]
    assert all("shape" not in repr(key) for key in package.guards)
    unit = {"input": (1,), "other": (1,), "output": (1,)}
    assert package.instantiate({name: (1127,) for name in unit}, unit, {"alpha": 1.0}) is not None
    assert package.instantiate({name: (1128,) for name in unit}, unit, {"alpha": 1.0}) is None


@pytest.mark.parametrize("rows, cols", ((1, 1), (4, 32), (5, 33), (37, 100), (64, 256)))
def test_packaged_bias_relu_two_dimensions(rows, cols):
    tensors = (Tensor(2, dtype=ninetoothed.float32), Tensor(1, dtype=ninetoothed.float32), Tensor(2, dtype=ninetoothed.float32))
    package = aot.MapPackage(_kernel(bias_arrangement, bias_application, tensors), {})
    rng = np.random.default_rng(rows * 1000 + cols)
    x, bias = rng.standard_normal((rows, cols), dtype=np.float32), rng.standard_normal(cols, dtype=np.float32)
    output = np.full((rows, cols), np.nan, dtype=np.float32)
    assert _instantiate_and_run(package, {"x": x, "bias": bias, "output": output}, {})
    np.testing.assert_array_equal(output, np.maximum(x + bias[None, :], 0))


@pytest.mark.parametrize("rows, cols", ((1, 7), (13, 100), (8, 1024)))
def test_packaged_whole_tile_reductions(rows, cols):
    tensors = (Tensor(2, dtype=ninetoothed.float32), Tensor(2, dtype=ninetoothed.float32))
    package = aot.MapPackage(_kernel(row_softmax_arrangement, row_softmax_application, tensors), {})
    assert package.launches[0][0].num_phases == 2
    rng = np.random.default_rng(cols)
    x = rng.standard_normal((rows, cols), dtype=np.float32)
    output = np.full((rows, cols), np.nan, dtype=np.float32)
    assert _instantiate_and_run(package, {"input": x, "output": output}, {})
    expected = torch.softmax(torch.from_numpy(x), dim=1).numpy()
    np.testing.assert_allclose(output, expected, rtol=1e-5, atol=1e-6)


def test_what_cannot_be_packaged_says_so():
    with pytest.raises(UnsupportedProgram, match="element type"):
        aot.MapPackage(_kernel(copy_arrangement, copy_application, (Tensor(1), Tensor(1))), {})
    jagged = (Tensor(2, jagged_dim=1, dtype=ninetoothed.float32), Tensor(2, jagged_dim=1, dtype=ninetoothed.float32))
    with pytest.raises(UnsupportedProgram, match="Jagged"):
        aot.MapPackage(_kernel(lambda x, y: (x.tile((1, 64)), y.tile((1, 64))), copy_application, jagged), {})


# ---- the generated C code ------------------------------------------------------------------

_CAPTURE_SOURCE = """
#include <string.h>
#include "ninetoothed_hip.h"
static NineToothedMapProgram captured[4];
static int count = 0;
NineToothedResult launch_nt_map(NineToothedStream stream, const NineToothedMapProgram *program) {
    (void)stream;
    if (count < 4) memcpy(&captured[count], program, sizeof *program);
    ++count;
    return 0;
}
int capture_count(void) { int n = count; count = 0; return n; }
const void *capture_program(int index) { return &captured[index]; }
unsigned long capture_size(void) { return sizeof(NineToothedMapProgram); }
"""


def _compile_against_capture(tmp_path, name, package):
    header, source = package.c_source(name)
    (tmp_path / f"{name}.h").write_text(header)
    (tmp_path / f"{name}.c").write_text(source)
    (tmp_path / "capture.c").write_text(_CAPTURE_SOURCE)
    library = tmp_path / f"{name}_capture.so"
    command = ["gcc", "-shared", "-fPIC", "-O1", "-Wall", "-Werror", f"-I{aot.INCLUDE_DIR}", f"-I{tmp_path}", str(tmp_path / f"{name}.c"), str(tmp_path / "capture.c"), "-o", str(library)]
    result = subprocess.run(command, capture_output=True, text=True)
    assert result.returncode == 0, result.stderr
    lib = ctypes.CDLL(str(library))
    lib.capture_program.restype = ctypes.c_void_p
    lib.capture_size.restype = ctypes.c_ulong
    assert lib.capture_size() == ctypes.sizeof(mapping.MapProgram)
    return lib


class _HostTensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("shape", ctypes.POINTER(ctypes.c_uint64)), ("strides", ctypes.POINTER(ctypes.c_int64))]


def _host_tensor(address, shape, strides, keep):
    shape_array = (ctypes.c_uint64 * len(shape))(*shape)
    strides_array = (ctypes.c_int64 * len(strides))(*strides)
    keep.extend((shape_array, strides_array))
    return _HostTensor(address, shape_array, strides_array)


def _host_scalar(value, keep):
    buffer = ctypes.c_double(value) if isinstance(value, float) else ctypes.c_int64(value)
    keep.append(buffer)
    return _HostTensor(ctypes.addressof(buffer), None, None)


@pytest.mark.parametrize("size, stride", ((1000003, 1), (4096, 1), (300, 2), (1, 1), (0, 1), (77, 0)))
def test_generated_c_code_builds_the_same_program_as_the_python_instantiation(tmp_path, size, stride):
    package = aot.MapPackage(_kernel(add_arrangement, add_application, add_tensors(ninetoothed.float16)), {})
    lib = _compile_against_capture(tmp_path, "add_c", package)
    lib.launch_add_c.argtypes = [ctypes.c_void_p] + [_HostTensor] * 4
    keep = []
    addresses = {"input": 0x1000, "other": 0x200000, "output": 0x4000000}
    shapes = {name: (size,) for name in addresses}
    strides = {"input": (stride,), "other": (1,), "output": (1,)}
    result = lib.launch_add_c(
        None, _host_tensor(addresses["input"], shapes["input"], strides["input"], keep), _host_tensor(addresses["other"], shapes["other"], strides["other"], keep),
        _host_scalar(-1.5, keep), _host_tensor(addresses["output"], shapes["output"], strides["output"], keep),
    )
    expected = package.instantiate(shapes, strides, {"alpha": -1.5})
    launched = lib.capture_count()
    if expected is None:
        assert result == 1 and launched == 0
        return
    if expected == []:
        assert result == 0 and launched == 0
        return
    assert result == 0 and launched == len(expected) == 1
    for index, (program, (_, _, operand_params)) in enumerate(zip(expected, package.launches)):
        for slot, param in enumerate(operand_params):
            program.operands[slot].data = addresses[package.parameters[param]]
        captured = ctypes.string_at(lib.capture_program(index), ctypes.sizeof(mapping.MapProgram))
        assert captured == bytes(program)


def test_generated_c_code_two_dimensions_and_declared_sizes(tmp_path):
    tensors = (Tensor(shape=(37, 100), dtype=ninetoothed.float32), Tensor(1, dtype=ninetoothed.float32), Tensor(2, dtype=ninetoothed.float32))
    package = aot.MapPackage(_kernel(bias_arrangement, bias_application, tensors), {})
    lib = _compile_against_capture(tmp_path, "bias_c", package)
    lib.launch_bias_c.argtypes = [ctypes.c_void_p] + [_HostTensor] * 3
    keep = []
    for rows, accepted in ((37, True), (38, False)):
        shapes = {"x": (rows, 100), "bias": (100,), "output": (rows, 100)}
        strides = {"x": (100, 1), "bias": (1,), "output": (128, 1)}
        result = lib.launch_bias_c(None, *(_host_tensor(0x1000 * (i + 1), shapes[name], strides[name], keep) for i, name in enumerate(("x", "bias", "output"))))
        expected = package.instantiate(shapes, strides, {})
        assert (expected is not None) == accepted and result == (0 if accepted else 1)
        if accepted:
            assert lib.capture_count() == 1
            program = expected[0]
            for slot, param in enumerate(package.launches[0][2]):
                program.operands[slot].data = 0x1000 * (param + 1)
            assert ctypes.string_at(lib.capture_program(0), ctypes.sizeof(mapping.MapProgram)) == bytes(program)


def test_make_packages_a_tile_map(tmp_path):
    kernel = ninetoothed.make(add_arrangement, add_application, add_tensors(ninetoothed.float16), caller="hip", kernel_name="add_fp16", output_dir=tmp_path)
    source = (tmp_path / "add_fp16.c").read_text()
    assert "static const NineToothedMapProgram add_fp16_program_0" in source and "launch_nt_map(stream, &program)" in source
    assert "*(const double *)alpha.data" in source
    assert hasattr(ctypes.CDLL(kernel.library_path), "launch_add_fp16")


# ---- GPU: the packaged libraries, called like the reference's tests call theirs -----------


@pytest.mark.gpu
@pytest.mark.parametrize("dtype, ninetoothed_dtype, tolerance", ((torch.float32, ninetoothed.float32, 1e-5), (torch.float16, ninetoothed.float16, 1e-3)))
@pytest.mark.parametrize("size", (98432, 1127, 256, 5))
def test_packaged_add_on_the_gpu(tmp_path, size, dtype, ninetoothed_dtype, tolerance):
    kernel = ninetoothed.make(add_arrangement, add_application, add_tensors(ninetoothed_dtype), caller="hip", kernel_name="add", output_dir=tmp_path)
    input, other = torch.randn(size, dtype=dtype, device="cuda"), torch.randn(size, dtype=dtype, device="cuda")
    alpha = torch.randn((), dtype=torch.float64)
    output = torch.full_like(input, float("nan"))
    kernel(input, other, alpha, output)
    assert torch.allclose(output, torch.add(input, other, alpha=alpha.item()), rtol=tolerance, atol=tolerance)
    # a view with a stride goes through the same package
    wide = torch.randn(size, 2, dtype=dtype, device="cuda")
    kernel(wide[:, 0], other, 2, output)
    assert torch.allclose(output, wide[:, 0] + 2 * other, rtol=tolerance, atol=tolerance)
    if size > 300:
        with pytest.raises(RuntimeError):
            kernel(input[:-300], other, alpha, output)  # another number of tiles
    kernel(input[:0], other[:0], alpha, output[:0])  # empty tensors: nothing to launch, no error


@pytest.mark.gpu
def test_packaged_fp32_scalar_and_static_non_power_of_two_sizes(tmp_path):
    tensors = (Tensor(1, dtype=ninetoothed.float32), Tensor(0, dtype=ninetoothed.float32), Tensor(1, dtype=ninetoothed.float32))
    kernel = ninetoothed.make(scale_arrangement, scale_application, tensors, caller="hip", kernel_name="fp32_scalar", output_dir=tmp_path)
    input = torch.randn(256, dtype=torch.float32, device="cuda")
    output = torch.empty_like(input)
    kernel(input, 0.125, output)
    assert torch.allclose(output, input * 0.125)

    kernel = ninetoothed.make(copy_arrangement, copy_application, (Tensor(1, dtype=ninetoothed.float32), Tensor(1, dtype=ninetoothed.float32)), caller="hip", kernel_name="copy3", output_dir=tmp_path)
    input = torch.randn((3,), dtype=torch.float32, device="cuda")
    output = torch.empty_like(input)
    kernel(input, output)
    assert torch.equal(input, output)


@pytest.mark.gpu
def test_packaged_normalisation_on_the_gpu(tmp_path):
    tensors = (Tensor(2, dtype=ninetoothed.float32), Tensor(2, dtype=ninetoothed.float32))
    kernel = ninetoothed.make(row_softmax_arrangement, row_softmax_application, tensors, caller="hip", kernel_name="row_softmax", output_dir=tmp_path)
    for rows, cols in ((13, 100), (512, 1024), (3, 5000)):
        input = torch.randn(rows, cols, device="cuda")
        output = torch.empty_like(input)
        kernel(input, output)
        assert torch.allclose(output, torch.softmax(input, dim=1), rtol=1e-5, atol=1e-6)


def _add_premake(size=None, dtype=None, block_size=None):
    arrangement = functools.partial(add_arrangement, block_size=block_size)
    return arrangement, add_application, add_tensors(dtype, size=size)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype, ninetoothed_dtype, tolerance", ((torch.float32, ninetoothed.float32, 1e-5), (torch.float16, ninetoothed.float16, 1e-3)))
@pytest.mark.parametrize("size", (20260128, 1127))
def test_build_dispatches_over_packaged_tile_maps(tmp_path, size, dtype, ninetoothed_dtype, tolerance):
    """tests/test_aot_auto_tuning.py:42-107 of the reference, restated."""
    configs = (
        ((), {"size": 20260128, "dtype": ninetoothed.float16, "block_size": 256}, {}),
        ((), {"size": 20260128, "dtype": ninetoothed.float16, "block_size": 1024}, {}),
        ((), {"size": 20260128, "dtype": ninetoothed.float32, "block_size": 512}, {}),
        ((), {"size": 20260128, "dtype": ninetoothed.float32, "block_size": 1024}, {}),
        ((), {"size": 1127, "dtype": ninetoothed.float16, "block_size": 64}, {"num_warps": 4}),
        ((), {"size": 1127, "dtype": ninetoothed.float16, "block_size": 64}, {"num_warps": 8}),
        ((), {"size": 1127, "dtype": ninetoothed.float16, "block_size": 256}, {"num_warps": 4, "num_stages": 1}),
        ((), {"size": 1127, "dtype": ninetoothed.float16, "block_size": 256}, {"num_warps": 8, "num_stages": 1}),
        ((), {"size": 1127, "dtype": ninetoothed.float32, "block_size": 512}, {}),
    )
    kernel = ninetoothed.build(_add_premake, configs, meta_parameters=("block_size",), caller="hip", kernel_name="add", output_dir=tmp_path)
    input, other = torch.randn((size,), dtype=dtype, device="cuda"), torch.randn((size,), dtype=dtype, device="cuda")
    alpha = torch.randn((), dtype=torch.float64)
    output = torch.empty_like(input)
    kernel(input, other, alpha, output, size, ninetoothed_dtype)
    assert torch.allclose(output, torch.add(input, other, alpha=alpha.item()), rtol=tolerance, atol=tolerance)
    with pytest.raises(RuntimeError):  # a size no configuration names
        kernel(input[:100], other[:100], alpha, output[:100], 100, ninetoothed_dtype)
