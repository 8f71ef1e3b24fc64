"""Element-wise / reducing tile programs (the reference's tests/test_add.py,
test_clone.py, test_pad.py, test_pow.py, test_dropout.py, test_max_pool2d.py,
test_generation.py:139-151) through the interpreter kernel.

CPU tests check the lowering (index and value programs) by executing it with
``oracle.map_machine`` against ``oracle.programs.tile_map``, which restates the
reference's semantics with offset tables; GPU tests run ``launch_nt_map``
through ``make`` / ``jit`` and compare with torch at the reference's test
shapes and with the oracle on small ones.
"""

import functools
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import ninetoothed_amd as ninetoothed
import ninetoothed_amd.language as ntl
from ninetoothed_amd import Symbol, Tensor, block_size, mapping, programs
from ninetoothed_amd.language import libdevice
from ninetoothed_amd.make import _dtype_tag, _storage
from ninetoothed_amd.recognition import UnsupportedProgram
from oracle import programs as oracle
from oracle.arrangement import View
from oracle.map_machine import Machine

# ---- the programs, written as in the reference's tests ------------------------------------

BLOCK_SIZE = Symbol("BLOCK_SIZE", meta=True)


@ninetoothed.jit
def add_kernel(
    lhs: Tensor(1).tile((BLOCK_SIZE,)),
    rhs: Tensor(1).tile((BLOCK_SIZE,)),
    output: Tensor(1).tile((BLOCK_SIZE,)),
):
    output = lhs + rhs  # noqa: F841


def clone_arrangement(input, output):
    block_shape = (ninetoothed.block_size(), ninetoothed.block_size())
    return input.tile(block_shape), output.tile(block_shape)


def clone_application(input, output):
    output = input  # noqa: F841


def pad_arrangement(input, output, input_slices, output_slices):
    return input[input_slices], output[output_slices]


def pow_arrangement(input, exponent, output, BLOCK_SIZE=block_size()):
    return input.tile((BLOCK_SIZE,)), exponent.tile((BLOCK_SIZE,)), output.tile((BLOCK_SIZE,))


def pow_application(input, exponent, output):
    output = libdevice.pow(input, exponent)  # noqa: F841


def dropout_arrangement(input, p, seed, output, BLOCK_SIZE=block_size()):
    return input.tile((BLOCK_SIZE,)), p, seed, output.tile((BLOCK_SIZE,))


def dropout_application(input, p, seed, output):
    output = ntl.where(ntl.rand(seed, input.offsets()) > p, input / (1 - p), 0)  # noqa: F841


def max_pool2d_arrangement(input, output, ceil_mode=False):
    BLOCK_SIZE = Symbol("BLOCK_SIZE", meta=True)
    WINDOW_HEIGHT = Symbol("WINDOW_HEIGHT", constexpr=True, upper_bound=16)
    WINDOW_WIDTH = Symbol("WINDOW_WIDTH", constexpr=True, upper_bound=16)
    input_arranged = input.tile((1, 1, WINDOW_HEIGHT, WINDOW_WIDTH), floor_mode=not ceil_mode)
    input_arranged = input_arranged.ravel()
    input_arranged = input_arranged.flatten(end_dim=4).flatten(start_dim=1)
    input_arranged = input_arranged.tile((BLOCK_SIZE, -1))
    output_arranged = output.tile((1, 1, 1, 1))
    output_arranged = output_arranged.ravel()
    output_arranged = output_arranged.flatten(end_dim=4).flatten(start_dim=1)
    output_arranged = output_arranged.tile((BLOCK_SIZE, -1))
    output_arranged.dtype = output_arranged.dtype.squeeze(1)
    return input_arranged, output_arranged


def max_pool2d_application(input, output):
    output = ntl.max(input, axis=1)  # noqa: F841


def scalar_add_arrangement(input, other, output, block_size=ninetoothed.block_size()):
    return input.tile((block_size,)), other, output.tile((block_size,))


def scalar_add_application(input, other, output):
    output = input + other  # noqa: F841


def fused_arrangement(x, y, scale, output):
    block_shape = (ninetoothed.block_size(), ninetoothed.block_size())
    return x.tile(block_shape), y.tile(block_shape), scale, output.tile(block_shape)


def fused_application(x, y, scale, output):
    output = ntl.where(x > y, ntl.exp(x - y) * scale, ntl.maximum(x, 0.5) / y)  # noqa: F841


def row_sum_arrangement(input, output):
    return input.tile((1, -1)).squeeze(1), output.tile((1,))


def row_sum_application(input, output):
    output = ntl.sum(input) * 2  # noqa: F841


def _pad_config(shape, pad):
    """tests/test_pad.py:67-95 of the reference, restated."""
    ndim = len(shape)
    output_shape, input_slices, output_slices = list(shape), [], []
    for i in range(ndim):
        left, right = pad[2 * (ndim - 1 - i)], pad[2 * (ndim - 1 - i) + 1]
        output_shape[i] += left + right
        input_slices.append(slice(max(0, -left), min(shape[i], shape[i] + right)))
        output_slices.append(slice(max(0, left), output_shape[i] - max(0, right)))
    return output_shape, tuple(input_slices), tuple(output_slices)


# ---- CPU: lowering executed by the numpy machine ------------------------------------------


def _run_on_machine(kernel, args, kwargs=None):
    kwargs = kwargs or {}
    env = kernel._environment(args, kwargs, check_device=False)
    flat = {}

    def storage(p):
        if p not in flat:
            tensor = _storage(args, p)
            size = 1 + sum((n - 1) * abs(s) for n, s in zip(tensor.shape, tensor.stride())) if tensor.numel() else 0
            flat[p] = torch.as_strided(tensor, (size,), (1,)).numpy()
        return flat[p]

    for store in kernel.program.stores:
        built = mapping.build(store, kernel.types, args, env, lambda p: _dtype_tag(_storage(args, p).dtype), lambda p: 0)
        if built is None:
            continue
        program, _, _, operand_params = built
        Machine(program, {slot: storage(p) for slot, p in enumerate(operand_params)}).run()


def test_lowering_add():
    lhs, rhs = torch.rand(1000), torch.rand(1000)
    out = torch.empty(1000)
    assert add_kernel.kind == "map"
    _run_on_machine(add_kernel, (lhs, rhs, out))
    assert torch.equal(out, lhs + rhs)


def test_lowering_clone_strided_against_oracle():
    kernel = ninetoothed.make(clone_arrangement, clone_application, (Tensor(2), Tensor(2)))
    source = torch.randn(37 * 50)
    input = torch.as_strided(source, (37, 23), (50, 2))
    out = torch.zeros(37, 23)
    _run_on_machine(kernel, (input, out))
    # the oracle works on offset tables of the strided source
    table = (np.arange(37)[:, None] * 50 + np.arange(23)[None, :] * 2).astype(np.intp)
    expected = np.zeros(37 * 23, dtype=np.float32)
    oracle.tile_map(lambda tile: tile, [(source.numpy(), View(table, [2]).tile((8, 16)), None)], expected, View.of_shape((37, 23)).tile((8, 16)))
    assert np.array_equal(out.numpy().reshape(-1), expected)
    assert torch.equal(out, input)


@pytest.mark.parametrize("shape, pad_", (((20, 13), (-3, 2, 4, -1)), ((2, 3), (1, 1, 1, 2)), ((2, 3, 4), (1, 3, 1, 0, 0, 0)), ((2, 3), (-1, -1, 0, 0))))
def test_lowering_pad(shape, pad_):
    input = torch.randn(shape)
    output_shape, input_slices, output_slices = _pad_config(shape, pad_)
    out = torch.full(output_shape, 7.0)
    kernel = ninetoothed.make(pad_arrangement, clone_application, (Tensor(len(shape)), Tensor(len(shape)), input_slices, output_slices))
    _run_on_machine(kernel, (input, out))
    assert torch.equal(out, F.pad(input, pad_, "constant", 7.0))


@pytest.mark.parametrize("ceil_mode", (False, True))
def test_lowering_max_pool2d_against_oracle(ceil_mode):
    kernel = ninetoothed.make(
        functools.partial(max_pool2d_arrangement, ceil_mode=ceil_mode), max_pool2d_application, (Tensor(4, other=float("-inf")), Tensor(4))
    )
    x = torch.randn(2, 3, 8, 7).half()
    expected = F.max_pool2d(x.float(), (3, 3), ceil_mode=ceil_mode).half()
    out = torch.zeros_like(expected)
    _run_on_machine(kernel, (x, out), dict(WINDOW_HEIGHT=3, WINDOW_WIDTH=3))
    assert torch.equal(out, expected)
    # the same arrangement on offset tables
    view_in = View.of_shape(x.shape).tile((1, 1, 3, 3), floor_mode=not ceil_mode).ravel().flatten(end_dim=4).flatten(start_dim=1).tile((4, -1))
    view_out = View.of_shape(expected.shape).tile((1, 1, 1, 1)).ravel().flatten(end_dim=4).flatten(start_dim=1).tile((4, -1)).squeeze(1, level=1)
    result = np.zeros(expected.numel(), dtype=np.float16)
    oracle.tile_map(lambda tile: tile.max(axis=1), [(x.numpy().reshape(-1), view_in, -np.inf)], result, view_out)
    assert np.array_equal(result, out.numpy().reshape(-1))


def test_lowering_dropout_matches_published_philox():
    kernel = ninetoothed.make(dropout_arrangement, dropout_application, (Tensor(1), Tensor(0), Tensor(0), Tensor(1)))
    x = torch.randn(349).half()
    out = torch.empty_like(x)
    p, seed = 0.3, 123456789
    _run_on_machine(kernel, (x, p, seed, out))
    keep = oracle.triton_rand(seed, np.arange(349)) > np.float32(p)
    scaled = (x.float().numpy() / np.float32(1 - p)).astype(np.float16)
    assert np.array_equal(out.numpy(), np.where(keep, scaled, np.float16(0)))
    assert abs(keep.mean() - 0.7) < 0.05


def test_philox_known_answers():
    # Random123's kat_vectors for philox4x32-10
    f = 0xFFFFFFFF
    assert [int(w) for w in oracle.philox4x32((0, 0, 0, 0), (0, 0))] == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert [int(w) for w in oracle.philox4x32((f, f, f, f), (f, f))] == [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]
    assert [int(w) for w in oracle.philox4x32((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0))] == [
        0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1,
    ]


def test_lowering_types_follow_the_reference_promotion():
    kernel = ninetoothed.make(fused_arrangement, fused_application, (Tensor(2), Tensor(2), Tensor(0), Tensor(2)))
    x, y = torch.randn(9, 11).half(), (torch.rand(9, 11) + 0.5).half()
    out = torch.empty(9, 11).half()
    _run_on_machine(kernel, (x, y, 1.5, out))
    xf, yf = x.float(), y.float()
    first = (torch.exp((x - y).float()).half().float() * 1.5)  # fp16 tile times run-time float: fp32
    second = (torch.maximum(x, torch.tensor(0.5).half()).float() / yf).half().float()  # stays fp16
    expected = torch.where(xf > yf, first, second).half()
    assert torch.allclose(out.float(), expected.float(), rtol=2e-3, atol=2e-3)


def test_lowering_full_reduction_and_post_operation():
    kernel = ninetoothed.make(row_sum_arrangement, row_sum_application, (Tensor(2), Tensor(1)))
    x = torch.randn(5, 33)
    out = torch.empty(5)
    _run_on_machine(kernel, (x, out))
    assert torch.allclose(out, x.sum(dim=1) * 2, rtol=1e-5, atol=1e-5)


def test_scalar_constexpr_and_empty_programs():
    kernel = ninetoothed.make(scalar_add_arrangement, scalar_add_application, (Tensor(1), Tensor(0, constexpr=True), Tensor(1)))
    x = torch.randn(1086)
    out = torch.empty_like(x)
    _run_on_machine(kernel, (x, math.pi, out))
    assert torch.equal(out, x + math.pi)


def test_programs_outside_the_class_are_reported():
    def arrangement(input, output):
        return input.tile((1, -1)), output.tile((1, -1))

    def application(input, output):
        output = ntl.dot(input, ntl.trans(input))  # noqa: F841

    with pytest.raises(UnsupportedProgram):
        ninetoothed.make(arrangement, application, (Tensor(2), Tensor(2)))


# ---- GPU: the interpreter kernel through make / jit -------------------------------------------

gpu = pytest.mark.gpu


def _served_by_map(kernel):
    assert kernel.last_plan.startswith("launch_nt_map"), kernel.last_plan


@gpu
def test_add():
    lhs, rhs = torch.rand(98432, device="cuda"), torch.rand(98432, device="cuda")
    out = torch.empty_like(lhs)
    add_kernel(lhs, rhs, out)
    _served_by_map(add_kernel)
    assert torch.equal(out, lhs + rhs)


@gpu
def test_clone_strided():
    input = torch.empty_strided((641, 280), (700, 300), device="cuda")
    input.copy_(torch.randn(641, 280, device="cuda"))
    out = torch.empty_like(input)
    kernel = ninetoothed.make(clone_arrangement, clone_application, (Tensor(2), Tensor(2)))
    kernel(input, out)
    _served_by_map(kernel)
    assert out.shape == input.shape and torch.equal(out, input)


@gpu
@pytest.mark.parametrize("dtype", (torch.float32, torch.float16))
@pytest.mark.parametrize("value", (0, 1, -1, float("-inf"), math.pi))
@pytest.mark.parametrize("shape, pad_", (((2026, 1207), (-100, 20, 99, -10)), ((2, 3), (1, 1, 1, 2)), ((2, 3, 4), (1, 3, 1, 0, 0, 0)), ((2, 3), (-1, -1, 0, 0))))
def test_pad(shape, pad_, value, dtype):
    input = torch.randn(shape, dtype=dtype, device="cuda")
    output_shape, input_slices, output_slices = _pad_config(shape, pad_)
    out = torch.full(output_shape, value, dtype=dtype, device="cuda")
    kernel = ninetoothed.make(pad_arrangement, clone_application, (Tensor(len(shape)), Tensor(len(shape)), input_slices, output_slices))
    kernel(input, out)
    _served_by_map(kernel)
    assert torch.equal(out, F.pad(input, pad_, "constant", value))


@gpu
def test_pow():
    input, exponent = torch.rand(44925, device="cuda"), torch.rand(44925, device="cuda")
    out = torch.empty_like(input)
    kernel = ninetoothed.make(pow_arrangement, pow_application, (Tensor(1), Tensor(1), Tensor(1)))
    kernel(input, exponent, out)
    _served_by_map(kernel)
    assert torch.allclose(out, torch.pow(input, exponent), equal_nan=True)


@gpu
def test_dropout():
    x = torch.randn(349, dtype=torch.float16, device="cuda")
    out = torch.empty_like(x)
    kernel = ninetoothed.make(dropout_arrangement, dropout_application, (Tensor(1), Tensor(0), Tensor(0), Tensor(1)))
    p = 0.3
    for seed in (7, 2**31 - 5):  # a second call with another seed reuses the plan
        kernel(x, p, seed, out)
        _served_by_map(kernel)
        keep = oracle.triton_rand(seed, np.arange(349)) > np.float32(p)
        scaled = (x.float().cpu().numpy() / np.float32(1 - p)).astype(np.float16)
        assert np.array_equal(out.cpu().numpy(), np.where(keep, scaled, np.float16(0)))
    non_zero_ratio = out.nonzero().numel() / x.numel()
    assert abs(non_zero_ratio - (1 - p)) < 0.05
    assert torch.allclose(out[out != 0], (x[out != 0] / (1 - p)))


@gpu
@pytest.mark.parametrize("ceil_mode", (False, True))
def test_max_pool2d(ceil_mode):
    x = torch.randn(32, 3, 64, 64, dtype=torch.float16, device="cuda")
    expected = F.max_pool2d(x, (3, 3), ceil_mode=ceil_mode)
    out = torch.empty_like(expected)
    kernel = ninetoothed.make(
        functools.partial(max_pool2d_arrangement, ceil_mode=ceil_mode), max_pool2d_application, (Tensor(4, other=float("-inf")), Tensor(4))
    )
    kernel(x, out, WINDOW_HEIGHT=3, WINDOW_WIDTH=3)
    _served_by_map(kernel)
    assert torch.equal(out, expected)


@gpu
def test_non_int_constexpr():
    x = torch.randn(1086, device="cuda")
    out = torch.empty_like(x)
    kernel = ninetoothed.make(scalar_add_arrangement, scalar_add_application, (Tensor(1), Tensor(0, constexpr=True), Tensor(1)))
    kernel(x, math.pi, out)
    _served_by_map(kernel)
    assert torch.allclose(out, x + math.pi)


@gpu
def test_fused_expression_against_machine():
    kernel = ninetoothed.make(fused_arrangement, fused_application, (Tensor(2), Tensor(2), Tensor(0), Tensor(2)))
    x, y = torch.randn(130, 70).half(), (torch.rand(130, 70) + 0.5).half()
    expected = torch.empty(130, 70).half()
    _run_on_machine(kernel, (x, y, 1.5, expected))
    out = torch.empty(130, 70, dtype=torch.float16, device="cuda")
    kernel(x.cuda(), y.cuda(), 1.5, out)
    _served_by_map(kernel)
    assert torch.allclose(out.cpu().float(), expected.float(), rtol=2e-3, atol=2e-3)


@gpu
@pytest.mark.parametrize("interpret", ("0", "1"))
def test_interpreter_and_specialised_kernels_agree(interpret, monkeypatch):
    # NT_MAP_INTERPRET=1 keeps launch_nt_map on the interpreter kernel (the path taken when
    # hipRTC is missing); both must produce the machine's result
    monkeypatch.setenv("NT_MAP_INTERPRET", interpret)
    kernel = ninetoothed.make(dropout_arrangement, dropout_application, (Tensor(1), Tensor(0), Tensor(0), Tensor(1)))
    x = torch.randn(5000).half()
    expected = torch.empty_like(x)
    _run_on_machine(kernel, (x, 0.25, 99, expected))
    out = torch.empty(5000, dtype=torch.float16, device="cuda")
    kernel(x.cuda(), 0.25, 99, out)
    assert torch.equal(out.cpu(), expected)
    pool = ninetoothed.make(
        functools.partial(max_pool2d_arrangement, ceil_mode=True), max_pool2d_application, (Tensor(4, other=float("-inf")), Tensor(4))
    )
    image = torch.randn(3, 5, 17, 19, dtype=torch.float16, device="cuda")
    pooled = torch.empty(3, 5, 6, 7, dtype=torch.float16, device="cuda")
    pool(image, pooled, WINDOW_HEIGHT=3, WINDOW_WIDTH=3)
    assert torch.equal(pooled, F.max_pool2d(image, (3, 3), ceil_mode=True))
    if interpret == "0":
        assert "nt_map_specialised" in open(pool._source).read()


@gpu
def test_row_sum():
    kernel = ninetoothed.make(row_sum_arrangement, row_sum_application, (Tensor(2), Tensor(1)))
    x = torch.randn(300, 257, device="cuda")
    out = torch.empty(300, device="cuda")
    kernel(x, out)
    _served_by_map(kernel)
    assert torch.allclose(out, x.sum(dim=1) * 2, rtol=1e-4, atol=1e-4)


def _row_max_application(input, output):
    output = ntl.max(input) - 1.0  # noqa: F841


@gpu
@pytest.mark.parametrize("rows, cols", ((3, 100003), (64, 16384), (2048, 16385), (1, 1 << 20)))
def test_few_long_rows_are_reduced_by_whole_workgroups(rows, cols):
    """Few outputs over long ranges: the workgroup shares an output, its waves exchange partial results through
    LDS (one wave per output otherwise).  Sums against float64, maxima exactly, a NaN in a row reaches its maximum."""
    x = torch.randn(rows, cols, device="cuda")
    out = torch.empty(rows, device="cuda")
    kernel = ninetoothed.make(row_sum_arrangement, row_sum_application, (Tensor(2), Tensor(1)))
    kernel(x, out)
    _served_by_map(kernel)
    assert torch.allclose(out.double(), x.double().sum(dim=1) * 2, rtol=1e-5, atol=1e-2)
    kernel = ninetoothed.make(row_sum_arrangement, _row_max_application, (Tensor(2, other=float("-inf")), Tensor(1)))
    x[rows - 1, cols // 3] = 1000.0
    if rows > 1:
        x[0, cols - 1] = float("nan")
    kernel(x, out)
    _served_by_map(kernel)
    expected = x.max(dim=1).values - 1.0
    assert torch.equal(out.isnan(), expected.isnan()) and torch.equal(out.nan_to_num(0.0), expected.nan_to_num(0.0))


@gpu
def test_empty_tensor_and_no_store():
    def arrangement(x):
        return x.tile((ninetoothed.block_size(),)).unsqueeze(0)

    def application(x):
        x

    kernel = ninetoothed.make(arrangement, application, (Tensor(1),))
    kernel(torch.randn((0,), device="cuda"))
    out = torch.empty(0, device="cuda")
    add_kernel(torch.empty(0, device="cuda"), torch.empty(0, device="cuda"), out)


def _expand_arrangement(x, BLOCK_SIZE=block_size()):
    return (x.expand((BLOCK_SIZE,)).tile((BLOCK_SIZE,)),)


def _no_store_application(x):
    x


def _single_tensor_arrangement(x):
    return x.tile((ninetoothed.block_size(),))


def test_programs_without_stores_are_accepted():
    # tests/test_expand.py:9-23 and tests/test_generation.py:59-70 of the reference
    assert ninetoothed.make(_expand_arrangement, _no_store_application, (Tensor(1),)).kind == "map"
    assert ninetoothed.make(_single_tensor_arrangement, _no_store_application, (Tensor(1),)).kind == "map"


@gpu
def test_expand_on_an_empty_tensor():
    kernel = ninetoothed.make(_expand_arrangement, _no_store_application, (Tensor(1),))
    kernel(torch.empty((0,), device="cuda"))
    kernel = ninetoothed.make(_single_tensor_arrangement, _no_store_application, (Tensor(1),))
    kernel(torch.randn(100, device="cuda"))


# ---- data-dependent level indices (tests/test_generation.py:72-115 of the reference) ----------


def _scatter_rows_arrangement(input, indices, output):
    input_arranged = input.tile((1, -1)).squeeze(1)
    input_arranged.dtype = input_arranged.dtype.squeeze(0)
    indices_arranged = indices.tile((1,))
    output_arranged = output.tile((1, -1)).tile((-1, -1)).squeeze(0).expand((input_arranged.shape[0],))
    output_arranged.dtype = output_arranged.dtype.squeeze(1)
    output_arranged.dtype.dtype = output_arranged.dtype.dtype.squeeze(0)
    return input_arranged, indices_arranged, output_arranged


def _scatter_rows_application(input, index, output):
    row = index

    output[row] = input


def _gather_rows_arrangement(table, indices, output):
    table_arranged = table.tile((1, -1)).tile((-1, -1)).squeeze(0).expand((indices.shape[0],))
    table_arranged.dtype = table_arranged.dtype.squeeze(1)
    table_arranged.dtype.dtype = table_arranged.dtype.dtype.squeeze(0)
    indices_arranged = indices.tile((1,))
    output_arranged = output.tile((1, -1)).squeeze(1)
    output_arranged.dtype = output_arranged.dtype.squeeze(0)
    return table_arranged, indices_arranged, output_arranged


def _gather_rows_application(table, index, output):
    output = table[index] * 2  # noqa: F841


def _scatter_kernel():
    options = {"constexpr": True}
    tensors = (Tensor(2, shape_options=options), Tensor(1, shape_options=options), Tensor(2, shape_options=options))
    return ninetoothed.make(_scatter_rows_arrangement, _scatter_rows_application, tensors)


def test_lowering_scatter_rows_by_loaded_index():
    kernel = _scatter_kernel()
    input = torch.randn(10, 128)
    indices = torch.randperm(1024)[:10]
    out = torch.zeros(1024, 128)
    expected = out.clone()
    _run_on_machine(kernel, (input, indices, out))
    expected[indices] = input
    assert torch.equal(out, expected)


def test_lowering_out_of_range_indices_are_skipped():
    kernel = _scatter_kernel()
    input = torch.randn(4, 8)
    indices = torch.tensor([3, -1, 20, 0])
    out = torch.zeros(20, 8)
    _run_on_machine(kernel, (input, indices, out))
    expected = torch.zeros(20, 8)
    expected[3], expected[0] = input[0], input[3]
    assert torch.equal(out, expected)


def test_lowering_gather_rows_by_loaded_index():
    kernel = ninetoothed.make(_gather_rows_arrangement, _gather_rows_application, (Tensor(2), Tensor(1), Tensor(2)))
    table = torch.randn(50, 24)
    indices = torch.randint(0, 50, (17,))
    out = torch.zeros(17, 24)
    _run_on_machine(kernel, (table, indices, out))
    assert torch.equal(out, table[indices] * 2)


@gpu
@pytest.mark.parametrize("interpret", ("0", "1"))
def test_rows_by_loaded_index(interpret, monkeypatch):
    monkeypatch.setenv("NT_MAP_INTERPRET", interpret)
    kernel = _scatter_kernel()
    input = torch.randn(10, 128, device="cuda")
    indices = torch.randperm(1024, device="cuda")[:10]
    out = torch.empty(1024, 128, device="cuda").normal_()
    expected = out.clone()
    kernel(input, indices, out)
    _served_by_map(kernel)
    expected[indices] = input
    assert torch.equal(out, expected)
    gather = ninetoothed.make(_gather_rows_arrangement, _gather_rows_application, (Tensor(2), Tensor(1), Tensor(2)))
    table = torch.randn(5000, 96, device="cuda")
    picks = torch.randint(0, 5000, (333,), device="cuda")
    rows = torch.empty(333, 96, device="cuda")
    gather(table, picks, rows)
    assert torch.equal(rows, table[picks] * 2)


def _mul_add_arrangement(lhs, rhs, output, block=block_size()):
    return lhs.tile((block,)), rhs.tile((block,)), output.tile((block,))


def _mul_add_application(lhs, rhs, output):
    output = lhs * rhs + 1  # noqa: F841


@gpu
@pytest.mark.parametrize("interpret", ("0", "1"))
def test_operations_are_rounded_one_by_one(interpret, monkeypatch):
    # a multiplication followed by an addition must not be contracted into a fused multiply-add
    monkeypatch.setenv("NT_MAP_INTERPRET", interpret)
    kernel = ninetoothed.make(_mul_add_arrangement, _mul_add_application, (Tensor(1),) * 3)
    lhs, rhs = torch.randn(100000), torch.randn(100000)
    out = torch.empty(100000, device="cuda")
    kernel(lhs.cuda(), rhs.cuda(), out)
    assert torch.equal(out.cpu(), lhs * rhs + 1)


# ---- elements of whole tensors by computed indices / raw pointers -----------------------------
# (the other three applications of the reference's tests/test_clone.py:23-37 and the atomic sum of
#  tests/test_data_ptr.py:11-18)


def _clone_by_pointer(input, output):
    output = ntl.load(  # noqa: F841
        input.source.data_ptr() + input.offsets(0)[:, None] * input.source.stride(0) + input.offsets(1)[None, :] * input.source.stride(1)
    )


def _clone_by_source_load(input, output):
    output = input.source[input.offsets(0)[:, None], input.offsets(1)[None, :]]  # noqa: F841


def _clone_by_source_store(input, output):
    output.source[output.offsets(0)[:, None], output.offsets(1)[None, :]] = input


_CLONES = (_clone_by_pointer, _clone_by_source_load, _clone_by_source_store)


def _transposed_gather(input, output):
    output = input.source[input.offsets(0)[None, :], input.offsets(1)[:, None]]  # noqa: F841


def _sum_arrangement(input, output, BLOCK_SIZE=1024):
    input_arranged = input.tile((BLOCK_SIZE,))
    return input_arranged, output.tile((-1,)).expand(input_arranged.shape)


def _sum_application(input, output):
    ntl.atomic_add(output.source.data_ptr(), ntl.sum(input))


def _strided_matrix(rows, cols, row_stride, col_stride, device="cpu"):
    storage = torch.randn(rows * row_stride, device=device)
    return torch.as_strided(storage, (rows, cols), (row_stride, col_stride))


@pytest.mark.parametrize("application", _CLONES)
def test_lowering_clone_through_indices_and_pointers(application):
    kernel = ninetoothed.make(clone_arrangement, application, (Tensor(2), Tensor(2)))
    assert kernel.kind == "map"
    input = _strided_matrix(41, 28, 30, 1)
    out = torch.full((41, 28), float("nan"))
    _run_on_machine(kernel, (input, out))
    assert torch.equal(out, input)


def test_lowering_rejects_offsets_laid_along_the_wrong_dimension():
    def arrangement(input, output):
        return input.tile((8, 8)), output.tile((8, 8))

    kernel = ninetoothed.make(arrangement, _transposed_gather, (Tensor(2), Tensor(2)))
    with pytest.raises(UnsupportedProgram):
        _run_on_machine(kernel, (torch.randn(16, 16), torch.empty(16, 16)))


def test_lowering_atomic_sum_through_a_pointer():
    kernel = ninetoothed.make(_sum_arrangement, _sum_application, (Tensor(1), Tensor(1, shape_options={"constexpr": True})))
    input = torch.randn(5000, dtype=torch.float64)
    out = torch.zeros(1, dtype=torch.float64)
    _run_on_machine(kernel, (input, out))
    # one partial sum per tile of 1024, added in tile order
    expected = sum(float(chunk.sum()) for chunk in input.split(1024))
    assert abs(out.item() - expected) < 1e-9
    assert abs(out.item() - input.sum().item()) < 1e-9


@gpu
@pytest.mark.parametrize("interpret", ("0", "1"))
@pytest.mark.parametrize("application", _CLONES)
def test_clone_through_indices_and_pointers(application, interpret, monkeypatch):
    """tests/test_clone.py:55-69 of the reference: a 641 x 280 matrix with strides (700, 300)."""
    monkeypatch.setenv("NT_MAP_INTERPRET", interpret)
    kernel = ninetoothed.make(clone_arrangement, application, (Tensor(2), Tensor(2)))
    input = torch.empty_strided((641, 280), (700, 300), device="cuda")
    input.copy_(torch.randn(641, 280))
    out = torch.full((641, 280), float("nan"), device="cuda")
    kernel(input, out)
    _served_by_map(kernel)
    assert torch.equal(out, input)


@gpu
@pytest.mark.parametrize("interpret", ("0", "1"))
def test_atomic_sum_through_a_pointer(interpret, monkeypatch):
    """tests/test_data_ptr.py:34-42 of the reference."""
    monkeypatch.setenv("NT_MAP_INTERPRET", interpret)
    kernel = ninetoothed.make(_sum_arrangement, _sum_application, (Tensor(1), Tensor(1, shape_options={"constexpr": True})))
    input = torch.randn(64180, device="cuda")
    for _ in range(2):
        out = torch.zeros(1, device="cuda")
        kernel(input, out)
        assert torch.allclose(out[0], torch.sum(input))
    counts = torch.zeros(1, dtype=torch.int32, device="cuda")
    kernel(torch.ones(64180, dtype=torch.int32, device="cuda"), counts)
    assert counts.item() == 64180


# ---- jagged tensors (the reference's tests/test_jagged.py) --------------------------------------

_JAGGED_BLOCK = Symbol("block_size", constexpr=True)


def _to_padded_arrangement(input, output, block_size=_JAGGED_BLOCK):
    tile_shape = (1,) + tuple(block_size for _ in range(1, input.ndim))
    return input.tile(tile_shape), output.tile(tile_shape)


def _jagged_copy_arrangement(dst, src, jagged_dim, block_size=_JAGGED_BLOCK):
    tile_shape = (1,) + tuple(block_size for _ in range(1, dst.ndim))
    return dst.tile(tile_shape), src.expand(tuple(-1 if dim != jagged_dim else dst.shape[dim] for dim in range(src.ndim))).tile(tile_shape)


def _jagged_copy_application(dst, src):
    dst = src  # noqa: F841


def _jagged_batches(jagged_dim, lengths, batch_shape, device="cpu"):
    batches = tuple(torch.randn(batch_shape[: jagged_dim - 1] + (n,) + batch_shape[jagged_dim:], device=device) for n in lengths)
    return torch.nested.nested_tensor(batches, layout=torch.jagged)


@pytest.mark.parametrize("jagged_dim", (1, 2))
def test_lowering_jagged_to_padded_and_expand(jagged_dim):
    nested = _jagged_batches(jagged_dim, (3, 6, 1, 9), (5, 7))
    kernel = ninetoothed.make(_to_padded_arrangement, clone_application, (Tensor(3, jagged_dim=jagged_dim, other=-1), Tensor(3)))
    expected = torch.nested.to_padded_tensor(nested, -1.0)
    out = torch.full(expected.shape, float("nan"))
    _run_on_machine(kernel, (nested, out), {"block_size": 4})
    assert torch.equal(out, expected)

    # a dense row / column written into every entry of a jagged destination
    copy = ninetoothed.make(functools.partial(_jagged_copy_arrangement, jagged_dim=jagged_dim), _jagged_copy_application, (Tensor(3, jagged_dim=jagged_dim), Tensor(3)))
    src = torch.randn(tuple(size if dim != jagged_dim else 1 for dim, size in enumerate(expected.shape)))
    before = nested.values().clone()
    _run_on_machine(copy, (nested, src), {"block_size": 4})
    assert not torch.equal(nested.values(), before)
    padded = torch.nested.to_padded_tensor(nested, float("nan"))
    inside = ~torch.isnan(padded)
    assert inside.sum().item() == nested.values().numel()
    assert torch.equal(padded[inside], src.expand_as(padded)[inside])


def test_jagged_arguments_are_checked():
    kernel = ninetoothed.make(_to_padded_arrangement, clone_application, (Tensor(3, jagged_dim=1, other=-1), Tensor(3)))
    nested = _jagged_batches(2, (3, 4), (5, 7))
    with pytest.raises(ValueError):  # jagged along another dimension than declared
        kernel._environment((nested, torch.empty(2, 5, 4)), {"block_size": 4}, check_device=False)
    with pytest.raises(TypeError):  # a dense tensor where a jagged one is declared
        kernel._environment((torch.empty(2, 5, 4), torch.empty(2, 5, 4)), {"block_size": 4}, check_device=False)
    with pytest.raises(ValueError):
        Tensor(3, jagged_dim=0)


@gpu
@pytest.mark.parametrize("interpret", ("0", "1"))
@pytest.mark.parametrize("num_batches", (2, 7, 16))
@pytest.mark.parametrize("jagged_dim", (1, 2))
def test_jagged_to_padded_tensor_and_expand(jagged_dim, num_batches, interpret, monkeypatch):
    """tests/test_jagged.py:55-158 of the reference (ndim 3, padding -1, block size 32)."""
    import random

    monkeypatch.setenv("NT_MAP_INTERPRET", interpret)
    generator = random.Random(17 * num_batches + jagged_dim)
    batch_shape = (generator.randint(1, 300), generator.randint(1, 300))
    lengths = [generator.randint(1, 300) for _ in range(num_batches)]
    nested = _jagged_batches(jagged_dim, lengths, batch_shape, device="cuda")
    kernel = ninetoothed.make(_to_padded_arrangement, clone_application, (Tensor(3, jagged_dim=jagged_dim, other=-1), Tensor(3)))
    expected = torch.nested.to_padded_tensor(nested, -1.0)
    out = torch.full(expected.shape, float("nan"), device="cuda")
    kernel(nested, out, block_size=32)
    _served_by_map(kernel)
    assert torch.equal(out, expected)

    copy = ninetoothed.make(functools.partial(_jagged_copy_arrangement, jagged_dim=jagged_dim), _jagged_copy_application, (Tensor(3, jagged_dim=jagged_dim), Tensor(3)))
    src = torch.randn(tuple(size if dim != jagged_dim else 1 for dim, size in enumerate(expected.shape)), device="cuda")
    copy(nested, src, block_size=32)
    padded = torch.nested.to_padded_tensor(nested, float("nan"))
    inside = ~torch.isnan(padded)
    assert inside.sum().item() == nested.values().numel()
    assert torch.equal(padded[inside], src.expand_as(padded)[inside])


@gpu
def test_offsets_beyond_32_bits():
    """Specialised kernels compute offsets in 32 bits when every index provably fits; this one does not."""
    kernel = ninetoothed.make(scalar_add_arrangement, scalar_add_application, (Tensor(1), Tensor(0), Tensor(1)))
    n = (1 << 31) + 4096
    input = torch.zeros(n, dtype=torch.int8, device="cuda")
    input[-5:] = torch.arange(5, dtype=torch.int8, device="cuda")
    input[:3] = 7
    out = torch.full((n,), -1, dtype=torch.int8, device="cuda")
    kernel(input, 1, out)
    _served_by_map(kernel)
    assert out[:4].tolist() == [8, 8, 8, 1] and out[-5:].tolist() == [1, 2, 3, 4, 5]
    assert int(out.to(torch.int32).sum().item()) == n + 21 + 10


# ---- whole-tile reductions used on the elements of the tile (normalisations) ---------------------


def _rows(tensor):
    arranged = tensor.tile((1, -1)).squeeze(1)
    arranged.dtype = arranged.dtype.squeeze(0)
    return arranged


def _row_arrangement(input, output):
    return _rows(input), _rows(output)


def _row_weight_arrangement(input, weight, output):
    return _rows(input), weight.tile((-1,)).expand((input.shape[0],)), _rows(output)


def _scaled_softmax_application(input, output):
    shifted = input * 2 - ntl.max(input * 2)
    numerator = ntl.exp(shifted)
    output = numerator / ntl.sum(numerator)  # noqa: F841


def _rms_norm_application(input, weight, output):
    mean_square = ntl.sum(input * input) / input.shape[-1]
    output = input * ntl.rsqrt(mean_square + 1e-6) * weight  # noqa: F841


def _layer_norm_application(input, weight, output):
    mean = ntl.sum(input) / input.shape[-1]
    centred = input - mean
    variance = ntl.sum(centred * centred) / input.shape[-1]
    output = centred * ntl.rsqrt(variance + 1e-5) * weight  # noqa: F841


def _normalisation_cases(device, dtype=torch.float32, rows=7, cols=300):
    x = torch.randn(rows, cols, device=device, dtype=dtype)
    w = torch.randn(cols, device=device, dtype=dtype)
    xf, wf = x.float(), w.float()
    softmax = ninetoothed.make(_row_arrangement, _scaled_softmax_application, (Tensor(2), Tensor(2)))
    rms_norm = ninetoothed.make(_row_weight_arrangement, _rms_norm_application, (Tensor(2), Tensor(1), Tensor(2)))
    layer_norm = ninetoothed.make(_row_weight_arrangement, _layer_norm_application, (Tensor(2), Tensor(1), Tensor(2)))
    return (
        (softmax, (x,), torch.softmax(xf * 2, -1)),
        (rms_norm, (x, w), xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + 1e-6) * wf),
        (layer_norm, (x, w), F.layer_norm(xf, (cols,), wf, None, 1e-5)),
    )


def test_lowering_whole_tile_reductions_in_tile_mode():
    for kernel, inputs, expected in _normalisation_cases("cpu"):
        assert kernel.kind == "map"
        out = torch.full_like(inputs[0], float("nan"))
        _run_on_machine(kernel, (*inputs, out))
        assert torch.allclose(out, expected, rtol=1e-5, atol=1e-6)


def test_tile_mode_program_layout():
    kernel, inputs, _ = _normalisation_cases("cpu")[2]
    out = torch.empty_like(inputs[0])
    args = (*inputs, out)
    env = kernel._environment(args, {}, check_device=False)
    program, description, _, _ = mapping.build(kernel.program.stores[0], kernel.types, args, env, lambda p: _dtype_tag(args[p].dtype), lambda p: 0)
    assert program.num_phases == 2 and program.num_grid == 1 and program.reduce_op == 0
    assert 0 < program.phase_end[0] < program.phase_end[1] < program.value_code_length
    assert "whole-tile reduction" in description
    # the second phase (variance) reads the first one (mean); nothing reads a later phase
    words = [program.value_code[i] for i in range(program.value_code_length)]
    reduced = [(i, w >> 8) for i, w in enumerate(words) if w & 0xFF == mapping.V["REDUCED"]]
    assert any(program.phase_end[0] <= i < program.phase_end[1] and k == 0 for i, k in reduced)
    assert all(k < sum(i >= program.phase_end[j] for j in range(program.num_phases)) for i, k in reduced)


@gpu
@pytest.mark.parametrize("interpret", ("0", "1"))
@pytest.mark.parametrize("dtype, tolerance", ((torch.float32, 1e-5), (torch.float16, 1e-2)))
def test_whole_tile_reductions_on_the_gpu(dtype, tolerance, interpret, monkeypatch):
    monkeypatch.setenv("NT_MAP_INTERPRET", interpret)
    # (rows of up to 512 elements take a wave each, four to a workgroup; rows of 2049 ... 8192 elements run
    # 512 threads per row, up to 16384 1024 threads, longer ones 256 again)
    for rows, cols in ((7, 300), (64, 4096), (3, 1), (1001, 32), (77, 512), (6, 513), (5, 2049), (33, 8192), (9, 8200), (17, 16384), (3, 20000)):
        for kernel, inputs, expected in _normalisation_cases("cuda", dtype, rows, cols):
            out = torch.full_like(inputs[0], float("nan"))
            kernel(*inputs, out)
            _served_by_map(kernel)
            assert torch.allclose(out.float(), expected, rtol=tolerance, atol=tolerance), (rows, cols, kernel.kernel_name)


# ---- a tile of lower rank broadcast along a tile of the expression (`bias[None, :]`) -------------


def _bias_arrangement(input, row_bias, column_bias, output):
    block_m, block_n = ninetoothed.block_size(), ninetoothed.block_size()
    tiled = input.tile((block_m, block_n))
    rows = row_bias.tile((block_n,)).unsqueeze(0).expand((tiled.shape[0], -1))
    columns = column_bias.tile((block_m,)).unsqueeze(1).expand((-1, tiled.shape[1]))
    return tiled, rows, columns, output.tile((block_m, block_n))


def _bias_application(input, row_bias, column_bias, output):
    output = input + row_bias[None, :] + column_bias[:, None] * 2  # noqa: F841


def test_lowering_broadcast_subscripts_on_tiles():
    kernel = ninetoothed.make(_bias_arrangement, _bias_application, (Tensor(2), Tensor(1), Tensor(1), Tensor(2)))
    x, r, c = torch.randn(37, 50), torch.randn(50), torch.randn(37)
    out = torch.full_like(x, float("nan"))
    _run_on_machine(kernel, (x, r, c, out), {name: 8 for name in kernel.meta_symbols})
    assert torch.equal(out, x + r[None, :] + c[:, None] * 2)


@gpu
@pytest.mark.parametrize("interpret", ("0", "1"))
def test_broadcast_subscripts_on_tiles(interpret, monkeypatch):
    monkeypatch.setenv("NT_MAP_INTERPRET", interpret)
    kernel = ninetoothed.make(_bias_arrangement, _bias_application, (Tensor(2), Tensor(1), Tensor(1), Tensor(2)))
    x, r, c = torch.randn(641, 280, device="cuda"), torch.randn(280, device="cuda"), torch.randn(641, device="cuda")
    out = torch.full_like(x, float("nan"))
    kernel(x, r, c, out)
    _served_by_map(kernel)
    assert torch.equal(out, x + r[None, :] + c[:, None] * 2)


@gpu
def test_one_kernel_called_from_several_threads():
    """Calls with one signature share a prepared launch whose argument structs are filled per call."""
    import threading

    n = 1 << 16
    matmul = ninetoothed.make(programs.matmul.arrangement, programs.matmul.application, programs.matmul.tensors())
    failures = []

    def worker(seed):
        generator = torch.Generator(device="cuda").manual_seed(seed)
        lhs = torch.randn(n, device="cuda", generator=generator)
        rhs = torch.randn(n, device="cuda", generator=generator)
        a = torch.randn(256, 128, device="cuda", generator=generator).half()
        b = torch.randn(128, 256, device="cuda", generator=generator).half()
        for _ in range(100):
            out = torch.empty(n, device="cuda")
            add_kernel(lhs, rhs, out, BLOCK_SIZE=1024)
            c = torch.empty(256, 256, dtype=torch.float16, device="cuda")
            matmul(a, b, c)
            if not torch.equal(out, lhs + rhs) or not torch.allclose(c, a @ b, rtol=1e-2, atol=1e-2):
                failures.append(seed)
                return

    threads = [threading.Thread(target=worker, args=(seed,)) for seed in range(4)]
    for thread in threads:
        thread.start()
    for thread in threads:
        thread.join()
    assert not failures


# ---- axis reductions laid back over the tile (`ntl.max(x, 1)[:, None]`) ---------------------------


def _row_block_arrangement(input, output):
    return input.tile((8, -1)), output.tile((8, -1))


def _row_block_softmax_application(input, output):
    shifted = input - ntl.max(input, 1)[:, None]
    numerator = ntl.exp(shifted)
    output = numerator / ntl.sum(numerator, axis=1)[:, None]  # noqa: F841


def _column_normalise_application(input, output):
    output = input / ntl.sum(input * input, axis=0)[None, :]  # noqa: F841


def test_lowering_axis_reductions_used_on_the_tile():
    x = torch.randn(37, 50)
    kernel = ninetoothed.make(_row_block_arrangement, _row_block_softmax_application, (Tensor(2, other=float("-inf")), Tensor(2)))
    out = torch.full_like(x, float("nan"))
    _run_on_machine(kernel, (x, out))
    assert torch.allclose(out, torch.softmax(x, -1), rtol=1e-5, atol=1e-7)

    def columns(input, output):
        return input.tile((-1, 4)), output.tile((-1, 4))

    kernel = ninetoothed.make(columns, _column_normalise_application, (Tensor(2), Tensor(2)))
    out = torch.full_like(x, float("nan"))
    _run_on_machine(kernel, (x, out))
    assert torch.allclose(out, x / (x * x).sum(0, keepdim=True), rtol=1e-5, atol=1e-7)

    def mixed(input, output):
        output = input - ntl.max(input, 1)[:, None] - ntl.max(input)  # noqa: F841

    kernel = ninetoothed.make(_row_block_arrangement, mixed, (Tensor(2, other=float("-inf")), Tensor(2)))
    with pytest.raises(UnsupportedProgram):
        _run_on_machine(kernel, (x, torch.empty_like(x)))


@gpu
@pytest.mark.parametrize("interpret", ("0", "1"))
def test_axis_reductions_used_on_the_tile(interpret, monkeypatch):
    monkeypatch.setenv("NT_MAP_INTERPRET", interpret)
    x = torch.randn(641, 1000, device="cuda")
    kernel = ninetoothed.make(_row_block_arrangement, _row_block_softmax_application, (Tensor(2, other=float("-inf")), Tensor(2)))
    out = torch.full_like(x, float("nan"))
    kernel(x, out)
    _served_by_map(kernel)
    assert torch.allclose(out, torch.softmax(x, -1), rtol=1e-5, atol=1e-7)


@gpu
@pytest.mark.parametrize("dtype", (torch.float32, torch.float16))
@pytest.mark.parametrize("shape", ((1000, 128), (37, 5000), (4096, 1000), (64, 127)))
def test_reductions_over_the_contiguous_dimension_share_a_wave(shape, dtype):
    """Row reductions of a row-major matrix: the generated kernel gives an output element to a wave,
    whose lanes stride the row (one thread per row would make a wave read 64 rows at once).
    Column reductions and short rows keep one thread per output.  Sums, maxima with a NaN, two
    reduced dimensions."""
    rows, cols = shape
    x = torch.randn(rows, cols, device="cuda").to(dtype)
    out = torch.full((rows,), float("nan"), dtype=dtype, device="cuda")
    kernel = ninetoothed.make(row_sum_arrangement, row_sum_application, (Tensor(2), Tensor(1)))
    kernel(x, out)
    _served_by_map(kernel)
    tolerance = dict(rtol=1e-4, atol=1e-3) if dtype == torch.float32 else dict(rtol=1e-2, atol=0.25)
    assert torch.allclose(out.float(), x.float().sum(dim=1) * 2, **tolerance)
    shared = "position += 64" in open(kernel._source).read()
    assert shared == (cols >= 128)

    def row_max_application(input, output):
        output = ntl.max(input)  # noqa: F841

    x[1, cols // 2] = float("nan")
    kernel = ninetoothed.make(row_sum_arrangement, row_max_application, (Tensor(2), Tensor(1)))
    kernel(x, out)
    expected = x.max(dim=1).values
    assert torch.isnan(out[1]) and torch.equal(out[[0] + list(range(2, rows))], expected[[0] + list(range(2, rows))])

    # columns: the outputs are the contiguous ones, a thread each
    def column_arrangement(input, output):
        return input.tile((-1, 1)).squeeze(0), output.tile((1,))

    x = torch.randn(rows, cols, device="cuda").to(dtype)
    column_out = torch.full((cols,), float("nan"), dtype=dtype, device="cuda")
    kernel = ninetoothed.make(column_arrangement, row_sum_application, (Tensor(2), Tensor(1)))
    kernel(x, column_out)
    assert torch.allclose(column_out.float(), x.float().sum(dim=0) * 2, **tolerance)
    assert "position += 64" not in open(kernel._source).read()

    # two reduced dimensions
    def plane_arrangement(input, output):
        return input.tile((1, -1, -1)).squeeze(2).squeeze(1), output.tile((1,))

    planes = torch.randn(9, rows // 8 + 1, 40, device="cuda").to(dtype)
    plane_out = torch.full((9,), float("nan"), dtype=dtype, device="cuda")
    kernel = ninetoothed.make(plane_arrangement, row_sum_application, (Tensor(3), Tensor(1)))
    kernel(planes, plane_out)
    assert torch.allclose(plane_out.float(), planes.float().sum(dim=(1, 2)) * 2, rtol=1e-2 if dtype == torch.float16 else 1e-4, atol=1.0 if dtype == torch.float16 else 1e-2)


# ---- element-wise maps over 16-bit tensors: groups of eight consecutive elements per thread ---------


def _generated_source(kernel, args, kwargs=None):
    """HIP source that launch_nt_map would compile for the kernel's (single) store with these arguments."""
    import ctypes

    from ninetoothed_amd import mapping, runtime
    from ninetoothed_amd.make import _dtype_tag

    env = kernel._environment(args, kwargs or {}, check_device=False)
    (store,) = kernel.program.stores
    program, _, _, _ = mapping.build(store, kernel.types, args, env, lambda p: _dtype_tag(_storage(args, p).dtype), lambda p: 0)
    buffer = ctypes.create_string_buffer(1 << 16)
    assert runtime.library().nt_map_source(ctypes.addressof(program), buffer, len(buffer)) == 0
    return buffer.value.decode()


def test_generated_source_groups_elements_of_16_bit_tensors():
    """Plain element-wise maps whose tensors are contiguous along the last variable read and write 16 bytes of a
    16-bit tensor per access; fp32 tensors alone stay at one element per thread (measured: faster), and so does
    anything whose last extent, padding or strides do not keep a group of eight together."""
    half = lambda *shape: torch.empty(*shape, dtype=torch.float16)  # noqa: E731
    grouped = _generated_source(add_kernel, (half(4096), half(4096), half(4096)), {"BLOCK_SIZE": 1024})
    assert "nt_vec_f16" in grouped and "groups" in grouped
    mixed = _generated_source(add_kernel, (half(4096), torch.empty(4096), torch.empty(4096)), {"BLOCK_SIZE": 1024})
    assert "const nt_vec_f16 loaded" in mixed and "const nt_vec_f32 loaded" in mixed
    assert "nt_vec" not in _generated_source(add_kernel, (torch.empty(4096), torch.empty(4096), torch.empty(4096)), {"BLOCK_SIZE": 1024})
    # (a tile of 12 elements: the last variable's extent is no multiple of 8)
    assert "nt_vec" not in _generated_source(add_kernel, (half(4096), half(4096), half(4096)), {"BLOCK_SIZE": 12})
    # every other element of a wider tensor: the operand does not advance by one element
    assert "nt_vec" not in _generated_source(add_kernel, (half(8192)[::2], half(4096), half(4096)), {"BLOCK_SIZE": 1024})
    # a broadcast operand (one value per row) shares its element within a group
    kernel = ninetoothed.make(_bias_arrangement, _bias_application, (Tensor(2), Tensor(1), Tensor(1), Tensor(2)))
    source = _generated_source(kernel, (half(64, 128), half(128), half(64), half(64, 128)), {name: 32 for name in kernel.meta_symbols})
    assert "nt_vec_f16" in source and "const float shared" in source
    # dropout draws random numbers: groups of four even for fp32 tensors
    dropout = ninetoothed.make(dropout_arrangement, dropout_application, (Tensor(1), Tensor(0), Tensor(0), Tensor(1)))
    assert "nt_vec_f32" in _generated_source(dropout, (torch.empty(4096), 0.3, 7, torch.empty(4096)))
    # tile mode: programs with one reduction, and rows of 16384 elements and more (measured: the others are faster element by element)
    softmax, rms_norm, layer_norm = (kernel for kernel, _, _ in _normalisation_cases("cpu"))
    assert "nt_vec_f16" in _generated_source(rms_norm, (half(64, 4096), half(4096), half(64, 4096)))
    assert "nt_vec" not in _generated_source(rms_norm, (half(64, 4100), half(4100), half(64, 4100)))
    assert "nt_vec" not in _generated_source(rms_norm, (torch.empty(64, 4096), torch.empty(4096), torch.empty(64, 4096)))
    assert "nt_vec" not in _generated_source(softmax, (half(64, 4096), half(64, 4096)))
    assert "nt_vec_f16" in _generated_source(softmax, (half(64, 16384), half(64, 16384)))
    assert "nt_vec_f16" in _generated_source(layer_norm, (half(64, 16384), half(16384), half(64, 16384)))


@gpu
@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
def test_grouped_elements_of_16_bit_tensors(dtype):
    """Results of the grouped kernels against torch: tensors at odd element offsets of sentinel-filled buffers (the
    16-byte accesses are unaligned), a row pitch of its own, a broadcast row and column, an fp32 output, padding."""
    n = 1 << 16
    storage = torch.full((3, n + 9), float("inf"), dtype=dtype, device="cuda")
    lhs, rhs = storage[0, 3 : 3 + n], storage[1, 5 : 5 + n]
    lhs.copy_(torch.randn(n, device="cuda").to(dtype))
    rhs.copy_(torch.randn(n, device="cuda").to(dtype))
    buffer = torch.full((n + 9,), 7.0, dtype=dtype, device="cuda")
    out = buffer[1 : 1 + n]
    add_kernel(lhs, rhs, out, BLOCK_SIZE=1024)
    _served_by_map(add_kernel)
    assert torch.equal(out, lhs + rhs)
    assert float(buffer[0]) == 7.0 and bool((buffer[1 + n :] == 7.0).all())
    wide = torch.empty(n, dtype=torch.float32, device="cuda")
    add_kernel(lhs, rhs, wide, BLOCK_SIZE=1024)
    assert torch.equal(wide, (lhs + rhs).float())  # (the sum is the tiles' type, widened when it is stored)
    kernel = ninetoothed.make(_bias_arrangement, _bias_application, (Tensor(2), Tensor(1), Tensor(1), Tensor(2)))
    x = torch.randn(641, 280 + 8, device="cuda").to(dtype)[:, :280]
    r, c = torch.randn(280, device="cuda").to(dtype), torch.randn(641, device="cuda").to(dtype)
    result = torch.full((641, 280), float("nan"), dtype=dtype, device="cuda")
    kernel(x, r, c, result)
    _served_by_map(kernel)
    # (every operation rounds to the tensors' type, as torch's do)
    assert torch.equal(result, x + r[None, :] + c[:, None] * 2)


@gpu
@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
def test_grouped_elements_in_tile_mode_match_the_interpreter(dtype, monkeypatch):
    """Normalisations over rows of 16-bit tensors whose length is a multiple of 8 keep a thread's elements in groups
    of eight (one 16-byte access per tensor and group): what the interpreter kernel computes element by element, up
    to the order of the row sums (an ulp of the tensors' type), for rows that one wave, 256, 512 and 1024 threads
    share, inputs at odd element offsets."""
    ulp = 2.0**-10 if dtype == torch.float16 else 2.0**-7
    for rows, cols in ((1001, 32), (77, 512), (64, 4096), (33, 8192), (17, 16384), (5, 2056)):
        storage = torch.full((rows, cols + 9), float("inf"), dtype=dtype, device="cuda")
        for kernel, inputs, expected in _normalisation_cases("cuda", dtype, rows, cols):
            shifted = storage[:, 3 : 3 + cols]
            shifted.copy_(inputs[0])
            inputs = (shifted,) + tuple(inputs[1:])
            results = []
            for interpret in ("1", "0"):
                monkeypatch.setenv("NT_MAP_INTERPRET", interpret)
                out = torch.full((rows, cols), float("nan"), dtype=dtype, device="cuda")
                kernel(*inputs, out)
                _served_by_map(kernel)
                results.append(out)
            assert torch.allclose(results[0].float(), results[1].float(), rtol=2 * ulp, atol=2 * ulp), (rows, cols, kernel.kernel_name)
            assert torch.allclose(results[1].float(), expected, rtol=2e-2, atol=2e-2), (rows, cols, kernel.kernel_name)
