"""Host logic: application tracing, program recognition and arrangement
analysis (no GPU needed)."""

import functools

import pytest

import ninetoothed_amd as ninetoothed
import ninetoothed_amd.language as ntl
from ninetoothed_amd import Symbol, Tensor, programs, recognition
from ninetoothed_amd.tracing import trace


def _env(types, shapes, extra=None, strides=None):
    env = dict(extra or {})
    for index, (tensor, shape) in enumerate(zip(types, shapes)):
        if shape is None:
            continue
        source = tensor.source
        layout = strides[index] if strides and strides[index] else None
        if layout is None:
            layout = [1] * len(shape)
            for dim in range(len(shape) - 2, -1, -1):
                layout[dim] = layout[dim + 1] * shape[dim + 1]
        for dim, size in enumerate(shape):
            env[source.size_string(dim)] = size
            env[source.stride_string(dim)] = layout[dim]
    return env


def _metas(kernel):
    return {name: 1 for name in kernel.meta_symbols}


# applications written with other variable names than the built-in programs


def renamed_matmul(input, other, output):
    acc = ntl.zeros(output.shape, dtype=ntl.float32)
    for step in range(input.shape[0]):
        acc += ntl.dot(input[step], other[step])
    output = acc  # noqa: F841


def not_a_known_program(input, other, output):
    acc = ntl.zeros(output.shape, dtype=ntl.float32)
    for step in range(input.shape[0]):
        acc += ntl.dot(input[step], other[step]) * 2
    output = acc  # noqa: F841


def addmm_through_helper(input, mat1, mat2, beta, alpha, output):
    product = ntl.zeros(output.shape, dtype=ntl.float32)
    programs.matmul.application_with_cast(mat1, mat2, product)
    output = beta * input + alpha * product  # noqa: F841


def test_digest_ignores_names_but_not_dataflow():
    types = programs.matmul.arrangement(*programs.matmul.tensors())
    reference = trace(programs.matmul.application, types).digest
    assert trace(renamed_matmul, programs.matmul.arrangement(*programs.matmul.tensors())).digest == reference
    assert trace(not_a_known_program, programs.matmul.arrangement(*programs.matmul.tensors())).digest != reference


def test_make_recognises_the_five_programs():
    kinds = {
        "matmul": ninetoothed.make(programs.matmul.arrangement, renamed_matmul, programs.matmul.tensors()),
        "addmm": ninetoothed.make(programs.addmm.arrangement, addmm_through_helper, programs.addmm.tensors()),
        "softmax": ninetoothed.make(programs.softmax.arrangement, programs.softmax.application, programs.softmax.tensors()),
        "attention": ninetoothed.make(programs.attention.arrangement, programs.attention.application, programs.attention.tensors()),
    }
    for kind, kernel in kinds.items():
        assert kernel.kind == kind
    conv = ninetoothed.make(programs.conv2d.arrangement, programs.conv2d.application, programs.conv2d.tensors())
    assert conv.kind == "matmul"  # conv2d is the matmul application on im2col views
    assert kinds["addmm"].details == {"cast": "fp16"}
    assert "launch" not in (kinds["matmul"].last_plan or "")
    with open(kinds["attention"]._source) as handle:
        assert "attention" in handle.read()


def test_unknown_application_is_reported():
    with pytest.raises(ninetoothed.UnsupportedProgram, match="not one of the programs"):
        ninetoothed.make(programs.matmul.arrangement, not_a_known_program, programs.matmul.tensors())


def test_matmul_analysis_strided_and_ragged():
    kernel = ninetoothed.make(programs.matmul.arrangement, programs.matmul.application, programs.matmul.tensors())
    env = _env(kernel.types, [(300, 100), (100, 200), (300, 200)], _metas(kernel))
    kind, info = recognition.analyze_gemm(*kernel.types, env)
    assert kind == "strided" and (info["m"], info["n"], info["k"]) == (300, 200, 100)
    assert (info["a"].row_stride, info["a"].col_stride) == (100, 1)
    # transposed rhs (column-major) and fixed integer blocks
    arrangement = functools.partial(programs.matmul.arrangement, BLOCK_SIZE_M=64, BLOCK_SIZE_N=32, BLOCK_SIZE_K=16)
    kernel = ninetoothed.make(arrangement, programs.matmul.application, programs.matmul.tensors())
    env = _env(kernel.types, [(300, 100), (100, 200), (300, 200)], strides=[None, [1, 100], None])
    kind, info = recognition.analyze_gemm(*kernel.types, env)
    assert kind == "strided" and (info["b"].row_stride, info["b"].col_stride) == (1, 100)
    assert info["blocks"] == {"m": 64, "n": 32, "k": 16}


def test_batched_matmul_analysis():
    """The matmul application under an arrangement with a leading batch dimension tiled by 1 is the
    batched product: grid (batch, blocks of M, blocks of N), per operand a batch stride."""
    kernel = ninetoothed.make(programs.matmul.batched_arrangement, programs.matmul.application, programs.matmul.batched_tensors())
    assert kernel.kind == "matmul"
    env = _env(kernel.types, [(5, 300, 100), (5, 100, 200), (5, 300, 200)], _metas(kernel))
    kind, info = recognition.analyze_gemm(*kernel.types, env)
    assert kind == "batched" and (info["batch"], info["m"], info["n"], info["k"]) == (5, 300, 200, 100)
    assert (info["a"].batch_stride, info["a"].row_stride, info["a"].col_stride) == (30000, 100, 1)
    assert (info["b"].batch_stride, info["b"].row_stride, info["b"].col_stride) == (20000, 200, 1)
    assert (info["c"].batch_stride, info["c"].row_stride, info["c"].col_stride) == (60000, 200, 1)
    # fixed blocks, a transposed rhs and an lhs that every product shares (batch stride 0, as `expand` gives)
    arrangement = functools.partial(programs.matmul.batched_arrangement, BLOCK_SIZE_M=64, BLOCK_SIZE_N=32, BLOCK_SIZE_K=16)
    kernel = ninetoothed.make(arrangement, programs.matmul.application, programs.matmul.batched_tensors())
    env = _env(kernel.types, [(5, 300, 100), (5, 100, 200), (5, 300, 200)], strides=[[0, 100, 1], [20000, 1, 100], None])
    kind, info = recognition.analyze_gemm(*kernel.types, env)
    assert kind == "batched" and info["blocks"] == {"m": 64, "n": 32, "k": 16}
    assert info["a"].batch_stride == 0 and (info["b"].row_stride, info["b"].col_stride) == (1, 100)
    # operands that disagree on the batch
    env = _env(kernel.types, [(4, 300, 100), (5, 100, 200), (5, 300, 200)])
    with pytest.raises(recognition.UnsupportedProgram):
        recognition.analyze_gemm(*kernel.types, env)


def test_matmul_analysis_rejects_inconsistent_operands():
    kernel = ninetoothed.make(programs.matmul.arrangement, programs.matmul.application, programs.matmul.tensors())
    env = _env(kernel.types, [(64, 32), (48, 64), (64, 64)], _metas(kernel))
    with pytest.raises(ninetoothed.UnsupportedProgram):
        recognition.analyze_gemm(*kernel.types, env)


def test_sliced_operand_becomes_a_base_offset():
    def arrangement(lhs, rhs, output):
        return programs.matmul.arrangement(lhs[2:, 4:], rhs, output)

    kernel = ninetoothed.make(arrangement, programs.matmul.application, programs.matmul.tensors())
    env = _env(kernel.types, [(34, 20), (16, 8), (32, 8)], _metas(kernel))
    kind, info = recognition.analyze_gemm(*kernel.types, env)
    assert kind == "strided" and (info["m"], info["n"], info["k"]) == (32, 8, 16)
    assert info["a"].base == 2 * 20 + 4


@pytest.mark.parametrize("padding", ((0, 0), (1, 1), (0, 1), (2, 0)))
@pytest.mark.parametrize("blocks", (None, 64))
def test_conv2d_analysis(padding, blocks):
    arrangement = programs.conv2d.arrangement
    if blocks:
        arrangement = functools.partial(arrangement, BLOCK_SIZE_M=blocks, BLOCK_SIZE_N=blocks, BLOCK_SIZE_K=blocks)
    kernel = ninetoothed.make(arrangement, programs.conv2d.application, programs.conv2d.tensors())
    n, c, h, w, k, r, s = 4, 64, 16, 16, 512, 3, 3
    p, q = h + 2 * padding[0] - r + 1, w + 2 * padding[1] - s + 1
    env = _env(kernel.types, [(n, c, h, w), (k, c, r, s), (n, k, p, q)], {**_metas(kernel), "padding_h": padding[0], "padding_w": padding[1]})
    kind, info = recognition.analyze_gemm(*kernel.types, env)
    assert kind == "conv2d"
    assert (info["pad_h"], info["pad_w"]) == padding
    assert (info["m"], info["n"], info["k"]) == (n * p * q, k, c * r * s)


@pytest.mark.parametrize("floor_mode", (True, False))
@pytest.mark.parametrize("stride, dilation, padding", (((2, 2), (1, 1), (1, 1)), ((1, 2), (2, 1), (0, 1)), ((3, 1), (1, 2), (2, 2))))
def test_conv2d_analysis_with_stride_and_dilation(stride, dilation, padding, floor_mode):
    """`tile(..., strides=(-1, -1, sh, sw), dilation=(1, 1, dh, dw))` in the conv2d arrangement is recognised, with
    the output size of either rounding (`floor_mode` or the default, which adds a window hanging over the edge)."""
    arrangement = functools.partial(programs.conv2d.arrangement, stride=stride, dilation=dilation, floor_mode=floor_mode)
    kernel = ninetoothed.make(arrangement, programs.conv2d.application, programs.conv2d.tensors())
    n, c, h, w, k, r, s = 2, 8, 17, 14, 16, 3, 3

    def windows(size, pad, taps, spacing, step):
        span = size + 2 * pad - spacing * (taps - 1) - 1
        return span // step + 1 if floor_mode else -(-span // step) + 1

    p, q = windows(h, padding[0], r, dilation[0], stride[0]), windows(w, padding[1], s, dilation[1], stride[1])
    env = _env(kernel.types, [(n, c, h, w), (k, c, r, s), (n, k, p, q)], {**_metas(kernel), "padding_h": padding[0], "padding_w": padding[1]})
    kind, info = recognition.analyze_gemm(*kernel.types, env)
    assert kind == "conv2d"
    assert (info["stride_h"], info["stride_w"], info["dilation_h"], info["dilation_w"]) == (*stride, *dilation)
    assert (info["pad_h"], info["pad_w"]) == padding and (info["m"], info["n"], info["k"]) == (n * p * q, k, c * r * s)
    fits = p == (h + 2 * padding[0] - dilation[0] * (r - 1) - 1) // stride[0] + 1 and q == (w + 2 * padding[1] - dilation[1] * (s - 1) - 1) // stride[1] + 1
    assert info["fits"] == fits
    # an output of another size is not that convolution
    env = _env(kernel.types, [(n, c, h, w), (k, c, r, s), (n, k, p + 1, q)], {**_metas(kernel), "padding_h": padding[0], "padding_w": padding[1]})
    with pytest.raises(ninetoothed.UnsupportedProgram):
        recognition.analyze_gemm(*kernel.types, env)


def test_conv2d_analysis_rejects_wrong_output_shape():
    kernel = ninetoothed.make(programs.conv2d.arrangement, programs.conv2d.application, programs.conv2d.tensors())
    env = _env(kernel.types, [(1, 8, 6, 6), (4, 8, 3, 3), (1, 4, 5, 4)], {**_metas(kernel), "padding_h": 0, "padding_w": 0})
    with pytest.raises(ninetoothed.UnsupportedProgram):
        recognition.analyze_gemm(*kernel.types, env)


def test_softmax_analysis():
    kernel = ninetoothed.make(programs.softmax.arrangement, programs.softmax.application, programs.softmax.tensors())
    kind, info = recognition.analyze_softmax(*kernel.types, _env(kernel.types, [(1823, 781)] * 2, {"BLOCK_SIZE": 781}))
    assert kind == "softmax" and info["input"] == {"rows": 1823, "cols": 781, "block": 781, "row_stride": 781, "col_stride": 1}
    kind, info = recognition.analyze_softmax(*kernel.types, _env(kernel.types, [(8, 100)] * 2, {"BLOCK_SIZE": 32}))
    assert info["output"]["block"] == 32
    kind, _ = recognition.analyze_softmax(*kernel.types, _env(kernel.types, [(0, 16)] * 2, {"BLOCK_SIZE": 16}))
    assert kind == "empty"


def test_softmax_needs_minus_infinity_padding():
    def arrangement(input, output, BLOCK_SIZE=programs.softmax.BLOCK_SIZE):
        return input.tile((1, BLOCK_SIZE)), output.tile((1, BLOCK_SIZE))

    kernel = ninetoothed.make(arrangement, programs.softmax.application, (Tensor(2), Tensor(2)))
    with pytest.raises(ninetoothed.UnsupportedProgram, match="-inf"):
        recognition.analyze_softmax(*kernel.types, _env(kernel.types, [(8, 100)] * 2, {"BLOCK_SIZE": 32}))
    # no padded positions -> the fill value does not matter
    recognition.analyze_softmax(*kernel.types, _env(kernel.types, [(8, 96)] * 2, {"BLOCK_SIZE": 32}))


def test_attention_analysis():
    kernel = ninetoothed.make(programs.attention.arrangement, programs.attention.application, programs.attention.tensors())
    shapes = [(2, 4, 1000, 64)] * 3 + [None, (2, 4, 1000, 64)]
    kind, info = recognition.analyze_attention(kernel.types[0], kernel.types[1], kernel.types[2], kernel.types[4], _env(kernel.types, shapes, _metas(kernel)))
    assert kind == "attention" and info["k"]["shape"] == [2, 4, 1000, 64]
    # different key length, [batch, seq, heads, dim] storage
    shapes = [(2, 4, 10, 64), (2, 4, 77, 64), (2, 4, 77, 64), None, (2, 4, 10, 64)]
    strides = [None, [4 * 77 * 64, 64, 4 * 64, 1], [4 * 77 * 64, 64, 4 * 64, 1], None, None]
    kind, info = recognition.analyze_attention(kernel.types[0], kernel.types[1], kernel.types[2], kernel.types[4], _env(kernel.types, shapes, _metas(kernel), strides))
    assert info["k"]["strides"] == [4 * 77 * 64, 64, 4 * 64, 1]


def test_kernel_call_checks_arguments_before_any_launch():
    import torch

    kernel = ninetoothed.make(programs.softmax.arrangement, programs.softmax.application, programs.softmax.tensors())
    with pytest.raises(TypeError):
        kernel(torch.zeros(2, 2))
    with pytest.raises(RuntimeError, match="no CPU path"):
        kernel(torch.zeros(2, 2), torch.zeros(2, 2), BLOCK_SIZE=2)


def test_equivalent_spellings_of_an_application_share_its_digest():
    """`ntl.dot(a, b, acc)`, positional dtypes / axes and `+=` are spellings, not other programs."""

    def with_accumulator_argument(lhs, rhs, output):
        accumulator = ntl.zeros(output.shape, dtype=ntl.float32)
        for k in range(lhs.shape[0]):
            accumulator = ntl.dot(lhs[k], rhs[k], accumulator)
        output = accumulator  # noqa: F841

    def with_positional_dtype(lhs, rhs, output):
        acc = ntl.zeros(output.shape, ntl.float32)
        for k in range(lhs.shape[0]):
            acc = acc + ntl.dot(lhs[k], rhs[k])
        output = acc  # noqa: F841

    def softmax_with_positional_axis(input, output):
        input_loaded = input
        row_minus_max = input_loaded - ntl.max(input_loaded, None)
        numerator = ntl.exp(row_minus_max)
        denominator = ntl.sum(numerator, None, False)
        output = numerator / denominator  # noqa: F841

    for application in (with_accumulator_argument, with_positional_dtype):
        kernel = ninetoothed.make(programs.matmul.arrangement, application, programs.matmul.tensors())
        assert kernel.kind == "matmul"
    kernel = ninetoothed.make(programs.softmax.arrangement, softmax_with_positional_axis, programs.softmax.tensors())
    assert kernel.kind == "softmax"
